"""The HIP kernels at the full sizes of the benchmark configurations, checked through properties
that do not need the (serial, minutes-long) CPU oracle on the whole input, plus the oracle on a
few sequences cut out of the batch:

* a value tensor that is constant per feature must come back as that constant (softmax weights
  sum to one; the reference's phantom denominator term 2^(-5e4 - m) is 0 in fp32 here),
* split-KV results must not depend on the chunk size, nor on where the pages of a sequence lie in the pool,
* lse of a sequence = log2 sum 2^(score), checked with a float64 torch computation per sequence,
* single sequences of the batch against the oracle.
"""
import os

import numpy as np
import pytest
import torch

import bench
import tvm_amd
from oracle import kernels as ok
from tests.gpu_util import DEV, host, i32
from tests.util import assert_close
from tvm_amd import kernels as K

pytestmark = pytest.mark.gpu
F16 = torch.float16


def _decode_inputs(batch, ctx_lo, ctx_hi, hq, seed, pool_pages):
    wl = bench.decode_workload(batch=batch, ctx_lo=ctx_lo, ctx_hi=ctx_hi, pool_pages=pool_pages, steps=1, seed=seed)
    t = wl["tables"][0]
    gen = torch.Generator(device=DEV)
    gen.manual_seed(seed)
    pages = torch.empty((pool_pages, 2, 8, 16, 128), dtype=F16, device=DEV)
    for lo in range(0, pool_pages, 8192):
        pages[lo:lo + 8192].copy_(torch.randn(pages[lo:lo + 8192].shape, generator=gen, device=DEV))
    q = torch.randn((batch, hq, 128), generator=gen, device=DEV).to(F16)
    return t, pages, q


def _decode(q, pages, t):
    b, hq, d = q.shape
    out = torch.empty_like(q)
    lse = torch.empty((b, hq), dtype=torch.float32, device=DEV)
    z = torch.zeros(b, dtype=torch.int32, device=DEV)
    K.batch_decode_paged_kv(q, pages, i32(t["page_indptr"]), i32(t["page_values"]), i32(t["last_page_len"]), z, z, out,
                            lse, 0, 1.0, 1e4, d ** -0.5)
    return out, lse


def _oracle_one_sequence(q, pages, t, b):
    lo, hi = int(t["page_indptr"][b]), int(t["page_indptr"][b + 1])
    ids = torch.tensor(t["page_values"][lo:hi], dtype=torch.int64, device=DEV)
    hp = host(pages[ids])
    hq = q.shape[1]
    eo = np.zeros((1, hq, 128), np.float16)
    el = np.zeros((1, hq), np.float32)
    z = np.zeros(1, np.int32)
    ok.decode(host(q[b:b + 1]), hp, np.array([0, hi - lo], np.int32), np.arange(hi - lo, dtype=np.int32),
              t["last_page_len"][b:b + 1], z, z, eo, el, 0, 1.0, 1e4, 128 ** -0.5)
    return eo[0], el[0]


@pytest.mark.parametrize("name,batch,lo,hi,hq,pool", [("configs[1]", 64, 1024, 8192, 32, 65536),
                                                       ("configs[3]", 8, 32768, 131072, 64, 65536)])
def test_decode_full_size_properties(name, batch, lo, hi, hq, pool):
    t, pages, q = _decode_inputs(batch, lo, hi, hq, seed=1 if batch == 64 else 3, pool_pages=pool)
    out, lse = _decode(q, pages, t)
    # the shortest and the longest sequence against the oracle
    lens = t["kv_len"]
    for b in (int(np.argmin(lens)), int(np.argmax(lens))) if batch == 64 else (int(np.argmin(lens)),):
        eo, el = _oracle_one_sequence(q, pages, t, b)
        assert_close(host(out[b]), eo, what=f"{name} seq {b} out")
        assert_close(host(lse[b]), el, atol=2e-3, rtol=1e-4, what=f"{name} seq {b} lse")
    # chunk-size independence of the split-KV path
    prev = tvm_amd.set_option("decode_chunk_pages", 8)
    try:
        out8, lse8 = _decode(q, pages, t)
        tvm_amd.set_option("decode_chunk_pages", 128)
        out128, lse128 = _decode(q, pages, t)
    finally:
        tvm_amd.set_option("decode_chunk_pages", prev)
    assert_close(host(out8), host(out128), atol=2e-3, rtol=2e-3, what=f"{name} chunk 8 vs 128")
    assert_close(host(lse8), host(lse128), atol=1e-3, rtol=1e-5, what=f"{name} lse chunk 8 vs 128")
    assert_close(host(out), host(out128), atol=2e-3, rtol=2e-3, what=f"{name} default chunk vs 128")
    # the same rows at consecutive page ids, the order in which a freshly filled cache hands pages out:
    # bit-identical (the page table is the only thing that knows where a page lies)
    ids = torch.tensor(np.asarray(t["page_values"]), dtype=torch.int64, device=DEV)
    packed = pages.index_select(0, ids)
    t_packed = dict(t, page_values=np.arange(ids.numel(), dtype=np.int32))
    out_p, lse_p = _decode(q, packed, t_packed)
    assert torch.equal(out_p, out) and torch.equal(lse_p, lse), f"{name}: result depends on where the pages lie"
    del packed
    # the chunk merge done by the last workgroup of each (sequence, kv head) against the same
    # arithmetic in a second kernel: bit-identical, every time (a stale read of another
    # workgroup's partial state would show here)
    prev = tvm_amd.set_option("decode_separate_merge", 1)
    try:
        out_sep, lse_sep = _decode(q, pages, t)
    finally:
        tvm_amd.set_option("decode_separate_merge", prev)
    for _ in range(20):
        out_f, lse_f = _decode(q, pages, t)
        assert torch.equal(out_f, out_sep) and torch.equal(lse_f, lse_sep), f"{name}: fused merge differs"
    # constant values come back unchanged
    feat = (torch.arange(128, device=DEV, dtype=torch.float32) / 64 - 1).to(F16)
    pages[:, 1] = feat
    outc, lsec = _decode(q, pages, t)
    assert torch.equal(lsec, lse), "lse must not depend on the values"
    assert_close(host(outc), np.broadcast_to(host(feat), outc.shape), atol=1e-3, rtol=1e-3, what=f"{name} constant V")


def test_chunked_prefill_full_size_properties():
    """configs[2]: ragged causal + paged non-causal + merge on 9842 new tokens."""
    pw = bench.prefill_workload()
    n = int(pw["q_indptr"][-1])
    hq, hkv, d, ps = bench.HQ, bench.HKV, bench.D, bench.PS
    gen = torch.Generator(device=DEV)
    gen.manual_seed(2)
    pages = torch.randn((pw["pool_pages"], 2, hkv, ps, d), generator=gen, device=DEV).to(F16)
    q = torch.randn((n, hq, d), generator=gen, device=DEV).to(F16)
    k = torch.randn((n, hkv, d), generator=gen, device=DEV).to(F16)
    v = torch.randn((n, hkv, d), generator=gen, device=DEV).to(F16)
    qi, pi = i32(pw["q_indptr"]), i32(pw["page_indptr"])
    pv, last = i32(pw["page_values"]), i32(pw["last_page_len"])
    nb = len(pw["chunk"])
    z, zn = torch.zeros(nb, dtype=torch.int32, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV)
    sm = d ** -0.5

    def run(pages_, v_):
        o1 = torch.empty((n, hq, d), dtype=F16, device=DEV)
        o2 = torch.empty_like(o1)
        l1 = torch.empty((n, hq), dtype=torch.float32, device=DEV)
        l2 = torch.empty_like(l1)
        K.batch_prefill_ragged_kv(q, qi, k, v_, qi, zn, z, o1, l1, 1, 0, 1.0, 1e4, sm)
        K.batch_prefill_paged_kv(q, qi, pages_, pi, pv, last, z, zn, o2, l2, 0, 0, 1.0, 1e4, sm)
        K.merge_state_inplace(o1, l1, o2, l2)
        return o1, l1

    out, lse = run(pages, v)
    # one short sequence against the oracle: self (causal) + prefix (all visible) + merge
    b = int(np.argmin(pw["chunk"] * (pw["chunk"] + pw["prefix"])))
    s, e = int(pw["q_indptr"][b]), int(pw["q_indptr"][b + 1])
    lo, hi = int(pw["page_indptr"][b]), int(pw["page_indptr"][b + 1])
    c = e - s
    hp = host(pages[torch.tensor(pw["page_values"][lo:hi], dtype=torch.int64, device=DEV)]) if hi > lo else \
        np.zeros((1, 2, hkv, ps, d), np.float16)
    eo1, el1 = np.zeros((c, hq, d), np.float16), np.zeros((c, hq), np.float32)
    eo2, el2 = np.zeros_like(eo1), np.zeros_like(el1)
    ind = np.array([0, c], np.int32)
    z1, zc = np.zeros(1, np.int32), np.zeros(c, np.int32)
    ok.prefill_ragged(host(q[s:e]), ind, host(k[s:e]), host(v[s:e]), ind, zc, z1, eo1, el1, 1, 0, 1.0, 1e4, sm)
    ok.prefill_paged(host(q[s:e]), ind, hp, np.array([0, hi - lo], np.int32), np.arange(hi - lo, dtype=np.int32),
                     pw["last_page_len"][b:b + 1], z1, zc, eo2, el2, 0, 0, 1.0, 1e4, sm)
    ok.merge_state_inplace(eo1, el1, eo2, el2)
    assert_close(host(out[s:e]), eo1, what=f"configs[2] seq {b} out")
    assert_close(host(lse[s:e]), el1, atol=2e-3, rtol=1e-4, what=f"configs[2] seq {b} lse")
    # constant values (new tokens and cached prefix alike) come back unchanged, lse does not move
    feat = (torch.arange(d, device=DEV, dtype=torch.float32) / 64 - 1).to(F16)
    pages_c = pages.clone()
    pages_c[:, 1] = feat
    outc, lsec = run(pages_c, feat.expand(n, hkv, d).contiguous())
    assert torch.equal(lsec, lse)
    assert_close(host(outc), np.broadcast_to(host(feat), outc.shape), atol=2e-3, rtol=2e-3, what="configs[2] constant V")


def test_chunked_prefill_step_of_the_benchmark_full_size():
    """configs[2] through exactly the two launches bench.py times (split + RoPE + append, then the
    one-pass kernel over cached prefix and new chunk): against the three-kernel composition of the
    reference (ragged causal + paged + merge) on every row, against the oracle on the cheapest
    sequence (from the raw qkv: RoPE, self, cross, merge), the appended page slots bit for bit, and
    constant values in, constant values out."""
    pw = bench.prefill_workload()
    gen = torch.Generator(device=DEV)
    gen.manual_seed(1)
    step, t = bench.make_prefill_step(torch, K, pw, gen, DEV)
    hq, hkv, d, ps = bench.HQ, bench.HKV, bench.D, bench.PS
    n = int(pw["q_indptr"][-1])
    nb = len(pw["chunk"])
    sm = d ** -0.5
    pages_before = t["pages"].clone()
    step(0)
    out, lse = t["out"].clone(), t["lse"].clone()
    # the step rotates q inside the attention kernel; the separate kernel gives the rows for the comparison
    K.fused_rope(t["qkv"], t["q_rope_position"], t["q"], torch.empty_like(t["k"]), torch.empty_like(t["v"]), 1)
    # (1) the reference's composition on the same rotated q / k / v
    z, zn = torch.zeros(nb, dtype=torch.int32, device=DEV), torch.zeros(n, dtype=torch.int32, device=DEV)
    o1, o2 = torch.empty_like(out), torch.empty_like(out)
    l1, l2 = torch.empty_like(lse), torch.empty_like(lse)
    K.batch_prefill_ragged_kv(t["q"], t["q_indptr"], t["k"], t["v"], t["q_indptr"], zn, z, o1, l1, 1, 0, 1.0, 1e4, sm)
    K.batch_prefill_paged_kv(t["q"], t["q_indptr"], t["pages"], t["page_indptr"], t["page_values"], t["last_page_len"],
                             z, zn, o2, l2, 0, 0, 1.0, 1e4, sm)
    K.merge_state_inplace(o1, l1, o2, l2)
    assert_close(host(out), host(o1), atol=2e-3, rtol=2e-3, what="one pass vs ragged + paged + merge, out")
    assert_close(host(lse), host(l1), atol=1e-3, rtol=1e-5, what="one pass vs ragged + paged + merge, lse")
    # (2) the cheapest sequence from the raw inputs through the oracle
    b = int(np.argmin(pw["chunk"] * (pw["chunk"] + pw["prefix"])))
    s, e = int(pw["q_indptr"][b]), int(pw["q_indptr"][b + 1])
    lo, hi = int(pw["page_indptr"][b]), int(pw["page_indptr"][b + 1])
    c = e - s
    pos = np.arange(c, dtype=np.int32) + int(pw["prefix"][b])
    qh, kh, vh = np.zeros((c, hq, d), np.float16), np.zeros((c, hkv, d), np.float16), np.zeros((c, hkv, d), np.float16)
    ok.fused_rope(host(t["qkv"][s:e]), pos, qh, kh, vh, 1)
    hp = host(pages_before[torch.tensor(pw["page_values"][lo:hi], dtype=torch.int64, device=DEV)]) if hi > lo else \
        np.zeros((1, 2, hkv, ps, d), np.float16)
    eo1, el1 = np.zeros((c, hq, d), np.float16), np.zeros((c, hq), np.float32)
    eo2, el2 = np.zeros_like(eo1), np.zeros_like(el1)
    ind = np.array([0, c], np.int32)
    z1, zc = np.zeros(1, np.int32), np.zeros(c, np.int32)
    ok.prefill_ragged(qh, ind, kh, vh, ind, zc, z1, eo1, el1, 1, 0, 1.0, 1e4, sm)
    if hi > lo:
        ok.prefill_paged(qh, ind, hp, np.array([0, hi - lo], np.int32), np.arange(hi - lo, dtype=np.int32),
                         pw["last_page_len"][b:b + 1], z1, zc, eo2, el2, 0, 0, 1.0, 1e4, sm)
        ok.merge_state_inplace(eo1, el1, eo2, el2)
    assert_close(host(out[s:e]), eo1, what=f"configs[2] one pass, seq {b} out vs oracle")
    assert_close(host(lse[s:e]), el1, atol=2e-3, rtol=1e-4, what=f"configs[2] one pass, seq {b} lse vs oracle")
    # (3) the appended slots hold the rotated k and the v rows, every other slot is untouched
    slots = torch.tensor(pw["append_position_map"], dtype=torch.int64, device=DEV)
    flat = t["pages"].permute(0, 3, 1, 2, 4).reshape(-1, 2, hkv, d)  # (slot, k|v, head, d)
    assert torch.equal(flat[slots, 0], t["k"]) and torch.equal(flat[slots, 1], t["v"])
    untouched = torch.ones(flat.shape[0], dtype=torch.bool, device=DEV)
    untouched[slots] = False
    flat_before = pages_before.permute(0, 3, 1, 2, 4).reshape(-1, 2, hkv, d)
    assert torch.equal(flat[untouched], flat_before[untouched])
    # (4) constant values (cached prefix and new tokens alike) come back unchanged; lse does not move
    feat = (torch.arange(d, device=DEV, dtype=torch.float32) / 64 - 1).to(F16)
    t["pages"][:, 1] = feat
    t["qkv"][:, hq + hkv:] = feat
    step(0)
    assert_close(host(t["lse"]), host(lse), atol=1e-4, rtol=1e-6, what="lse must not depend on the values")
    assert_close(host(t["out"]), np.broadcast_to(host(feat), t["out"].shape), atol=2e-3, rtol=2e-3,
                 what="configs[2] one pass, constant V")


def test_mla_full_size_properties():
    """configs[4]: decode batch 32 (split-KV route) and a 1024-token chunk on a 2048-token prefix."""
    hq, dl, dr, ps = 128, 512, 64, 64
    sm = 192 ** -0.5
    rng = np.random.default_rng(4)
    for name, prefix, chunk, causal in (("decode", rng.integers(2048, 8192, size=32, endpoint=True) - 1,
                                         np.ones(32, dtype=np.int64), 0),
                                        ("prefill", np.full(4, 2048), np.full(4, 1024), 1)):
        kv = prefix + chunk
        npg = (kv + ps - 1) // ps
        pool = int(npg.sum()) + 8
        perm = rng.permutation(pool).astype(np.int32)
        pg = (torch.randn((pool, ps, dl + dr), device=DEV) * 0.5).to(F16)
        ip = np.concatenate([[0], np.cumsum(npg)])
        qi = np.concatenate([[0], np.cumsum(chunk)])
        n = int(qi[-1])
        q = (torch.randn((n, hq, dl + dr), device=DEV) * 0.5).to(F16)
        last = ((kv - 1) % ps + 1).astype(np.int32)

        def run(pages_):
            o = torch.empty((n, hq, dl), dtype=F16, device=DEV)
            lse = torch.empty((n, hq), dtype=torch.float32, device=DEV)
            K.batch_prefill_paged_kv_mla(q, i32(qi), pages_, i32(ip), i32(perm[:ip[-1]]), i32(last), o, lse, causal, sm)
            return o, lse

        out, lse = run(pg)
        # the first query token of the shortest sequence against the oracle (one row tile of 128 heads)
        b = int(np.argmin(kv))
        ids = torch.tensor(perm[ip[b]:ip[b + 1]], dtype=torch.int64, device=DEV)
        t0 = int(qi[b])
        kv_seen = int(kv[b] - chunk[b] + 1) if causal else int(kv[b])
        npages_seen = (kv_seen + ps - 1) // ps
        eo, el = np.zeros((1, hq, dl), np.float16), np.zeros((1, hq), np.float32)
        ok.prefill_paged_mla(host(q[t0:t0 + 1]), np.array([0, 1], np.int32), host(pg[ids[:npages_seen]]),
                             np.array([0, npages_seen], np.int32), np.arange(npages_seen, dtype=np.int32),
                             np.array([(kv_seen - 1) % ps + 1], np.int32), eo, el, 0, sm, d_latent=dl)
        assert_close(host(out[t0]), eo[0], what=f"mla {name} seq {b} out")
        assert_close(host(lse[t0]), el[0], atol=2e-3, rtol=1e-4, what=f"mla {name} seq {b} lse")
        # a latent part that is constant per feature comes back unchanged; the rope part keeps the scores apart
        feat = (torch.arange(dl, device=DEV, dtype=torch.float32) / 256 - 1).to(F16)
        pgc = pg.clone()
        pgc[:, :, :dl] = feat
        qc = q.clone()
        qc[:, :, :dl] = 0  # scores then come from the rope part alone and are the same in both runs
        q_saved, q = q, qc
        out0, lse0 = run(pg)
        outc, lsec = run(pgc)
        q = q_saved
        assert torch.equal(lsec, lse0)
        assert_close(host(outc), np.broadcast_to(host(feat), outc.shape), atol=2e-3, rtol=2e-3,
                     what=f"mla {name} constant latent")
