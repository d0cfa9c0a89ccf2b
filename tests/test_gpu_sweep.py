"""Seeded random sweeps of the HIP path against the CPU oracle: attention entry points (decode, paged /
ragged / one-pass prefill, both tree-attention forms) over random head shapes, head dims, page sizes,
batch sizes and sequence lengths on and around the 16 / 32 / 64 / 128 boundaries, with sliding-window
caches, per-layer windows and inline RoPE; the MLA kernel over random page sizes, head counts and
decode- and prefill-shaped batches; and random operation sequences (prefill, decode, mixed steps,
forks inside pages, popn, removal) through the cache object, page tables and cached K/V compared with
the oracle cache after every step.  Every case prints its description before it launches anything."""
import json

import numpy as np
import pytest
import torch

from oracle import kernels as ok
from tests.gpu_util import DEV, dev, host, i32
from tests.util import assert_close, build_paged_kv, random_forest, tree_order
from tvm_amd import kernels as K

pytestmark = pytest.mark.gpu
F16 = np.float16
HEADS = [(32, 8), (8, 8), (16, 1), (64, 8), (12, 1), (24, 2), (40, 8), (8, 2), (4, 4), (6, 2), (20, 1), (64, 1), (32, 1)]
KINDS = ["decode", "paged", "ragged", "tree_paged", "both", "tree_ragged"]


def _lens(rng, b, hi):
    out = []
    for k in rng.integers(0, 6, size=b):
        if k == 0:
            out.append(int(rng.integers(0, 3)))
        elif k == 1:
            out.append(int(rng.choice([15, 16, 17, 31, 32, 33, 63, 64, 65, 127, 128, 129])))
        elif k == 2:
            out.append(int(rng.integers(1, hi)))
        else:
            out.append(int(rng.integers(1, max(2, hi // 8))))
    return out


def _window_spec(rng, kv, q_lens=None, causal=False):
    """Per sequence (physical length, sink size, window offset) of a sliding-window cache."""
    spec = []
    for i, n in enumerate(kv):
        n = max(n, 1)
        off = int(rng.integers(0, n + 1))
        sink = int(rng.integers(0, off + 1)) if off else 0
        if causal:  # the logical length must cover the queries
            while min(sink, off) + n - off < q_lens[i]:
                n += 16
        elif min(sink, off) + n - off == 0:
            off = n - 1
        spec.append((n, min(sink, off), off))
    return spec


def _check(go, gl, eo, el, desc, no_keys=None):
    g_o, g_l = host(go), host(gl)
    if no_keys is not None and no_keys.any():
        assert not g_o[no_keys].any() and np.all(g_l[no_keys] == np.float32(-5e4)), f"rows without keys {desc}"
        g_o, g_l, eo, el = g_o[~no_keys], g_l[~no_keys], eo[~no_keys], el[~no_keys]
    assert_close(g_o, eo, what=f"out {desc}")
    assert_close(g_l, el, atol=3e-3, rtol=1e-4, what=f"lse {desc}")


def _kernel_case(case, padded_d=None):
    """padded_d: a head dim of 80, 96 or 112 -- built for the plain decode, paged and ragged kernels."""
    rng = np.random.default_rng(77000 + case)
    kind = KINDS[case % 6] if padded_d is None else ["decode", "paged", "ragged"][case % 3]
    hq, hkv = HEADS[int(rng.integers(len(HEADS)))]
    d = int(rng.choice([64, 128, 128, 256]))
    ps = int(rng.choice([16, 16, 32, 64, 128]))
    b = int(rng.choice([1, 2, 5, 17, 64, 65, 80])) if kind != "decode" else int(rng.choice([1, 3, 33, 64, 100, 130]))
    if d == 256 or hq >= 16:
        b = min(b, 17)
    sliding = int(rng.integers(2)) if kind in ("decode", "paged") else 0
    rotary = int(rng.integers(2)) if kind in ("decode", "paged", "ragged", "tree_ragged") else 0
    if padded_d is not None:
        d, sliding, rotary = padded_d, 0, 0
    desc = json.dumps(dict(case=case, kind=kind, hq=hq, hkv=hkv, d=d, ps=ps, b=b, sliding=sliding, rotary=rotary))
    print("CASE", desc, flush=True)

    def need(ls):
        return 3 + sum((n + ps - 1) // ps for n in ls)

    def outputs(n):
        return (np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32),
                torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV),
                torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV))

    sm = d ** -0.5
    no_keys = None
    if kind == "decode":
        kv = _lens(rng, b, 2000 if hq <= 16 else 800)
        spec = _window_spec(rng, kv) if sliding else None
        if spec:
            kv = [s[0] for s in spec]
        pages, ip, pv, last, _, _ = build_paged_kv(rng, kv, need(kv), hkv, ps, d)
        info = last if not spec else np.array([last, [s[2] for s in spec], [s[1] for s in spec]], np.int32)
        q = rng.standard_normal((b, hq, d)).astype(F16)
        k_off = rng.integers(0, 300, size=b).astype(np.int32)
        logical = np.array([n if not spec else spec[i][1] + n - spec[i][2] for i, n in enumerate(kv)])
        q_pos = np.maximum(k_off + logical - 1, 0).astype(np.int32)
        eo, el, go, gl = outputs(b)
        ok.decode(q, pages, ip, pv, info, k_off, q_pos, eo, el, rotary, 1.0, 1e4, sm)
        K.batch_decode_paged_kv(dev(q), dev(pages), i32(ip), i32(pv), i32(info), i32(k_off), i32(q_pos), go, gl,
                                rotary, 1.0, 1e4, sm)
    elif kind in ("paged", "both"):
        ql = [max(1, x) for x in _lens(rng, b, 160)]
        kv = _lens(rng, b, 500)
        causal = int(rng.integers(2)) if kind == "paged" else 0
        window = int(rng.choice([0, 0, 5, 40, 300])) if (kind == "paged" and causal and sliding) else 0
        if kind == "paged" and causal:
            kv = [max(k, q_) for k, q_ in zip(kv, ql)]
        spec = _window_spec(rng, kv, ql, bool(causal)) if (sliding and kind == "paged") else None
        if spec:
            kv = [s[0] for s in spec]
        pages, ip, pv, last, _, _ = build_paged_kv(rng, kv, need(kv), hkv, ps, d)
        info = last if spec is None else np.array([last, [s[2] for s in spec], [s[1] for s in spec]], np.int32)
        n = sum(ql)
        ind = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
        q = rng.standard_normal((n, hq, d)).astype(F16)
        eo, el, go, gl = outputs(n)
        if kind == "paged":
            k_off = rng.integers(0, 200, size=b).astype(np.int32)
            logical = [kv[i] if spec is None else spec[i][1] + kv[i] - spec[i][2] for i in range(b)]
            q_pos = np.concatenate([np.maximum(k_off[i] + logical[i] - ql[i] + np.arange(ql[i]), 0)
                                    for i in range(b)]).astype(np.int32)
            print("  ", json.dumps(dict(causal=causal, window=window)), flush=True)
            ok.prefill_paged(q, ind, pages, ip, pv, info, k_off, q_pos, eo, el, causal, rotary, 1.0, 1e4, sm,
                             sliding_window_size=window)
            K.batch_prefill_paged_kv(dev(q), i32(ind), dev(pages), i32(ip), i32(pv), i32(info), i32(k_off), i32(q_pos),
                                     go, gl, causal, rotary, 1.0, 1e4, sm, sliding_window_size=window)
            if causal and window > 0:
                no_keys = np.concatenate([np.arange(n_) >= window - 1 for n_ in ql])
        else:
            k = rng.standard_normal((n, hkv, d)).astype(F16)
            v = rng.standard_normal((n, hkv, d)).astype(F16)
            zq, zb = np.zeros(n, np.int32), np.zeros(b, np.int32)
            to, tl = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
            ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, sm)
            ok.prefill_paged(q, ind, pages, ip, pv, last, zb, zq, to, tl, 0, 0, 1.0, 1e4, sm)
            ok.merge_state_inplace(eo, el, to, tl)
            K.batch_prefill_cached_and_new_kv(dev(q), i32(ind), dev(k), dev(v), dev(pages), i32(ip), i32(pv), i32(last),
                                              go, gl, sm)
    elif kind == "ragged":
        # the oracle's ragged kernel recomputes RoPE per score element: keep those cases short
        ql = [max(1, x) for x in _lens(rng, b, (100 if rotary else 240) // (2 if hq >= 40 else 1))]
        causal = int(rng.integers(2))
        n = sum(ql)
        ind = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
        q = rng.standard_normal((n, hq, d)).astype(F16)
        k = rng.standard_normal((n, hkv, d)).astype(F16)
        v = rng.standard_normal((n, hkv, d)).astype(F16)
        k_off = rng.integers(0, 200, size=b).astype(np.int32)
        q_pos = np.concatenate([k_off[i] + np.arange(ql[i]) for i in range(b)]).astype(np.int32)
        eo, el, go, gl = outputs(n)
        ok.prefill_ragged(q, ind, k, v, ind, q_pos, k_off, eo, el, causal, rotary, 1.0, 1e4, sm)
        K.batch_prefill_ragged_kv(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(q_pos), i32(k_off), go, gl, causal,
                                  rotary, 1.0, 1e4, sm)
    elif kind == "tree_paged":
        b = min(b, 17)
        trees = [random_forest(rng, int(rng.choice([1, 2, 7, 15, 31, 33, 63, 100]))) for _ in range(b)]
        prefix = _lens(rng, b, 700)
        new = [int(rng.integers(1, len(t) + 1)) for t in trees]
        kv = [p_ + len(t) for p_, t in zip(prefix, trees)]
        pages, ip, pv, last, _, _ = build_paged_kv(rng, kv, need(kv), hkv, ps, d)
        ind = np.concatenate([[0], np.cumsum(new)]).astype(np.int32)
        n = int(ind[-1])
        q = rng.standard_normal((n, hq, d)).astype(F16)
        tind = np.concatenate([[0], np.cumsum([len(t) for t in trees])]).astype(np.int32)
        labels = np.concatenate([tree_order(t) for t in trees])
        zb, zq = np.zeros(b, np.int32), np.zeros(n, np.int32)
        eo, el, go, gl = outputs(n)
        ok.tree_attn_paged(q, ind, pages, ip, pv, last, zb, zq, eo, el, 0, 1.0, 1e4, sm, tind, labels)
        K.tree_attn_paged_kv(dev(q), i32(ind), dev(pages), i32(ip), i32(pv), i32(last), i32(zb), i32(zq), go, gl, 0,
                             1.0, 1e4, sm, i32(tind), i32(labels))
    else:
        b = min(b, 17)
        trees = [random_forest(rng, int(rng.choice([1, 2, 7, 15, 31, 33, 63, 64, 65, 100, 200]))) for _ in range(b)]
        sizes = [len(t) for t in trees]
        n = sum(sizes)
        ind = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
        q = rng.standard_normal((n, hq, d)).astype(F16)
        k = rng.standard_normal((n, hkv, d)).astype(F16)
        v = rng.standard_normal((n, hkv, d)).astype(F16)
        mask = np.concatenate([tree_order(t) for t in trees])
        depth = []
        for i, t in enumerate(trees):
            dep = []
            for parent in t:
                dep.append(0 if parent == -1 else dep[parent] + 1)
            depth += [100 * i + x for x in dep]
        q_pos = np.array(depth, np.int32)
        eo, el, go, gl = outputs(n)
        ok.tree_attn_ragged(q, ind, k, v, ind, q_pos, ind, mask, eo, el, rotary, 1.0, 1e4, sm)
        K.batch_tree_attn(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(q_pos), i32(ind), i32(mask), go, gl, rotary,
                          1.0, 1e4, sm)
    _check(go, gl, eo, el, desc, no_keys)


@pytest.mark.parametrize("block", range(10))
def test_random_attention_kernel_cases(block):
    """15 cases per block, 150 in all; the first mismatch fails the block and names its case."""
    for case in range(15 * block, 15 * block + 15):
        _kernel_case(case)


@pytest.mark.parametrize("block", range(2))
def test_random_attention_kernel_cases_with_forced_splits(block):
    """Every paged prefill launch split three ways over its keys and decode chunks of 8 pages: the
    split / merge paths on shapes that would not take them by themselves."""
    import tvm_amd

    prev_splits = tvm_amd.set_option("prefill_kv_splits", 3)
    prev_chunk = tvm_amd.set_option("decode_chunk_pages", 8)
    try:
        for case in range(1000 + 12 * block, 1000 + 12 * block + 12):
            _kernel_case(case)
    finally:
        tvm_amd.set_option("prefill_kv_splits", prev_splits)
        tvm_amd.set_option("decode_chunk_pages", prev_chunk)


@pytest.mark.parametrize("d", [80, 96, 112])
def test_random_attention_kernel_cases_head_dims_80_96_112(d):
    for case in range(2000 + d, 2000 + d + 9):
        _kernel_case(case, padded_d=d)


def _mla_case(case):
    import tests.test_gpu_mla as TM

    rng = np.random.default_rng(88000 + case)
    ps = int(rng.choice([8, 16, 24, 64, 64, 128]))
    heads = int(rng.choice([128, 128, 16, 32, 40, 64, 8]))
    decode = int(rng.integers(2))
    b = int(rng.choice([1, 2, 7, 32, 65, 130])) if decode else int(rng.choice([1, 2, 5, 9]))
    hi = 2500 if decode else 500
    if heads >= 64:
        b, hi = min(b, 16), hi // 3
    kv = []
    for _ in range(b):
        k = int(rng.integers(0, 5))
        kv.append(int(rng.integers(0, 3)) if k == 0 else
                  int(rng.choice([31, 32, 33, 63, 64, 65, 127, 128, 129])) if k == 1 else
                  int(rng.integers(1, hi)) if k == 2 else int(rng.integers(1, max(2, hi // 8))))
    causal = 0 if decode else int(rng.integers(2))
    if decode:
        ql = [1] * b
        if rng.random() < 0.2:
            ql[int(rng.integers(b))] = 2  # not a decode step after all
    else:
        ql = [int(rng.integers(1, 130)) for _ in range(b)]
    if causal:
        kv = [max(k, q_) for k, q_ in zip(kv, ql)]
    desc = json.dumps(dict(case=case, ps=ps, heads=heads, b=b, decode=decode, causal=causal, kv=kv[:12], ql=ql[:12]))
    print("MLA CASE", desc, flush=True)
    npages = 3 + sum((n + ps - 1) // ps for n in kv)
    go, gl, eo, el = TM._mla_both(rng, kv, ql, ps, npages, causal=causal, heads=heads)
    assert_close(go, eo, what=f"mla out {desc}")
    assert_close(gl, el, atol=3e-3, rtol=1e-4, what=f"mla lse {desc}")


@pytest.mark.parametrize("block", range(3))
def test_random_mla_cases(block):
    for case in range(10 * block, 10 * block + 10):
        _mla_case(case)


def _cache_sequence(conf):
    from tests.test_gpu_cache import Mirror

    rng = np.random.default_rng(99000 + conf)
    ps = int(rng.choice([16, 32, 64]))
    hq, hkv = [(32, 8), (8, 2), (8, 8), (16, 1), (12, 4)][int(rng.integers(5))]
    d = int(rng.choice([64, 128, 128, 256]))
    rope_mode = int(rng.choice([0, 1, 1, 2]))
    print("CACHE CONF", json.dumps(dict(conf=conf, ps=ps, hq=hq, hkv=hkv, d=d, rope_mode=rope_mode)), flush=True)
    m = Mirror([16, 8192, 1024, ps, 0], 2, hq, hkv, d, rope_mode=rope_mode)
    m.rng = np.random.default_rng(7 + conf)
    live, children, next_id = [], {}, 0
    for _ in range(20):
        op = rng.choice(["prefill", "decode", "decode", "fork", "popn", "remove", "mixed"])
        if not live or (op == "prefill" and len(live) < 10):
            batch = []
            for _ in range(int(rng.integers(1, 4))):
                batch.append((next_id, int(rng.integers(1, 3 * ps + 6))))
                live.append(next_id)
                children[next_id] = 0
                next_id += 1
            print("  prefill", batch, flush=True)
            m.step(batch)
        elif op in ("decode", "prefill", "mixed"):
            ids = [int(x) for x in rng.permutation(live)[:int(rng.integers(1, len(live) + 1))]]
            ids = [s for s in ids if children[s] == 0 and m.lengths[s] < 400]
            if ids:
                batch = [(s, 1 if op != "mixed" else int(rng.choice([1, 1, 2, 5, ps, ps + 1, 70]))) for s in ids]
                print(" ", op, batch, flush=True)
                m.step(batch)
        elif op == "fork" and len(live) < 14:
            parent = int(rng.choice(live))
            if m.lengths[parent] == 0:
                continue
            pos = int(rng.choice([-1, int(rng.integers(1, m.lengths[parent] + 1))]))
            n = int(rng.choice([1, 3, ps, 40]))
            print("  fork", parent, "->", next_id, "at", pos, "then", n, flush=True)
            m.step([((next_id, parent, pos), n)])
            live.append(next_id)
            children[next_id] = 0
            children[parent] += 1
            next_id += 1
        elif op == "popn":
            cand = [s for s in live if children[s] == 0 and m.lengths[s] > 1]
            if cand:
                s = int(rng.choice(cand))
                n = int(rng.integers(1, m.lengths[s]))
                print("  popn", s, n, flush=True)
                m.o.popn(s, n)
                m.g.popn(s, n)
                m.lengths[s] -= n
        elif op == "remove":
            cand = [s for s in live if children[s] == 0]
            if cand and len(live) > 1:
                s = int(rng.choice(cand))
                print("  remove", s, flush=True)
                m.o.remove_sequence(s)
                m.g.remove_sequence(s)
                live.remove(s)


@pytest.mark.parametrize("block", range(3))
def test_random_cache_operation_sequences(block):
    for conf in range(10 * block, 10 * block + 10):
        _cache_sequence(conf)
