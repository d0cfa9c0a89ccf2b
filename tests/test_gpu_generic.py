"""The generic matrix-core kernels on the GPU: float32 storage (through the tensor-level boundary, where the
dtype travels in the tensor), and fp16 with pages and head dims the tuned kernels are not built for (through
the pointer-level launchers, which hand such shapes over).  Checked against the CPU oracle built for the same
storage type; with float32 storage the tolerance is that of float32 sums in a different order."""
import numpy as np
import pytest
import torch

from oracle import kernels as ok
from tests.gpu_util import DEV, dev, host, i32
from tests.util import REFERENCE_TREES, assert_close, build_paged_kv, random_forest, tree_order
from tvm_amd import KVError
from tvm_amd import dlpack as dl
from tvm_amd import kernels as K

pytestmark = pytest.mark.gpu
F16, F32 = np.float16, np.float32


def T(a):
    """A numpy array as a device tensor and its DLTensor."""
    t = dev(a)
    return t, dl.tensor(t)


def TI(a):
    t = i32(a)
    return dl.tensor(t)


def tol(dtype):
    return dict(atol=2e-4, rtol=2e-4) if dtype == F32 else dict(atol=1e-2, rtol=1e-2)


def paged_case(rng, kv_lens, q_lens, hq, hkv, d, ps, dtype):
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, kv_lens, 4 + sum((n + ps - 1) // ps for n in kv_lens), hkv, ps, d,
                                                       dtype=dtype)
    n = sum(q_lens)
    qindptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(dtype)
    return pages, indptr, values, last, qindptr, q


@pytest.mark.parametrize("hq,hkv,d,ps", [(32, 8, 128, 16), (8, 2, 64, 16), (8, 8, 128, 32), (6, 2, 72, 12), (16, 1, 256, 16),
                                         (40, 2, 128, 16)])
def test_float32_decode_and_paged_prefill(hq, hkv, d, ps):
    rng = np.random.default_rng(300)
    kv_lens = [0, 1, 15, 16, 17, 300, 1000, 64, 2500]
    b = len(kv_lens)
    pages, indptr, values, last, _, _ = paged_case(rng, kv_lens, [1] * b, hq, hkv, d, ps, F32)
    z = np.zeros(b, np.int32)
    q = rng.standard_normal((b, hq, d)).astype(F32)
    eo, el = np.zeros((b, hq, d), F32), np.zeros((b, hq), F32)
    ok.decode(q, pages, indptr, values, last, z, z, eo, el, 0, 1.0, 1e4, d ** -0.5)
    _, pages_dl = T(pages)
    keep = pages_dl
    out, out_dl = T(np.full((b, hq, d), 7.0, F32))
    lse, lse_dl = T(np.full((b, hq), 7.0, F32))
    dl.call("batch_decode_paged_kv", T(q)[1], pages_dl, TI(indptr), TI(values), TI(last), TI(z), TI(z), out_dl, lse_dl, 0, 1.0,
            1e4, d ** -0.5)
    assert_close(host(out), eo, what="f32 decode out", **tol(F32))
    assert_close(host(lse), el, atol=2e-4, rtol=1e-5, what="f32 decode lse")
    q_lens = [3, 1, 2, 16, 5, 64, 130, 2, 40]
    for causal in (0, 1):
        lens = [max(k, ql) for k, ql in zip(kv_lens, q_lens)] if causal else kv_lens
        pages, indptr, values, last, qindptr, q = paged_case(rng, lens, q_lens, hq, hkv, d, ps, F32)
        n = len(q)
        eo, el = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
        ok.prefill_paged(q, qindptr, pages, indptr, values, last, z, np.zeros(n, np.int32), eo, el, causal, 0, 1.0, 1e4, d ** -0.5)
        out, out_dl = T(np.full((n, hq, d), 7.0, F32))
        lse, lse_dl = T(np.full((n, hq), 7.0, F32))
        dl.call("batch_prefill_paged_kv", T(q)[1], TI(qindptr), T(pages)[1], TI(indptr), TI(values), TI(last), TI(z),
                TI(np.zeros(n, np.int32)), out_dl, lse_dl, causal, 0, 1.0, 1e4, d ** -0.5, 0)
        # a sequence without keys: out 0 and lse -5e4, as the reference's kernels leave their initial state
        assert_close(host(out), eo, what=f"f32 paged prefill out, causal {causal}", **tol(F32))
        assert_close(host(lse), el, atol=2e-4, rtol=1e-5, what=f"f32 paged prefill lse, causal {causal}")
    del keep


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (4, 4, 100)])
def test_float32_ragged_tree_merge_and_rope(hq, hkv, d):
    rng = np.random.default_rng(301)
    lens = [300, 5, 1, 200, 33]
    n = sum(lens)
    ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F32) for h in (hq, hkv, hkv))
    zq, zb = np.zeros(n, np.int32), np.zeros(len(lens), np.int32)
    for causal in (1, 0):
        eo, el = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
        ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, causal, 0, 1.0, 1e4, d ** -0.5)
        out, out_dl = T(np.full((n, hq, d), 7.0, F32))
        lse, lse_dl = T(np.full((n, hq), 7.0, F32))
        dl.call("batch_prefill_ragged_kv", T(q)[1], TI(ind), T(k)[1], T(v)[1], TI(ind), TI(zq), TI(zb), out_dl, lse_dl, causal, 0,
                1.0, 1e4, d ** -0.5)
        assert_close(host(out), eo, what=f"f32 ragged out, causal {causal}", **tol(F32))
        assert_close(host(lse), el, atol=2e-4, rtol=1e-5, what="f32 ragged lse")
    # merge_state_inplace on the two states of a split key axis = attention over all keys (here: just the arithmetic)
    v1, v2 = (rng.standard_normal((7, hq, d)).astype(F32) for _ in range(2))
    s1, s2 = ((rng.standard_normal((7, hq)) * 3).astype(F32) for _ in range(2))
    s2[0] = -5e4
    ev, es = v1.copy(), s1.copy()
    ok.merge_state_inplace(ev, es, v2, s2)
    gv, gv_dl = T(v1)
    gs, gs_dl = T(s1)
    dl.call("merge_state_inplace", gv_dl, gs_dl, T(v2)[1], T(s2)[1])
    assert_close(host(gv), ev, atol=1e-5, rtol=1e-5, what="f32 merge v")
    assert_close(host(gs), es, atol=1e-5, rtol=1e-6, what="f32 merge s")
    # token trees (ragged)
    trees = REFERENCE_TREES + [random_forest(rng, 70)]
    tl = [len(t) for t in trees]
    n = sum(tl)
    ind = np.concatenate([[0], np.cumsum(tl)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F32) for h in (hq, hkv, hkv))
    mask = np.concatenate([tree_order(t) for t in trees]).astype(np.int32)
    eo, el = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
    ok.tree_attn_ragged(q, ind, k, v, ind, np.zeros(n, np.int32), ind, mask, eo, el, 0, 1.0, 1e4, d ** -0.5)
    out, out_dl = T(np.full((n, hq, d), 7.0, F32))
    lse, lse_dl = T(np.full((n, hq), 7.0, F32))
    dl.call("batch_tree_attn", T(q)[1], TI(ind), T(k)[1], T(v)[1], TI(ind), TI(np.zeros(n, np.int32)), TI(ind),
            TI(mask.reshape(-1)), out_dl, lse_dl, 0, 1.0, 1e4, d ** -0.5)
    assert_close(host(out), eo, what="f32 tree out", **tol(F32))
    assert_close(host(lse), el, atol=2e-4, rtol=1e-5, what="f32 tree lse")
    # split + RoPE (slot 24) and append / gather (slots 13, 26)
    if d % 2 == 0:
        pos = np.array([0, 1, 2, 3, 100, 511, 2047, 4095, 7, 9, 33], np.int32)
        n = len(pos)
        qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F32)
        eq, ek, ev = np.zeros((n, hq, d), F32), np.zeros((n, hkv, d), F32), np.zeros((n, hkv, d), F32)
        ok.fused_rope(qkv, pos, eq, ek, ev, 1)
        gq, gq_dl = T(np.zeros_like(eq))
        gk, gk_dl = T(np.zeros_like(ek))
        gv, gv_dl = T(np.zeros_like(ev))
        dl.call("fused_rope", T(qkv)[1], TI(pos), gq_dl, gk_dl, gv_dl, 1, None, None, 1.0, 1e4)
        assert np.array_equal(host(gv), ev)
        # device sin / cos against libm at angles up to 4095 rad: a few float32 ulps of the angle's sine
        assert_close(host(gq), eq, atol=2e-5, rtol=1e-5, what="f32 rope q")
        assert_close(host(gk), ek, atol=2e-5, rtol=1e-5, what="f32 rope k")


def test_float32_page_slots_bit_exact():
    rng = np.random.default_rng(302)
    hkv, d, ps, npages = 2, 128, 16, 12
    pages = rng.standard_normal((npages, 2, hkv, ps, d)).astype(F32)
    n = 9
    k, v = (rng.standard_normal((n, hkv, d)).astype(F32) for _ in range(2))
    pos = np.array([0, 17, -1, 33, 34, 35, 191, 100, -1], np.int32)
    expect = pages.copy()
    ok.transpose_append(expect, k, v, pos)
    pt, pages_dl = T(pages)
    dl.call("transpose_append", pages_dl, T(k)[1], T(v)[1], TI(pos))
    assert np.array_equal(host(pt), expect)
    ok.copy_single_page(expect, 2, 7, 5)
    dl.call("copy_single_page", pages_dl, 2, 7, 5)
    assert np.array_equal(host(pt), expect)
    copy_indptr = np.array([0, 2, 2, 5], np.int32)
    src_dst = np.array([[33, 35, 100, 17, 191], [32, 33, 96, 97, 98]], np.int32)
    ok.compact_kv_copy(expect, copy_indptr, src_dst, 3)
    dl.call("compact_kv_copy", pages_dl, TI(copy_indptr), TI(src_dst), 3)
    assert np.array_equal(host(pt), expect)
    gather = np.array([32, 33, 96, 97, 98, 0, 17], np.int32)
    ek, ev = np.zeros((3, len(gather), hkv, d), F32), np.zeros((3, len(gather), hkv, d), F32)
    ok.debug_get_kv(expect, gather, ek, ev, 1)
    gk, gk_dl = T(np.zeros_like(ek))
    gv, gv_dl = T(np.zeros_like(ev))
    dl.call("debug_get_kv", pages_dl, TI(gather), gk_dl, gv_dl, 1)
    assert np.array_equal(host(gk), ek) and np.array_equal(host(gv), ev)


def test_float32_tree_attention_over_pages_and_refusals():
    from oracle import closed_form as cf
    rng = np.random.default_rng(303)
    hq, hkv, d, ps = 8, 2, 128, 16
    prefix = [10, 0, 129, 700]
    trees = [REFERENCE_TREES[0], REFERENCE_TREES[3], random_forest(rng, 31), random_forest(rng, 63)]
    new_lens = [7, 14, 16, 63]
    kv_lens = [p + len(t) for p, t in zip(prefix, trees)]
    pages, pindptr, pvalues, last, _, _ = build_paged_kv(rng, kv_lens, 80, hkv, ps, d, dtype=F32)
    qindptr = np.concatenate([[0], np.cumsum(new_lens)]).astype(np.int32)
    q = rng.standard_normal((int(qindptr[-1]), hq, d)).astype(F32)
    tindptr = np.concatenate([[0], np.cumsum([len(t) for t in trees])]).astype(np.int32)
    labels = np.concatenate([tree_order(t) for t in trees]).astype(np.int32)
    n = len(q)
    zb, zq = np.zeros(len(trees), np.int32), np.zeros(n, np.int32)
    eo, el = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
    ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, eo, el, 0, 1.0, 1e4, d ** -0.5, tindptr, labels)
    out, out_dl = T(np.full((n, hq, d), 7.0, F32))
    lse, lse_dl = T(np.full((n, hq), 7.0, F32))
    _, pages_dl = T(pages)
    dl.call("tree_attn_paged_kv", T(q)[1], TI(qindptr), pages_dl, TI(pindptr), TI(pvalues), TI(last), TI(zb), TI(zq), out_dl, lse_dl,
            0, 1.0, 1e4, d ** -0.5, TI(tindptr), TI(labels.reshape(-1)))
    assert_close(host(out), eo, what="f32 tree paged out", **tol(F32))
    assert_close(host(lse), el, atol=2e-4, rtol=1e-5, what="f32 tree paged lse")
    # RoPE inside the kernel over a token tree in the page pool is not built (the reference's kernel asserts the same)
    with pytest.raises(KVError, match="token trees over the page pool"):
        dl.call("tree_attn_paged_kv", T(q)[1], TI(qindptr), pages_dl, TI(pindptr), TI(pvalues), TI(last), TI(zb), TI(zq), out_dl,
                lse_dl, 1, 1.0, 1e4, d ** -0.5, TI(tindptr), TI(labels.reshape(-1)))
    with pytest.raises(KVError, match="float16"):   # mixed storage types in one call
        dl.call("batch_prefill_paged_kv", T(q.astype(F16))[1], TI(qindptr), pages_dl, TI(pindptr), TI(pvalues), TI(last), TI(zb),
                TI(zq), out_dl, lse_dl, 0, 0, 1.0, 1e4, d ** -0.5, 0)


@pytest.mark.parametrize("hq,hkv,d,ps", [(8, 2, 128, 16), (8, 4, 72, 12)])
def test_float32_sliding_window_cache_window_mask_and_inline_rope(hq, hkv, d, ps):
    """float32 storage with the (3, batch) length_info of a sliding-window cache, the per-layer window mask and RoPE
    inside the kernel, through the tensor-level boundary: decode and paged prefill, ragged prefill with rotation."""
    from tests.util import assert_close_where_keys, rows_without_keys
    rng = np.random.default_rng(305 + d)
    spec = [(100, 4, 20), (257, 0, 0), (330, 16, 48), (33, 2, 2), (ps, 0, 0), (90, 0, 17)]   # physical length, sink, window offset
    need = 4 + sum((x[0] + ps - 1) // ps for x in spec)
    pages, pindptr, pvalues, last, _, _ = build_paged_kv(rng, [x[0] for x in spec], need, hkv, ps, d, dtype=F32)
    info = np.array([last, [x[2] for x in spec], [x[1] for x in spec]], np.int32)
    logical = np.array([n - off + sink for n, sink, off in spec])
    b = len(spec)
    k_off = rng.integers(0, 200, size=b).astype(np.int32)
    _, pages_dl = T(pages)
    q = rng.standard_normal((b, hq, d)).astype(F32)
    q_pos = (k_off + logical - 1).astype(np.int32)
    for rotary in (0, 1):
        eo, el = np.zeros((b, hq, d), F32), np.zeros((b, hq), F32)
        ok.decode(q, pages, pindptr, pvalues, info, k_off, q_pos, eo, el, rotary, 1.0, 1e4, d ** -0.5)
        out, out_dl = T(np.full((b, hq, d), 7.0, F32))
        lse, lse_dl = T(np.full((b, hq), 7.0, F32))
        dl.call("batch_decode_paged_kv", T(q)[1], pages_dl, TI(pindptr), TI(pvalues), TI(info), TI(k_off), TI(q_pos), out_dl, lse_dl,
                rotary, 1.0, 1e4, d ** -0.5)
        assert_close(host(out), eo, what=f"f32 sliding decode out, rotary {rotary}", atol=1e-3, rtol=1e-3)
        assert_close(host(lse), el, atol=1e-3, rtol=1e-4, what=f"f32 sliding decode lse, rotary {rotary}")
    sq_lens = [7, 64, 33, 3, 1, 30]
    n = sum(sq_lens)
    qindptr = np.concatenate([[0], np.cumsum(sq_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F32)
    q_pos = np.concatenate([k_off[i] + logical[i] - sq_lens[i] + np.arange(sq_lens[i]) for i in range(b)]).astype(np.int32)
    for causal, window, rotary in ((0, 0, 1), (1, 40, 1), (1, 12, 0)):
        eo, el = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
        ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, info, k_off, q_pos, eo, el, causal, rotary, 1.0, 1e4, d ** -0.5,
                         sliding_window_size=window)
        out, out_dl = T(np.full((n, hq, d), 7.0, F32))
        lse, lse_dl = T(np.full((n, hq), 7.0, F32))
        dl.call("batch_prefill_paged_kv", T(q)[1], TI(qindptr), pages_dl, TI(pindptr), TI(pvalues), TI(info), TI(k_off), TI(q_pos),
                out_dl, lse_dl, causal, rotary, 1.0, 1e4, d ** -0.5, window)
        assert_close_where_keys(host(out), host(lse), eo, el, rows_without_keys(sq_lens, causal, window), 1e-3,
                                f"f32 sliding paged, causal {causal}, window {window}, rotary {rotary}")
    lens = [130, 5, 1, 70]
    n = sum(lens)
    ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F32) for h in (hq, hkv, hkv))
    off = rng.integers(0, 100, size=len(lens)).astype(np.int32)
    pos = np.concatenate([off[i] + np.arange(lens[i]) for i in range(len(lens))]).astype(np.int32)
    eo, el = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
    ok.prefill_ragged(q, ind, k, v, ind, pos, off, eo, el, 1, 1, 1.0, 1e4, d ** -0.5)
    out, out_dl = T(np.full((n, hq, d), 7.0, F32))
    lse, lse_dl = T(np.full((n, hq), 7.0, F32))
    dl.call("batch_prefill_ragged_kv", T(q)[1], TI(ind), T(k)[1], T(v)[1], TI(ind), TI(pos), TI(off), out_dl, lse_dl, 1, 1, 1.0, 1e4,
            d ** -0.5)
    assert_close(host(out), eo, what="f32 ragged out, rotary", atol=1e-3, rtol=1e-3)
    assert_close(host(lse), el, atol=1e-3, rtol=1e-4, what="f32 ragged lse, rotary")


@pytest.mark.parametrize("hq,hkv,d,ps", [(32, 8, 128, 24), (8, 2, 64, 5), (8, 2, 128, 1), (8, 2, 72, 16), (16, 4, 40, 48),
                                         (8, 1, 200, 7)])
def test_fp16_pages_and_head_dims_outside_the_tuned_set(hq, hkv, d, ps):
    """Page sizes other than 16 / 32 / 64 / 128 and head dims other than 64 / 80 / 96 / 112 / 128 / 256 through the
    pointer-level launchers: decode, paged prefill (both masks), ragged prefill, both token-tree forms, the
    split + RoPE kernel and merge_state_inplace."""
    rng = np.random.default_rng(304)
    kv_lens = [0, 1, ps, ps + 1, 300, 77, 1200]
    b = len(kv_lens)
    pages, indptr, values, last, _, _ = paged_case(rng, kv_lens, [1] * b, hq, hkv, d, ps, F16)
    z = np.zeros(b, np.int32)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), F32)
    ok.decode(q, pages, indptr, values, last, z, z, eo, el, 0, 1.0, 1e4, d ** -0.5)
    go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_decode_paged_kv(dev(q), dev(pages), i32(indptr), i32(values), i32(last), i32(z), i32(z), go, gl, 0, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="decode out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="decode lse")
    q_lens = [3, 1, 2, ps + 1, 64, 30, 130]
    for causal in (0, 1):
        lens = [max(k, ql) for k, ql in zip(kv_lens, q_lens)] if causal else kv_lens
        pages, indptr, values, last, qindptr, q = paged_case(rng, lens, q_lens, hq, hkv, d, ps, F16)
        n = len(q)
        zq = np.zeros(n, np.int32)
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), F32)
        ok.prefill_paged(q, qindptr, pages, indptr, values, last, z, zq, eo, el, causal, 0, 1.0, 1e4, d ** -0.5)
        go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(indptr), i32(values), i32(last), i32(z), i32(zq), go, gl,
                                 causal, 0, 1.0, 1e4, d ** -0.5)
        assert_close(host(go), eo, what=f"paged out, causal {causal}")
        assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"paged lse, causal {causal}")
    # token tree over pages
    prefix = [10, 0, 129]
    trees = [REFERENCE_TREES[0], REFERENCE_TREES[3], random_forest(rng, 31)]
    new_lens = [7, 14, 16]
    kv2 = [p + len(t) for p, t in zip(prefix, trees)]
    pages, pindptr, pvalues, last, _, _ = build_paged_kv(rng, kv2, 4 + sum((x + ps - 1) // ps for x in kv2), hkv, ps, d)
    qindptr = np.concatenate([[0], np.cumsum(new_lens)]).astype(np.int32)
    q = rng.standard_normal((int(qindptr[-1]), hq, d)).astype(F16)
    tindptr = np.concatenate([[0], np.cumsum([len(t) for t in trees])]).astype(np.int32)
    labels = np.concatenate([tree_order(t) for t in trees]).astype(np.int32)
    n = len(q)
    zb, zq = np.zeros(3, np.int32), np.zeros(n, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), F32)
    ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, eo, el, 0, 1.0, 1e4, d ** -0.5, tindptr, labels)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.tree_attn_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb), i32(zq), go, gl, 0, 1.0,
                         1e4, d ** -0.5, i32(tindptr), i32(labels))
    assert_close(host(go), eo, what="tree paged out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="tree paged lse")
    if d in (64, 128):
        return  # the ragged kernels and the page kernels do not depend on the page size
    lens = [300, 5, 1, 200]
    n = sum(lens)
    ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F16) for h in (hq, hkv, hkv))
    zq, zb = np.zeros(n, np.int32), np.zeros(len(lens), np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), F32)
    ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_ragged_kv(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(zq), i32(zb), go, gl, 1, 0, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="ragged out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="ragged lse")
    trees = REFERENCE_TREES + [random_forest(rng, 40)]
    tl = [len(t) for t in trees]
    n = sum(tl)
    ind = np.concatenate([[0], np.cumsum(tl)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F16) for h in (hq, hkv, hkv))
    mask = np.concatenate([tree_order(t) for t in trees]).astype(np.int32)
    zq = np.zeros(n, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), F32)
    ok.tree_attn_ragged(q, ind, k, v, ind, zq, ind, mask, eo, el, 0, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_tree_attn(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(zq), i32(ind), i32(mask), go, gl, 0, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="tree ragged out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="tree ragged lse")
    # split + RoPE at this head dim
    pos = np.array([0, 1, 2, 3, 100, 511, 2047, 7, 9], np.int32)
    n = len(pos)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    eq, ek, ev = np.zeros((n, hq, d), F16), np.zeros((n, hkv, d), F16), np.zeros((n, hkv, d), F16)
    ok.fused_rope(qkv, pos, eq, ek, ev, 1)
    gq, gk, gv = (torch.zeros(x.shape, dtype=torch.float16, device=DEV) for x in (eq, ek, ev))
    K.fused_rope(dev(qkv), i32(pos), gq, gk, gv, 1)
    assert np.array_equal(host(gv), ev)
    assert_close(host(gq), eq, atol=2e-3, rtol=2e-3, what="rope q")
    assert_close(host(gk), ek, atol=2e-3, rtol=2e-3, what="rope k")


@pytest.mark.parametrize("hq,hkv,d,ps", [(16, 4, 96, 16), (8, 2, 80, 24), (8, 2, 128, 24), (8, 2, 48, 5), (4, 4, 160, 16),
                                         (8, 1, 112, 32)])
def test_fp16_extended_forms_outside_the_tuned_set(hq, hkv, d, ps):
    """The sliding-window cache (attention sinks, an evicted gap), the per-layer window mask and RoPE inside the
    kernel at head dims and page sizes the tuned extended kernels are not built for: paged prefill, decode, ragged
    prefill, the ragged token-tree form, and a frequency variant."""
    from tests.test_oracle_kernels import sliding_case
    from tests.util import assert_close_where_keys, rows_without_keys
    rng = np.random.default_rng(500 + d + ps)
    spec = [(100, 4, 20), (257, 0, 0), (330, 16, 48), (33, 2, 2), (ps, 0, 0), (90, 0, 17), (900, 8, 40)]
    spec = [(n, min(sink, n), min(max(off, min(sink, n)), n)) for n, sink, off in spec]
    sq_lens = [7, 64, 33, 3, 1, 30, 40]
    need = 4 + sum((x[0] + ps - 1) // ps for x in spec)
    pages, pindptr, pvalues, info, k_log, _ = sliding_case(rng, spec, hkv, d, ps=ps, npages=need)
    n = sum(sq_lens)
    qindptr = np.concatenate([[0], np.cumsum(sq_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k_off = rng.integers(0, 200, size=len(spec)).astype(np.int32)
    q_pos = np.concatenate([k_off[i] + len(k_log[i]) - sq_lens[i] + np.arange(sq_lens[i]) for i in range(len(spec))])
    q_pos = q_pos.astype(np.int32)
    for causal, window, rotary in ((0, 0, 1), (1, 40, 1), (1, 12, 0)):
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), F32)
        ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, info, k_off, q_pos, eo, el, causal, rotary, 1.0, 1e4, d ** -0.5,
                         sliding_window_size=window)
        go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(info), i32(k_off), i32(q_pos),
                                 go, gl, causal, rotary, 1.0, 1e4, d ** -0.5, sliding_window_size=window)
        assert_close_where_keys(host(go), host(gl), eo, el, rows_without_keys(sq_lens, causal, window), 2e-3,
                                f"sliding paged, causal {causal}, window {window}, rotary {rotary}")
    b = len(spec)
    qd = rng.standard_normal((b, hq, d)).astype(F16)
    qd_pos = (k_off + np.array([len(k) for k in k_log]) - 1).astype(np.int32)
    for rotary, scaling in ((0, None), (1, None), (1, {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                                       "high_freq_factor": 4.0, "original_max_position_embeddings": 64})):
        eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), F32)
        with ok.inline_rope_scaling(scaling):
            ok.decode(qd, pages, pindptr, pvalues, info, k_off, qd_pos, eo, el, rotary, 1.0, 1e4, d ** -0.5)
        go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_decode_paged_kv(dev(qd), dev(pages), i32(pindptr), i32(pvalues), i32(info), i32(k_off), i32(qd_pos), go, gl,
                                rotary, 1.0, 1e4, d ** -0.5, rope_scaling=scaling)
        assert_close(host(go), eo, what=f"sliding decode out, rotary {rotary}, {scaling and scaling['rope_type']}")
        assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"sliding decode lse, rotary {rotary}")
    if d in (64, 128):
        return  # the ragged forms of these head dims are the tuned kernels'
    lens = [300, 5, 1, 200]
    n = sum(lens)
    ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F16) for h in (hq, hkv, hkv))
    k_off = rng.integers(0, 100, size=len(lens)).astype(np.int32)
    q_pos = np.concatenate([k_off[i] + np.arange(lens[i]) for i in range(len(lens))]).astype(np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), F32)
    ok.prefill_ragged(q, ind, k, v, ind, q_pos, k_off, eo, el, 1, 1, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_ragged_kv(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(q_pos), i32(k_off), go, gl, 1, 1, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="ragged out, rotary")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="ragged lse, rotary")
    trees = REFERENCE_TREES + [random_forest(rng, 40)]
    tl = [len(t) for t in trees]
    n = sum(tl)
    ind = np.concatenate([[0], np.cumsum(tl)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F16) for h in (hq, hkv, hkv))
    mask = np.concatenate([tree_order(t) for t in trees]).astype(np.int32)
    q_pos = rng.integers(0, 300, size=n).astype(np.int32)  # a node's depth in a real tree; any values pin the lookup
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), F32)
    ok.tree_attn_ragged(q, ind, k, v, ind, q_pos, ind, mask, eo, el, 1, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_tree_attn(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(q_pos), i32(ind), i32(mask), go, gl, 1, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="tree ragged out, rotary")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="tree ragged lse, rotary")


def _random_generic_case(case):
    """One random launch of the generic kernel: storage type, head shape, head dim, page size, sequence lengths
    and the form of the call (decode, paged prefill with either mask, ragged prefill, both token-tree forms) all
    drawn from the seed; float32 storage goes through the tensor-level boundary, fp16 through the launchers."""
    rng = np.random.default_rng(88000 + case)
    dtype = F32 if rng.random() < 0.5 else F16
    hq, hkv = [(8, 2), (4, 4), (32, 8), (12, 1), (20, 2), (48, 2)][rng.integers(6)]
    step = 4 if dtype == F32 else 8
    d = int(rng.integers(2, 256 // step + 1)) * step
    if dtype == F16 and d in (64, 80, 96, 112, 128, 256):
        ps = int(rng.choice([1, 3, 5, 7, 8, 12, 24, 40, 48, 100]))   # a page size the tuned kernels do not have
    else:
        ps = int(rng.choice([1, 3, 5, 8, 12, 16, 24, 32, 48, 64, 100]))
    kind = ["decode", "paged", "paged_causal", "ragged", "tree_ragged", "tree_paged"][rng.integers(6)]
    b = int(rng.integers(1, 9))
    edge = [0, 1, 15, 16, 17, 31, 32, 33, ps, ps + 1, 2 * ps - 1, 255, 256, 257]
    length = lambda hi: int(rng.choice(edge)) if rng.random() < 0.4 else int(rng.integers(0, hi))
    torch_dtype = torch.float32 if dtype == F32 else torch.float16
    what = f"case {case}: {kind} {np.dtype(dtype).name} heads {hq}/{hkv} d {d} page {ps}"

    def outputs(n):
        return (torch.full((n, hq, d), 7.0, dtype=torch_dtype, device=DEV), torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV))

    sm = d ** -0.5
    if kind in ("decode", "paged", "paged_causal", "tree_paged"):
        causal = int(kind == "paged_causal")
        if kind == "tree_paged":
            trees = [random_forest(rng, int(rng.integers(1, 40))) for _ in range(b)]
            new_lens = [int(rng.integers(1, len(t) + 1)) for t in trees]
            kv_lens = [length(400) + len(t) for t in trees]
            q_lens = new_lens
        else:
            kv_lens = [length(1500) for _ in range(b)]
            q_lens = [1] * b if kind == "decode" else [max(1, length(150)) for _ in range(b)]
            if causal:
                kv_lens = [max(k, ql) for k, ql in zip(kv_lens, q_lens)]
        pages, indptr, values, last, qindptr, q = paged_case(rng, kv_lens, q_lens, hq, hkv, d, ps, dtype)
        n = len(q)
        zb, zq = np.zeros(b, np.int32), np.zeros(n, np.int32)
        eo, el = np.zeros((n, hq, d), dtype), np.zeros((n, hq), F32)
        go, gl = outputs(n)
        if kind == "tree_paged":
            tindptr = np.concatenate([[0], np.cumsum([len(t) for t in trees])]).astype(np.int32)
            labels = np.concatenate([tree_order(t) for t in trees]).astype(np.int32)
            ok.tree_attn_paged(q, qindptr, pages, indptr, values, last, zb, zq, eo, el, 0, 1.0, 1e4, sm, tindptr, labels)
            if dtype == F32:
                dl.call("tree_attn_paged_kv", T(q)[1], TI(qindptr), T(pages)[1], TI(indptr), TI(values), TI(last), TI(zb), TI(zq),
                        dl.tensor(go), dl.tensor(gl), 0, 1.0, 1e4, sm, TI(tindptr), TI(labels.reshape(-1)))
            else:
                K.tree_attn_paged_kv(dev(q), i32(qindptr), dev(pages), i32(indptr), i32(values), i32(last), i32(zb), i32(zq), go, gl,
                                     0, 1.0, 1e4, sm, i32(tindptr), i32(labels))
        elif kind == "decode":
            ok.decode(q, pages, indptr, values, last, zb, zb, eo, el, 0, 1.0, 1e4, sm)
            if dtype == F32:
                dl.call("batch_decode_paged_kv", T(q)[1], T(pages)[1], TI(indptr), TI(values), TI(last), TI(zb), TI(zb),
                        dl.tensor(go), dl.tensor(gl), 0, 1.0, 1e4, sm)
            else:
                K.batch_decode_paged_kv(dev(q), dev(pages), i32(indptr), i32(values), i32(last), i32(zb), i32(zb), go, gl, 0, 1.0,
                                        1e4, sm)
        else:
            ok.prefill_paged(q, qindptr, pages, indptr, values, last, zb, zq, eo, el, causal, 0, 1.0, 1e4, sm)
            if dtype == F32:
                dl.call("batch_prefill_paged_kv", T(q)[1], TI(qindptr), T(pages)[1], TI(indptr), TI(values), TI(last), TI(zb),
                        TI(zq), dl.tensor(go), dl.tensor(gl), causal, 0, 1.0, 1e4, sm, 0)
            else:
                K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(indptr), i32(values), i32(last), i32(zb), i32(zq),
                                         go, gl, causal, 0, 1.0, 1e4, sm)
    else:
        if kind == "tree_ragged":
            trees = [random_forest(rng, int(rng.integers(1, 70))) for _ in range(b)]
            lens = [len(t) for t in trees]
        else:
            lens = [max(1, length(300)) for _ in range(b)]
        n = sum(lens)
        ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        q, k, v = (rng.standard_normal((n, h, d)).astype(dtype) for h in (hq, hkv, hkv))
        zq, zb = np.zeros(n, np.int32), np.zeros(b, np.int32)
        eo, el = np.zeros((n, hq, d), dtype), np.zeros((n, hq), F32)
        go, gl = outputs(n)
        if dtype == F16 and d in (64, 128, 256) or (dtype == F16 and kind == "ragged" and d in (80, 96, 112)):
            return  # the tuned kernels' shapes: covered by their own sweep
        if kind == "tree_ragged":
            mask = np.concatenate([tree_order(t) for t in trees]).astype(np.int32)
            ok.tree_attn_ragged(q, ind, k, v, ind, zq, ind, mask, eo, el, 0, 1.0, 1e4, sm)
            if dtype == F32:
                dl.call("batch_tree_attn", T(q)[1], TI(ind), T(k)[1], T(v)[1], TI(ind), TI(zq), TI(ind), TI(mask.reshape(-1)),
                        dl.tensor(go), dl.tensor(gl), 0, 1.0, 1e4, sm)
            else:
                K.batch_tree_attn(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(zq), i32(ind), i32(mask), go, gl, 0, 1.0, 1e4, sm)
        else:
            causal = int(rng.integers(2))
            ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, causal, 0, 1.0, 1e4, sm)
            if dtype == F32:
                dl.call("batch_prefill_ragged_kv", T(q)[1], TI(ind), T(k)[1], T(v)[1], TI(ind), TI(zq), TI(zb), dl.tensor(go),
                        dl.tensor(gl), causal, 0, 1.0, 1e4, sm)
            else:
                K.batch_prefill_ragged_kv(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(zq), i32(zb), go, gl, causal, 0, 1.0,
                                          1e4, sm)
    assert_close(host(go), eo, what=what + " out", **tol(dtype))
    assert_close(host(gl), el, atol=2e-3 if dtype == F16 else 3e-4, rtol=1e-4, what=what + " lse")


@pytest.mark.parametrize("block", range(4))
def test_random_generic_kernel_cases(block):
    for case in range(block * 20, block * 20 + 20):
        _random_generic_case(case)


def _random_generic_extended_case(case):
    """One random launch of the generic kernel's extended form: a sliding-window cache with random sinks and evicted
    gaps (or a plain one), RoPE inside the kernel or not, the per-layer window mask; decode, paged prefill or ragged
    prefill; storage type, head shape, head dim and page size drawn from the seed."""
    from tests.util import assert_close_where_keys, rows_without_keys
    rng = np.random.default_rng(99000 + case)
    dtype = F32 if rng.random() < 0.5 else F16
    hq, hkv = [(8, 2), (4, 4), (32, 8), (12, 1), (20, 2)][rng.integers(5)]
    step = 8 if dtype == F32 else 16
    d = int(rng.integers(1, 256 // step + 1)) * step
    if dtype == F16 and d in (64, 128, 256):
        ps = int(rng.choice([1, 3, 5, 8, 12, 24, 40, 100]))   # a page size the tuned kernels do not have
    else:
        ps = int(rng.choice([1, 3, 5, 8, 12, 16, 24, 32, 64, 100]))
    kind = ["decode", "paged", "ragged"][rng.integers(3)]
    rotary = int(rng.integers(2)) if kind != "ragged" else 1
    sliding = int(rng.integers(2)) if kind != "ragged" else 0
    if not rotary and not sliding:
        rotary = 1
    b = int(rng.integers(1, 7))
    sm = d ** -0.5
    torch_dtype = torch.float32 if dtype == F32 else torch.float16
    what = f"extended case {case}: {kind} {np.dtype(dtype).name} heads {hq}/{hkv} d {d} page {ps} rotary {rotary} sliding {sliding}"

    def outputs(n):
        return (torch.full((n, hq, d), 7.0, dtype=torch_dtype, device=DEV), torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV))

    if kind == "ragged":
        lens = [int(rng.integers(1, 200)) for _ in range(b)]
        n = sum(lens)
        ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        q, k, v = (rng.standard_normal((n, h, d)).astype(dtype) for h in (hq, hkv, hkv))
        off = rng.integers(0, 3000, size=b).astype(np.int32)
        pos = np.concatenate([off[i] + np.arange(lens[i]) for i in range(b)]).astype(np.int32)
        causal = int(rng.integers(2))
        eo, el = np.zeros((n, hq, d), dtype), np.zeros((n, hq), F32)
        ok.prefill_ragged(q, ind, k, v, ind, pos, off, eo, el, causal, 1, 1.0, 1e4, sm)
        go, gl = outputs(n)
        if dtype == F32:
            dl.call("batch_prefill_ragged_kv", T(q)[1], TI(ind), T(k)[1], T(v)[1], TI(ind), TI(pos), TI(off), dl.tensor(go),
                    dl.tensor(gl), causal, 1, 1.0, 1e4, sm)
        else:
            K.batch_prefill_ragged_kv(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(pos), i32(off), go, gl, causal, 1, 1.0, 1e4, sm)
        assert_close(host(go), eo, what=what + " out", atol=4e-3 if dtype == F16 else 1e-3, rtol=1e-2 if dtype == F16 else 1e-3)
        assert_close(host(gl), el, atol=2e-3 if dtype == F16 else 1e-3, rtol=1e-4, what=what + " lse")
        return
    phys = [int(rng.integers(1, 700)) for _ in range(b)]
    sinks = [int(rng.integers(0, min(n, 20) + 1)) if sliding else 0 for n in phys]
    offs = [int(rng.integers(s, n + 1)) if sliding else 0 for s, n in zip(sinks, phys)]
    offs = [min(o, n - 1) if o > s else s for o, s, n in zip(offs, sinks, phys)]   # at least one visible key
    logical = np.array([n - o + s for n, o, s in zip(phys, offs, sinks)])
    need = 4 + sum((n + ps - 1) // ps for n in phys)
    pages, indptr, values, last, _, _ = build_paged_kv(rng, phys, need, hkv, ps, d, dtype=dtype)
    info = np.array([last, offs, sinks], np.int32) if sliding else np.asarray(last, np.int32)
    k_off = rng.integers(0, 3000, size=b).astype(np.int32)
    if kind == "decode":
        q = rng.standard_normal((b, hq, d)).astype(dtype)
        q_pos = (k_off + logical - 1).astype(np.int32)
        eo, el = np.zeros((b, hq, d), dtype), np.zeros((b, hq), F32)
        ok.decode(q, pages, indptr, values, info, k_off, q_pos, eo, el, rotary, 1.0, 1e4, sm)
        go, gl = outputs(b)
        if dtype == F32:
            dl.call("batch_decode_paged_kv", T(q)[1], T(pages)[1], TI(indptr), TI(values), TI(info), TI(k_off), TI(q_pos),
                    dl.tensor(go), dl.tensor(gl), rotary, 1.0, 1e4, sm)
        else:
            K.batch_decode_paged_kv(dev(q), dev(pages), i32(indptr), i32(values), i32(info), i32(k_off), i32(q_pos), go, gl, rotary,
                                    1.0, 1e4, sm)
        assert_close(host(go), eo, what=what + " out", atol=4e-3 if dtype == F16 else 1e-3, rtol=1e-2 if dtype == F16 else 1e-3)
        assert_close(host(gl), el, atol=2e-3 if dtype == F16 else 1e-3, rtol=1e-4, what=what + " lse")
        return
    q_lens = [int(rng.integers(1, min(int(n), 90) + 1)) for n in logical]
    n = sum(q_lens)
    qindptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(dtype)
    q_pos = np.concatenate([k_off[i] + logical[i] - q_lens[i] + np.arange(q_lens[i]) for i in range(b)]).astype(np.int32)
    causal = int(rng.integers(2))
    window = int(rng.choice([0, 5, 40, 1024])) if (causal and sliding) else 0
    eo, el = np.zeros((n, hq, d), dtype), np.zeros((n, hq), F32)
    ok.prefill_paged(q, qindptr, pages, indptr, values, info, k_off, q_pos, eo, el, causal, rotary, 1.0, 1e4, sm,
                     sliding_window_size=window)
    go, gl = outputs(n)
    if dtype == F32:
        dl.call("batch_prefill_paged_kv", T(q)[1], TI(qindptr), T(pages)[1], TI(indptr), TI(values), TI(info), TI(k_off), TI(q_pos),
                dl.tensor(go), dl.tensor(gl), causal, rotary, 1.0, 1e4, sm, window)
    else:
        K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(indptr), i32(values), i32(info), i32(k_off), i32(q_pos), go,
                                 gl, causal, rotary, 1.0, 1e4, sm, sliding_window_size=window)
    no_keys = rows_without_keys(q_lens, causal, window if sliding else 0)
    assert_close_where_keys(host(go), host(gl), eo, el, no_keys, 2e-3 if dtype == F16 else 1e-3, what)


@pytest.mark.parametrize("block", range(2))
def test_random_generic_extended_cases(block):
    for case in range(block * 20, block * 20 + 20):
        _random_generic_extended_case(case)
