"""Pins the C oracle (oracle/kv_kernels.c) to closed forms, invariants and brute force.

No formula of the oracle is retyped here: the expected values come from oracle/closed_form.py
(the numpy definitions that the reference's own tests use) and from special cases whose answer
is known a priori.
"""
import numpy as np
import pytest

from oracle import closed_form as cf
from oracle import kernels as ok
from tests.util import REFERENCE_TREES, assert_close, build_paged_kv, random_forest, tree_order

F16 = np.float16


# ----------------------------------------------------------------------------- RoPE
@pytest.mark.parametrize("d", [64, 128])
def test_rope_matches_closed_form(d):
    rng = np.random.default_rng(0)
    hq, hkv = 8, 2
    positions = np.array([0, 1, 2, 17, 2047, 131071], np.int32)
    n = len(positions)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    q = np.zeros((n, hq, d), F16)
    k = np.zeros((n, hkv, d), F16)
    v = np.zeros((n, hkv, d), F16)
    ok.fused_rope(qkv, positions, q, k, v, 1)
    exp_q = cf.apply_rotary(qkv[:, :hq], positions)
    exp_k = cf.apply_rotary(qkv[:, hq:hq + hkv], positions)
    # fp16 rounding of the result (2^-11 relative) plus fp32 angle error at pos 131071
    # (ulp(131071) ~ 0.0078 rad times |x| <~ 4)
    small = positions < 4096
    assert_close(q[small], exp_q[small], atol=2e-3, rtol=2e-3, what="q rope")
    assert_close(k[small], exp_k[small], atol=2e-3, rtol=2e-3, what="k rope")
    assert_close(q, exp_q, atol=6e-2, rtol=2e-3, what="q rope long")
    assert np.array_equal(v, qkv[:, hq + hkv:]), "v must be a plain split"


def test_rope_invariants():
    rng = np.random.default_rng(1)
    d, hq, hkv, n = 128, 4, 4, 5
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    q = np.zeros((n, hq, d), F16)
    k = np.zeros((n, hkv, d), F16)
    v = np.zeros((n, hkv, d), F16)
    # position 0 is the identity
    ok.fused_rope(qkv, np.zeros(n, np.int32), q, k, v, 1)
    assert np.array_equal(q, qkv[:, :hq]) and np.array_equal(k, qkv[:, hq:hq + hkv])
    # apply_rope = 0 is a plain split at any position
    ok.fused_rope(qkv, np.arange(n, dtype=np.int32) * 1000, q, k, v, 0)
    assert np.array_equal(q, qkv[:, :hq]) and np.array_equal(k, qkv[:, hq:hq + hkv])
    # rotation preserves the norm of every (d, d + D/2) pair
    pos = np.array([3, 50, 700, 9000, 65000], np.int32)
    ok.fused_rope(qkv, pos, q, k, v, 1)
    x = qkv[:, :hq].astype(np.float64)
    y = q.astype(np.float64)
    n_in = x[..., :d // 2] ** 2 + x[..., d // 2:] ** 2
    n_out = y[..., :d // 2] ** 2 + y[..., d // 2:] ** 2
    assert_close(n_out, n_in, atol=2e-2, rtol=5e-3, what="pair norm")
    # the relative-position property: <rope(q,p), rope(k,p)> depends on p only through p-p = 0
    dot_in = (qkv[:, :hq].astype(np.float64) * np.repeat(qkv[:, hq:hq + hkv], 1, axis=1).astype(np.float64)).sum(-1)
    dot_out = (q.astype(np.float64) * k.astype(np.float64)).sum(-1)
    assert_close(dot_out, dot_in, atol=5e-2, rtol=1e-2, what="relative position")


# ----------------------------------------------------------------------------- append / gather
def test_append_gather_round_trip_and_skip():
    rng = np.random.default_rng(2)
    hkv, ps, d, npages = 3, 16, 64, 9
    pages = np.zeros((npages, 2, hkv, ps, d), F16)
    n = 40
    slots = rng.permutation(npages * ps)[:n].astype(np.int32)
    slots[5] = -1
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    ok.transpose_append(pages, k, v, slots)
    # brute force: the documented layout pages[p // ps, 0|1, h, p % ps, :]
    expect = np.zeros_like(pages)
    for i, p in enumerate(slots):
        if p >= 0:
            expect[p // ps, 0, :, p % ps] = k[i]
            expect[p // ps, 1, :, p % ps] = v[i]
    assert np.array_equal(pages, expect)
    keep = slots >= 0
    kd = np.zeros((2, keep.sum(), hkv, d), F16)
    vd = np.zeros_like(kd)
    ok.debug_get_kv(pages, slots[keep], kd, vd, 1)
    assert np.array_equal(kd[1], k[keep]) and np.array_equal(vd[1], v[keep])
    assert not kd[0].any()


def test_append_gather_mla_round_trip():
    rng = np.random.default_rng(3)
    ps, d, npages, n = 64, 576, 4, 70
    pages = np.zeros((npages, ps, d), F16)
    slots = rng.permutation(npages * ps)[:n].astype(np.int32)
    slots[0] = -1
    kv = rng.standard_normal((n, d)).astype(F16)
    ok.transpose_append_mla(pages, kv, slots)
    flat = pages.reshape(npages * ps, d)
    assert np.array_equal(flat[slots[1:]], kv[1:])
    assert np.count_nonzero(flat.any(axis=1)) == n - 1
    out = np.zeros((1, n - 1, d), F16)
    ok.debug_get_kv_mla(pages, slots[1:], out, 0)
    assert np.array_equal(out[0], kv[1:])


def test_copy_single_page_and_compact_copy():
    rng = np.random.default_rng(4)
    hkv, ps, d, npages = 2, 16, 32, 5
    pages = rng.standard_normal((npages, 2, hkv, ps, d)).astype(F16)
    before = pages.copy()
    ok.copy_single_page(pages, 1, 3, 7)
    assert np.array_equal(pages[3, :, :, :7], before[1, :, :, :7])
    assert np.array_equal(pages[3, :, :, 7:], before[3, :, :, 7:])
    assert np.array_equal(np.delete(pages, 3, axis=0), np.delete(before, 3, axis=0))
    # compact copy: batch of 2, copies src->dst slot by slot
    before = pages.copy()
    indptr = np.array([0, 2, 3], np.int32)
    src_dst = np.array([[20, 21, 70], [17, 18, 65]], np.int32)
    ok.compact_kv_copy(pages, indptr, src_dst, 2)
    flat_b = before.transpose(0, 3, 1, 2, 4).reshape(npages * ps, 2, hkv, d)
    flat_a = pages.transpose(0, 3, 1, 2, 4).reshape(npages * ps, 2, hkv, d)
    for s, t in src_dst.T:
        assert np.array_equal(flat_a[t], flat_b[s])
    mla = rng.standard_normal((4, 64, 576)).astype(F16)
    mb = mla.copy()
    ok.copy_single_page_mla(mla, 0, 2, 33)
    assert np.array_equal(mla[2, :33], mb[0, :33]) and np.array_equal(mla[2, 33:], mb[2, 33:])


# ----------------------------------------------------------------------------- attention
def _decode_case(rng, kv_lens, hq, hkv, d, ps=16, npages=64):
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, kv_lens, npages, hkv, ps, d)
    b = len(kv_lens)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    out = np.zeros((b, hq, d), F16)
    lse = np.zeros((b, hq), np.float32)
    zeros = np.zeros(b, np.int32)
    ok.decode(q, pages, indptr, values, last, zeros, zeros, out, lse, 0, 1.0, 1e4, d ** -0.5)
    return q, ks, vs, out, lse


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (4, 4, 64), (8, 1, 128)])
def test_decode_matches_softmax_closed_form(hq, hkv, d):
    rng = np.random.default_rng(5)
    kv_lens = [1, 15, 16, 17, 100, 0]
    q, ks, vs, out, lse = _decode_case(rng, kv_lens, hq, hkv, d)
    for i, n in enumerate(kv_lens):
        if n == 0:
            assert not out[i].any() and np.all(lse[i] == np.float32(-5e4))
            continue
        eo, el = cf.attention(q[i:i + 1], ks[i], vs[i], d ** -0.5, causal=False)
        assert_close(out[i], eo[0], atol=2e-3, rtol=2e-3, what=f"decode out seq {i}")
        assert_close(lse[i], el[0], atol=1e-3, rtol=1e-4, what=f"decode lse seq {i}")


def test_decode_single_key_returns_its_value():
    rng = np.random.default_rng(6)
    q, ks, vs, out, lse = _decode_case(rng, [1], 4, 2, 64)
    assert np.array_equal(out[0], np.repeat(vs[0][0], 2, axis=0))


def _ragged_case(rng, lens, hq, hkv, dqk, dv, causal):
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, dqk)).astype(F16)
    k = rng.standard_normal((n, hkv, dqk)).astype(F16)
    v = rng.standard_normal((n, hkv, dv)).astype(F16)
    out = np.zeros((n, hq, dv), F16)
    lse = np.zeros((n, hq), np.float32)
    ok.prefill_ragged(q, indptr, k, v, indptr, np.zeros(n, np.int32), np.zeros(len(lens), np.int32),
                      out, lse, causal, 0, 1.0, 1e4, dqk ** -0.5)
    return indptr, q, k, v, out, lse


@pytest.mark.parametrize("hq,hkv,dqk,dv,causal", [(8, 2, 128, 128, 1), (4, 4, 192, 128, 1), (4, 2, 64, 64, 0)])
def test_ragged_prefill_matches_closed_form(hq, hkv, dqk, dv, causal):
    rng = np.random.default_rng(7)
    lens = [1, 5, 33, 16]
    indptr, q, k, v, out, lse = _ragged_case(rng, lens, hq, hkv, dqk, dv, causal)
    for i in range(len(lens)):
        s, e = indptr[i], indptr[i + 1]
        eo, el = cf.attention(q[s:e], k[s:e], v[s:e], dqk ** -0.5, causal=bool(causal))
        assert_close(out[s:e], eo, atol=2e-3, rtol=2e-3, what=f"ragged out seq {i}")
        assert_close(lse[s:e], el, atol=1e-3, rtol=1e-4, what=f"ragged lse seq {i}")


def test_ragged_first_row_sees_only_itself():
    rng = np.random.default_rng(8)
    indptr, q, k, v, out, lse = _ragged_case(rng, [9], 4, 2, 64, 64, 1)
    assert np.array_equal(out[0], np.repeat(v[0], 2, axis=0))


@pytest.mark.parametrize("causal", [0, 1])
def test_paged_prefill_matches_closed_form(causal):
    rng = np.random.default_rng(9)
    hq, hkv, d = 8, 2, 128
    kv_lens = [40, 16, 0, 75]
    q_lens = [7, 16, 3, 30]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, kv_lens, 32, hkv, 16, d)
    n = sum(q_lens)
    qindptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    out = np.zeros((n, hq, d), F16)
    lse = np.zeros((n, hq), np.float32)
    zb = np.zeros(len(kv_lens), np.int32)
    ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, last, zb, np.zeros(n, np.int32), out, lse,
                     causal, 0, 1.0, 1e4, d ** -0.5)
    for i, (nk, nq) in enumerate(zip(kv_lens, q_lens)):
        s, e = qindptr[i], qindptr[i + 1]
        if nk == 0:
            assert not out[s:e].any() and np.all(lse[s:e] == np.float32(-5e4))
            continue
        eo, el = cf.attention(q[s:e], ks[i], vs[i], d ** -0.5, causal=bool(causal))
        assert_close(out[s:e], eo, atol=2e-3, rtol=2e-3, what=f"paged out seq {i}")
        assert_close(lse[s:e], el, atol=1e-3, rtol=1e-4, what=f"paged lse seq {i}")


def test_decode_equals_paged_prefill_with_one_query():
    rng = np.random.default_rng(10)
    hq, hkv, d = 8, 4, 64
    kv_lens = [33, 7]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, kv_lens, 8, hkv, 16, d)
    q = rng.standard_normal((2, hq, d)).astype(F16)
    o1, o2 = np.zeros((2, hq, d), F16), np.zeros((2, hq, d), F16)
    l1, l2 = np.zeros((2, hq), np.float32), np.zeros((2, hq), np.float32)
    z = np.zeros(2, np.int32)
    ok.decode(q, pages, pindptr, pvalues, last, z, z, o1, l1, 0, 1.0, 1e4, 0.125)
    ok.prefill_paged(q, np.array([0, 1, 2], np.int32), pages, pindptr, pvalues, last, z, z, o2, l2,
                     0, 0, 1.0, 1e4, 0.125)
    assert np.array_equal(o1, o2) and np.array_equal(l1, l2)


def test_inline_rope_equals_rope_then_attend():
    """rotary_mode=1 inside the kernels must equal RoPE applied up front (NORMAL mode)."""
    rng = np.random.default_rng(11)
    hq, hkv, d, n = 4, 2, 64, 21
    k_raw = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    q_raw = rng.standard_normal((1, hq, d)).astype(F16)
    pages = np.zeros((4, 2, hkv, 16, d), F16)
    slots = np.arange(n, dtype=np.int32) + 16
    ok.transpose_append(pages, k_raw, v, slots)
    pindptr, pvalues, last = np.array([0, 2], np.int32), np.array([1, 2], np.int32), np.array([5], np.int32)
    out_inline = np.zeros((1, hq, d), F16)
    lse_inline = np.zeros((1, hq), np.float32)
    ok.decode(q_raw, pages, pindptr, pvalues, last, np.array([100], np.int32), np.array([100 + n - 1], np.int32),
              out_inline, lse_inline, 1, 1.0, 1e4, d ** -0.5)
    k_rot = cf.apply_rotary(k_raw, 100 + np.arange(n)).astype(F16)
    q_rot = cf.apply_rotary(q_raw, [100 + n - 1]).astype(F16)
    eo, el = cf.attention(q_rot, k_rot, v, d ** -0.5, causal=False)
    assert_close(out_inline[0], eo[0], atol=3e-3, rtol=3e-3, what="inline rope out")


# ----------------------------------------------------------------------------- token trees
def test_tree_order_interval_test_is_the_ancestor_relation():
    """What the kernels evaluate on the (first, second) labels equals the mask built from the parent
    pointers, for the reference's trees and random forests."""
    rng = np.random.default_rng(30)
    trees = REFERENCE_TREES + [random_forest(rng, n) for n in (1, 2, 9, 40, 256)]
    for parents in trees:
        lab = tree_order(parents).astype(np.int64)
        sees = (lab[:, None, 0] >= lab[None, :, 0]) & (lab[:, None, 0] < lab[None, :, 1])
        assert np.array_equal(sees, cf.tree_ancestor_mask(parents)), parents


def _tree_ragged_case(rng, trees, hq, hkv, d):
    lens = [len(t) for t in trees]
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    mask = np.concatenate([tree_order(t) for t in trees])
    return indptr, q, k, v, mask


@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (4, 4, 64)])
def test_tree_attn_ragged_matches_closed_form(hq, hkv, d):
    rng = np.random.default_rng(31)
    trees = REFERENCE_TREES + [random_forest(rng, 70)]
    indptr, q, k, v, mask = _tree_ragged_case(rng, trees, hq, hkv, d)
    out = np.zeros_like(q)
    lse = np.zeros(q.shape[:2], np.float32)
    ok.tree_attn_ragged(q, indptr, k, v, indptr, np.zeros(len(q), np.int32), indptr, mask, out, lse,
                        0, 1.0, 1e4, d ** -0.5)
    for i, parents in enumerate(trees):
        s, e = indptr[i], indptr[i + 1]
        eo, el = cf.attention(q[s:e], k[s:e], v[s:e], d ** -0.5, mask=cf.tree_ancestor_mask(parents))
        assert_close(out[s:e], eo, atol=2e-3, rtol=2e-3, what=f"tree out seq {i}")
        assert_close(lse[s:e], el, atol=1e-3, rtol=1e-4, what=f"tree lse seq {i}")
    # a root sees only itself
    assert np.array_equal(out[0], np.repeat(v[0], hq // hkv, axis=0))


def test_tree_attn_on_chains_is_causal_attention():
    rng = np.random.default_rng(32)
    hq, hkv, d = 8, 2, 64
    trees = [list(range(-1, n - 1)) for n in (1, 7, 33)]
    indptr, q, k, v, mask = _tree_ragged_case(rng, trees, hq, hkv, d)
    zeros = np.zeros(len(q), np.int32)
    o1, o2 = np.zeros_like(q), np.zeros_like(q)
    l1, l2 = np.zeros(q.shape[:2], np.float32), np.zeros(q.shape[:2], np.float32)
    ok.tree_attn_ragged(q, indptr, k, v, indptr, zeros, indptr, mask, o1, l1, 0, 1.0, 1e4, 0.125)
    ok.prefill_ragged(q, indptr, k, v, indptr, zeros, np.zeros(3, np.int32), o2, l2, 1, 0, 1.0, 1e4, 0.125)
    assert np.array_equal(o1, o2) and np.array_equal(l1, l2)


def tree_paged_case(rng, prefix_lens, trees, new_lens, hq, hkv, d, ps=16, npages=64):
    """Sequences whose pages hold a prefix followed by the nodes of a token tree; the queries are
    the last new_lens[i] nodes of each tree (a tree can grow over several steps)."""
    kv_lens = [p + len(t) for p, t in zip(prefix_lens, trees)]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, kv_lens, npages, hkv, ps, d)
    qindptr = np.concatenate([[0], np.cumsum(new_lens)]).astype(np.int32)
    q = rng.standard_normal((int(qindptr[-1]), hq, d)).astype(F16)
    tindptr = np.concatenate([[0], np.cumsum([len(t) for t in trees])]).astype(np.int32)
    labels = np.concatenate([tree_order(t) for t in trees])
    masks = []
    for p, t, nq in zip(prefix_lens, trees, new_lens):
        m = np.ones((nq, p + len(t)), bool)
        m[:, p:] = cf.tree_ancestor_mask(t)[len(t) - nq:]
        masks.append(m)
    return pages, pindptr, pvalues, last, ks, vs, qindptr, q, tindptr, labels, masks


def test_tree_attn_paged_matches_closed_form():
    rng = np.random.default_rng(33)
    hq, hkv, d = 8, 2, 128
    prefix = [10, 20, 30, 40, 0]
    trees = REFERENCE_TREES + [random_forest(rng, 50)]
    new_lens = [7, 8, 10, 7, 50]  # sequences 1 and 3: the tree already had nodes from earlier steps
    (pages, pindptr, pvalues, last, ks, vs, qindptr, q, tindptr, labels, masks) = tree_paged_case(
        rng, prefix, trees, new_lens, hq, hkv, d)
    out = np.zeros_like(q)
    lse = np.zeros(q.shape[:2], np.float32)
    zb = np.zeros(len(trees), np.int32)
    ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, np.zeros(len(q), np.int32), out, lse,
                       0, 1.0, 1e4, d ** -0.5, tindptr, labels)
    for i in range(len(trees)):
        s, e = qindptr[i], qindptr[i + 1]
        eo, el = cf.attention(q[s:e], ks[i], vs[i], d ** -0.5, mask=masks[i])
        assert_close(out[s:e], eo, atol=2e-3, rtol=2e-3, what=f"tree paged out seq {i}")
        assert_close(lse[s:e], el, atol=1e-3, rtol=1e-4, what=f"tree paged lse seq {i}")


def test_tree_attn_paged_on_chains_is_causal_paged_prefill():
    rng = np.random.default_rng(34)
    hq, hkv, d = 4, 2, 64
    prefix = [5, 31]
    trees = [list(range(-1, 8)), list(range(-1, 19))]
    new_lens = [9, 4]
    (pages, pindptr, pvalues, last, ks, vs, qindptr, q, tindptr, labels, masks) = tree_paged_case(
        rng, prefix, trees, new_lens, hq, hkv, d)
    zb, zq = np.zeros(2, np.int32), np.zeros(len(q), np.int32)
    o1, o2 = np.zeros_like(q), np.zeros_like(q)
    l1, l2 = np.zeros(q.shape[:2], np.float32), np.zeros(q.shape[:2], np.float32)
    ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, o1, l1, 0, 1.0, 1e4, 0.125,
                       tindptr, labels)
    ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, o2, l2, 1, 0, 1.0, 1e4, 0.125)
    assert np.array_equal(o1, o2) and np.array_equal(l1, l2)


# ----------------------------------------------------------------------------- merge
def test_layer_sliding_window_mask_known_answer():
    """The reference's own known-answer vector for the paged prefill kernel built with
    sliding_window_size = 3 (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_tir.py:98-156):
    zero queries, V = 1, 3, 5 in the first three slots, two query rows -> out[:, 0, 0] = [4, 5]."""
    hq, hkv, d = 4, 2, 64
    q = np.zeros((2, hq, d), F16)
    pages = np.zeros((1, 2, hkv, 16, d), F16)
    for position, value in enumerate([1, 3, 5]):
        pages[0, 1, :, position, :] = value
    out, lse = np.zeros_like(q), np.zeros((2, hq), np.float32)
    ok.prefill_paged(q, np.array([0, 2], np.int32), pages, np.array([0, 1], np.int32), np.array([0], np.int32),
                     np.array([[3], [0], [0]], np.int32), np.array([0], np.int32), np.array([3, 4], np.int32),
                     out, lse, 1, 0, 1.0, 1e4, d ** -0.5, sliding_window_size=3)
    assert_close(out[:, 0, 0], np.array([4, 5], F16), atol=1e-3, rtol=1e-3, what="sliding window known answer")
    assert np.all(out == out[:, :1, :1])


def sliding_case(rng, spec, hkv, d, ps=16, npages=96):
    """spec: list of (physical_len, sink, window_offset).  Returns the page pool, tables, the (3, B)
    length_info and, per sequence, the K/V rows in LOGICAL order (sink tokens, then the window)."""
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, [s[0] for s in spec], npages, hkv, ps, d)
    info = np.array([last, [s[2] for s in spec], [s[1] for s in spec]], np.int32)
    k_log = [np.concatenate([k[:sink], k[off:]]) for k, (n, sink, off) in zip(ks, spec)]
    v_log = [np.concatenate([v[:sink], v[off:]]) for v, (n, sink, off) in zip(vs, spec)]
    return pages, indptr, values, info, k_log, v_log


SLIDING_SPEC = [(100, 4, 20), (257, 0, 0), (700, 16, 48), (33, 2, 2), (17, 0, 5), (1, 0, 0), (64, 16, 32)]


def test_sliding_cache_decode_is_attention_over_sink_plus_window():
    """length_info (3, B): the kernel attends to the first `sink` tokens and to the tokens from
    `window_offset` on (python/tvm/relax/frontend/nn/llm/_kernel_common.py:155-170); with inline
    RoPE the key with logical index t sits at position k_rope_pos_offset + t."""
    rng = np.random.default_rng(21)
    hq, hkv, d = 8, 2, 128
    pages, indptr, values, info, k_log, v_log = sliding_case(rng, SLIDING_SPEC, hkv, d)
    b = len(SLIDING_SPEC)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    k_off = rng.integers(0, 300, size=b).astype(np.int32)
    q_pos = (k_off + np.array([len(k) for k in k_log]) - 1).astype(np.int32)
    for rotary in (0, 1):
        out, lse = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
        ok.decode(q, pages, indptr, values, info, k_off, q_pos, out, lse, rotary, 1.0, 1e4, d ** -0.5)
        for i in range(b):
            kk, qq = k_log[i], q[i:i + 1]
            if rotary:
                kk = cf.apply_rotary(kk, k_off[i] + np.arange(len(kk))).astype(F16)
                qq = cf.apply_rotary(qq, [q_pos[i]]).astype(F16)
            eo, el = cf.attention(qq, kk, v_log[i], d ** -0.5, causal=False)
            assert_close(out[i], eo[0], atol=3e-3, rtol=3e-3, what=f"sliding decode out seq {i} rotary {rotary}")
            assert_close(lse[i], el[0], atol=2e-3, rtol=1e-4, what=f"sliding decode lse seq {i} rotary {rotary}")


def test_merge_closed_form_and_special_cases():
    rng = np.random.default_rng(12)
    n, h, d = 6, 4, 64
    v1 = rng.standard_normal((n, h, d)).astype(F16)
    v2 = rng.standard_normal((n, h, d)).astype(F16)
    s1 = (rng.standard_normal((n, h)) * 3).astype(np.float32)
    s2 = (rng.standard_normal((n, h)) * 3).astype(np.float32)
    s2[0] = -5e4  # empty other side -> unchanged
    s2[1] = s1[1]  # equal weights -> mean
    ev, es = cf.merge(v1, s1, v2, s2)
    mv, ms = v1.copy(), s1.copy()
    ok.merge_state_inplace(mv, ms, v2, s2)
    assert_close(mv, ev, atol=1e-3, rtol=1e-3, what="merge v")
    assert_close(ms, es, atol=1e-5, rtol=1e-6, what="merge s")
    assert np.array_equal(mv[0], v1[0]) and np.array_equal(ms[0], s1[0])
    assert_close(mv[1], (v1[1].astype(np.float64) + v2[1].astype(np.float64)) / 2, atol=1e-3, rtol=1e-3)


def test_self_plus_cross_merge_equals_full_attention():
    """merge(ragged causal over the chunk, paged non-causal over the prefix) = attention over
    prefix+chunk: the identity the chunked-prefill composition of the cache relies on."""
    rng = np.random.default_rng(13)
    hq, hkv, d = 8, 2, 128
    prefix, chunk = 45, 19
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, [prefix], 8, hkv, 16, d)
    q = rng.standard_normal((chunk, hq, d)).astype(F16)
    k = rng.standard_normal((chunk, hkv, d)).astype(F16)
    v = rng.standard_normal((chunk, hkv, d)).astype(F16)
    ind = np.array([0, chunk], np.int32)
    o_self, l_self = np.zeros((chunk, hq, d), F16), np.zeros((chunk, hq), np.float32)
    o_cross, l_cross = np.zeros((chunk, hq, d), F16), np.zeros((chunk, hq), np.float32)
    z1 = np.zeros(1, np.int32)
    zc = np.zeros(chunk, np.int32)
    ok.prefill_ragged(q, ind, k, v, ind, zc, z1, o_self, l_self, 1, 0, 1.0, 1e4, d ** -0.5)
    ok.prefill_paged(q, ind, pages, pindptr, pvalues, last, z1, zc, o_cross, l_cross, 0, 0, 1.0, 1e4, d ** -0.5)
    ok.merge_state_inplace(o_self, l_self, o_cross, l_cross)
    eo, el = cf.attention(q, np.concatenate([ks[0], k]), np.concatenate([vs[0], v]), d ** -0.5, causal=True)
    assert_close(o_self, eo, atol=3e-3, rtol=3e-3, what="merged out")
    assert_close(l_self, el, atol=1e-3, rtol=1e-4, what="merged lse")


# ----------------------------------------------------------------------------- MLA
def test_mla_absorbed_equals_expanded_definition():
    """Absorbed latent attention (what the paged MLA kernel computes) against the definition:
    expand the latent with w_kv and run plain multi-head attention."""
    rng = np.random.default_rng(14)
    h, d_lat, d_rope, d_nope, d_v, ps = 4, 32, 8, 16, 12, 8
    prefix, nq = 21, 3
    latent = (rng.standard_normal((prefix, d_lat + d_rope)) * 0.5).astype(F16)
    w_kv = (rng.standard_normal((d_lat, h * (d_nope + d_v))) * 0.3).astype(np.float64)
    pages = np.zeros((5, ps, d_lat + d_rope), F16)
    page_ids = np.array([3, 0, 4], np.int32)
    slots = np.array([page_ids[t // ps] * ps + t % ps for t in range(prefix)], np.int32)
    ok.transpose_append_mla(pages, latent, slots)
    q = (rng.standard_normal((nq, h, d_nope + d_rope)) * 0.5).astype(np.float64)
    w = w_kv.reshape(d_lat, h, d_nope + d_v)
    w_uk, w_uv = w[..., :d_nope], w[..., d_nope:]
    q_abs = np.concatenate([np.einsum("qhn,lhn->qhl", q[..., :d_nope], w_uk), q[..., d_nope:]], axis=-1).astype(F16)
    out = np.zeros((nq, h, d_lat), F16)
    lse = np.zeros((nq, h), np.float32)
    sm = (d_nope + d_rope) ** -0.5
    ok.prefill_paged_mla(q_abs, np.array([0, nq], np.int32), pages, np.array([0, 3], np.int32), page_ids,
                         np.array([prefix - 2 * ps], np.int32), out, lse, 0, sm, d_latent=d_lat)
    k_full, v_full = cf.mla_expand(latent, w_kv, h, d_nope, d_v)
    eo, el = cf.attention(q, k_full, v_full, sm, causal=False)
    got = np.einsum("qhl,lhv->qhv", out.astype(np.float64), w_uv)
    assert_close(got, eo, atol=1e-2, rtol=1e-2, what="mla out")
    assert_close(lse, el, atol=2e-2, rtol=1e-3, what="mla lse")


def test_mla_absorbed_causal_equals_expanded_definition():
    """The causal form of the paged MLA kernel (the chunk's own rows are in the pages already,
    python/tvm/relax/frontend/nn/llm/_prefill_kernels.py:1021-1031): query row r of nq sees the first
    kv_len - nq + r + 1 cached rows; against the expanded definition with the causal mask, two
    sequences of different lengths, one of them with as many queries as cached rows."""
    rng = np.random.default_rng(15)
    h, d_lat, d_rope, d_nope, d_v, ps = 4, 32, 8, 16, 12, 8
    kv_lens, nqs = [21, 6], [5, 6]
    w_kv = (rng.standard_normal((d_lat, h * (d_nope + d_v))) * 0.3).astype(np.float64)
    w = w_kv.reshape(d_lat, h, d_nope + d_v)
    w_uk, w_uv = w[..., :d_nope], w[..., d_nope:]
    pages = np.zeros((6, ps, d_lat + d_rope), F16)
    page_ids = np.array([3, 0, 4, 5], np.int32)  # 3 pages for sequence 0, 1 for sequence 1
    page_indptr = np.array([0, 3, 4], np.int32)
    latents, q_abs_all, qs = [], [], []
    for b, (n, nq) in enumerate(zip(kv_lens, nqs)):
        latent = (rng.standard_normal((n, d_lat + d_rope)) * 0.5).astype(F16)
        ids = page_ids[page_indptr[b]:page_indptr[b + 1]]
        slots = np.array([ids[t // ps] * ps + t % ps for t in range(n)], np.int32)
        ok.transpose_append_mla(pages, latent, slots)
        q = (rng.standard_normal((nq, h, d_nope + d_rope)) * 0.5).astype(np.float64)
        q_abs_all.append(np.concatenate([np.einsum("qhn,lhn->qhl", q[..., :d_nope], w_uk), q[..., d_nope:]], axis=-1))
        latents.append(latent)
        qs.append(q)
    q_abs = np.concatenate(q_abs_all).astype(F16)
    total = sum(nqs)
    out, lse = np.zeros((total, h, d_lat), F16), np.zeros((total, h), np.float32)
    sm = (d_nope + d_rope) ** -0.5
    last = np.array([(n - 1) % ps + 1 for n in kv_lens], np.int32)
    ok.prefill_paged_mla(q_abs, np.array([0, nqs[0], total], np.int32), pages, page_indptr, page_ids, last, out, lse,
                         1, sm, d_latent=d_lat)
    cursor = 0
    for b, nq in enumerate(nqs):
        k_full, v_full = cf.mla_expand(latents[b], w_kv, h, d_nope, d_v)
        eo, el = cf.attention(qs[b], k_full, v_full, sm, causal=True)
        got = np.einsum("qhl,lhv->qhv", out[cursor:cursor + nq].astype(np.float64), w_uv)
        assert_close(got, eo, atol=1e-2, rtol=1e-2, what=f"causal mla out, seq {b}")
        assert_close(lse[cursor:cursor + nq], el, atol=2e-2, rtol=1e-3, what=f"causal mla lse, seq {b}")
        cursor += nq
    # the first query row of sequence 1 sees exactly one cached row: its value comes back
    first = out[nqs[0]].astype(np.float64)
    assert_close(first, np.broadcast_to(latents[1][0, :d_lat].astype(np.float64), first.shape), atol=2e-3, rtol=2e-3,
                 what="a row that sees one key returns that key's latent")


# ------------------------------------------------------------------------ RoPE frequency variants
LLAMA3 = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
YARN = {"rope_type": "yarn", "factor": 40.0, "beta_fast": 32, "beta_slow": 1, "original_max_position_embeddings": 4096}


def test_llama3_angles_match_the_published_piecewise_rule():
    """Llama-3.1's rule as published with the model: frequencies whose wavelength is below
    original_max / high_freq_factor stay, those above original_max / low_freq_factor are divided by
    `factor`, those in between blend linearly in original_max / wavelength.  float64 numpy, a
    different structure (where / masks) from the reference's clip expression."""
    D, theta = 128, 5e5
    i = np.arange(D // 2, dtype=np.float64)
    inv_freq = 1.0 / theta ** (2 * i / D)
    wavelen = 2 * np.pi / inv_freq
    old, low, high, factor = 8192.0, 1.0, 4.0, 8.0
    expect = np.where(wavelen > old / low, inv_freq / factor, inv_freq)
    smooth = (old / wavelen - low) / (high - low)
    medium = ~(wavelen < old / high) & ~(wavelen > old / low)
    expect = np.where(medium, (1 - smooth) * inv_freq / factor + smooth * inv_freq, expect)
    assert medium.any() and (wavelen > old / low).any() and (wavelen < old / high).any()
    pos = 1000.0
    for d in range(D):
        angle, mag = ok.rope_angle(LLAMA3, pos, d, D, theta)
        assert mag == 1.0
        np.testing.assert_allclose(angle, pos * expect[d % (D // 2)], rtol=2e-6)


def test_yarn_angles_match_the_published_blend_without_rounding():
    """YaRN as published (find_correction_dim, linear ramp, blend of interpolated and extrapolated
    frequencies) with the two deviations of the reference: the correction dims are not floored / ceiled
    (position_embedding.py:203-217) and the ramp is indexed by the element, so the upper half of the
    head (d >= D/2) gets the ramp value of d, not of d - D/2 (:244-247)."""
    D, theta = 128, 1e4
    factor, beta_fast, beta_slow, orig = 40.0, 32.0, 1.0, 4096.0

    def correction_dim(rot):
        return D * np.log(orig / (rot * 2 * np.pi)) / (2 * np.log(theta))

    low, high = max(correction_dim(beta_fast), 0.0), min(correction_dim(beta_slow), D - 1.0)
    d = np.arange(D, dtype=np.float64)
    pos_freqs = theta ** ((2 * d % D) / D)
    ramp = np.clip((d - low) / (high - low), 0, 1)
    expect = (1.0 / (factor * pos_freqs)) * ramp + (1.0 / pos_freqs) * (1 - ramp)
    assert 0 < low < high < D / 2  # the ramp is inside the lower half; the upper half is fully interpolated
    pos = 777.0
    for e in range(D):
        angle, mag = ok.rope_angle(YARN, pos, e, D, theta)
        assert mag == 1.0
        np.testing.assert_allclose(angle, pos * expect[e], rtol=3e-6)
    # every element of the upper half is interpolated: its angle is the default one over `factor`
    for e in (D // 2, D // 2 + 5, D - 1):
        plain, _ = ok.rope_angle({}, pos, e, D, theta)
        np.testing.assert_allclose(ok.rope_angle(YARN, pos, e, D, theta)[0], plain / factor, rtol=3e-6)


def test_rope_variants_reduce_to_default():
    D, theta = 64, 1e4
    rng = np.random.default_rng(3)
    n, hq, hkv = 6, 4, 2
    qkv = rng.standard_normal((n, hq + 2 * hkv, D)).astype(np.float16)
    pos = np.array([0, 1, 17, 300, 4095, 70000], np.int32)

    def run(scaling, ext=None, apply_rope=1):
        q, k, v = np.zeros((n, hq, D), np.float16), np.zeros((n, hkv, D), np.float16), np.zeros((n, hkv, D), np.float16)
        ok.fused_rope_scaled(qkv, pos, q, k, v, apply_rope, scaling, theta=theta, ext_factors=ext)
        return q, k, v

    eq, ek, ev = np.zeros((n, hq, D), np.float16), np.zeros((n, hkv, D), np.float16), np.zeros((n, hkv, D), np.float16)
    ok.fused_rope(qkv, pos, eq, ek, ev, 1, theta=theta)
    # no scaling, and longrope with unit factors and no extension: bit for bit the plain kernel
    for scaling, ext in (({}, None), ({"rope_type": "longrope", "max_position_embeddings": 4096,
                                       "original_max_position_embeddings": 4096}, np.ones(D, np.float32))):
        q, k, v = run(scaling, ext)
        assert np.array_equal(q, eq) and np.array_equal(k, ek) and np.array_equal(v, ev)
    # yarn with factor 1 and llama3 with factor 1 are the plain frequencies up to float32 rounding
    for scaling in (dict(YARN, factor=1.0), dict(LLAMA3, factor=1.0)):
        q, k, v = run(scaling)
        assert np.array_equal(v, ev)
        assert_close(q, eq, atol=2e-2, rtol=1e-2, what="factor-1 scaling q")  # angles of ~7e4 rad carry ~1e-2 abs error in float32
        assert np.mean(q == eq) > 0.9
    # apply_rope = 0 copies
    q, k, v = run(LLAMA3, apply_rope=0)
    assert np.array_equal(q, qkv[:, :hq]) and np.array_equal(k, qkv[:, hq:hq + hkv])


@pytest.mark.parametrize("d,rotary_dim", [(128, 32), (128, 64), (64, 16), (128, 40), (128, 128)])
def test_partial_rotation_is_the_closed_form_on_the_first_features(d, rotary_dim):
    """rotary_dim < head_dim (python/tvm/relax/frontend/nn/llm/position_embedding.py:507-520): the first
    rotary_dim features rotate as a head of that width would (the reference test's closed form on that slice,
    pairs (i, i + rotary_dim/2), frequencies over rotary_dim), the others pass through bit for bit."""
    rng = np.random.default_rng(90 + rotary_dim)
    hq, hkv = 4, 2
    pos = np.array([0, 1, 17, 511, 2047, 4096], np.int32)
    n = len(pos)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    q, k, v = np.zeros((n, hq, d), F16), np.zeros((n, hkv, d), F16), np.zeros((n, hkv, d), F16)
    ok.fused_rope_scaled(qkv, pos, q, k, v, 1, {"rope_type": "default", "rotary_dim": rotary_dim})
    assert np.array_equal(v, qkv[:, hq + hkv:])
    for got, src in ((q, qkv[:, :hq]), (k, qkv[:, hq:hq + hkv])):
        assert np.array_equal(got[..., rotary_dim:], src[..., rotary_dim:])
        want = cf.apply_rotary(src[..., :rotary_dim], pos)
        assert_close(got[..., :rotary_dim], want, atol=2e-3, rtol=2e-3, what=f"partial rotation, {rotary_dim} of {d}")
    if rotary_dim == d:  # the whole head: the plain kernel (to one fp16 ulp: the two loops round in different places)
        q2, k2, v2 = np.zeros_like(q), np.zeros_like(k), np.zeros_like(v)
        ok.fused_rope(qkv, pos, q2, k2, v2, 1)
        assert_close(q, q2, atol=1e-3, rtol=1e-3, what="whole-head rotary_dim q")
        assert_close(k, k2, atol=1e-3, rtol=1e-3, what="whole-head rotary_dim k")


@pytest.mark.parametrize("d,rotary_dim", [(128, 128), (128, 64), (64, 32)])
def test_gptj_pairing_is_the_default_rotation_of_the_deinterleaved_head(d, rotary_dim):
    """rope_type gptj (position_embedding.py:70-76, 509-514) rotates the pairs (2i, 2i + 1) at the frequency the
    default rule gives pair i: moving the even features to the front and the odd ones behind them turns it into
    the default rotation, so the reference test's closed form on the permuted slice pins it."""
    rng = np.random.default_rng(95 + rotary_dim)
    hq, hkv = 4, 2
    pos = np.array([0, 1, 17, 511, 2047, 4096], np.int32)
    n = len(pos)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    q, k, v = np.zeros((n, hq, d), F16), np.zeros((n, hkv, d), F16), np.zeros((n, hkv, d), F16)
    ok.fused_rope_scaled(qkv, pos, q, k, v, 1, {"rope_type": "gptj", "rotary_dim": rotary_dim})
    assert np.array_equal(v, qkv[:, hq + hkv:])
    for got, src in ((q, qkv[:, :hq]), (k, qkv[:, hq:hq + hkv])):
        assert np.array_equal(got[..., rotary_dim:], src[..., rotary_dim:])
        part = src[..., :rotary_dim]
        rotated = cf.apply_rotary(np.concatenate([part[..., 0::2], part[..., 1::2]], axis=-1), pos)
        want = np.empty_like(rotated)
        want[..., 0::2], want[..., 1::2] = rotated[..., :rotary_dim // 2], rotated[..., rotary_dim // 2:]
        assert_close(got[..., :rotary_dim], want, atol=2e-3, rtol=2e-3, what=f"gptj rotation, {rotary_dim} of {d}")


def test_llama4_is_the_llama3_rule_on_the_frequency_of_pair_d_over_2():
    """rope_freq_llama4 (position_embedding.py:79-127) smooths like llama3 but takes the frequency of pair d // 2
    (no wrap at the half): element d gets the angle llama3 gives element d // 2.  With equal low and high factors it
    is a hard threshold on the wavelength: frequencies whose wavelength exceeds original_max / low_freq_factor are
    divided by the factor, the others kept."""
    theta, r = 5e5, 128
    sc = {"rope_type": "llama4", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
    l3 = dict(sc, rope_type="llama3")
    for d in range(r):
        a4, m4 = ok.rope_angle(sc, 1234.0, d, r, theta)
        a3, _ = ok.rope_angle(l3, 1234.0, d // 2, r, theta)
        assert m4 == 1.0 and a4 == a3, d
    hard = dict(sc, high_freq_factor=1.0)
    for d in range(r):
        orig = np.float32(1.0) / np.float32(theta) ** (np.float32(2 * (d // 2)) / np.float32(r))
        wavelength = 2 * np.pi / orig
        a, _ = ok.rope_angle(hard, 100.0, d, r, theta)
        want = 100.0 * (orig / 8.0 if wavelength > 8192 else orig)
        assert abs(a - want) <= 1e-5 * abs(want), d


def test_longrope_factors_and_magnitude():
    """The angle is the default one over the factor of the dimension; cos and sin carry
    sqrt(1 + ln(max/orig)/ln(orig)); the long factors apply only to calls with more rows than orig."""
    D, theta = 64, 1e4
    scaling = {"rope_type": "longrope", "max_position_embeddings": 131072, "original_max_position_embeddings": 4}
    ext = np.concatenate([np.linspace(1.0, 4.0, D // 2), np.linspace(1.0, 1.5, D // 2)]).astype(np.float32)
    plain, _ = ok.rope_angle({}, 33.0, 7, D, theta)
    angle, mag = ok.rope_angle(scaling, 33.0, 7, D, theta, ext[:D // 2])
    np.testing.assert_allclose(angle, plain / ext[7], rtol=1e-6)
    np.testing.assert_allclose(mag, np.sqrt(1 + np.log(131072 / 4) / np.log(4)), rtol=1e-6)
    angle_hi, _ = ok.rope_angle(scaling, 33.0, 7 + D // 2, D, theta, ext[:D // 2])
    assert angle_hi == angle  # both halves of a pair share the factor (index d mod D/2)
    rng = np.random.default_rng(4)
    hq, hkv = 2, 1
    for n, half in ((3, ext[D // 2:]), (5, ext[:D // 2])):  # 3 rows <= orig: short factors; 5 rows > orig: long
        qkv = rng.standard_normal((n, hq + 2 * hkv, D)).astype(np.float16)
        pos = np.arange(10, 10 + n, dtype=np.int32)
        q, k, v = np.zeros((n, hq, D), np.float16), np.zeros((n, hkv, D), np.float16), np.zeros((n, hkv, D), np.float16)
        ok.fused_rope_scaled(qkv, pos, q, k, v, 1, scaling, theta=theta, ext_factors=ext)
        x = qkv[:, 0].astype(np.float64)
        i = np.arange(D // 2)
        ang = pos[:, None].astype(np.float64) / (half.astype(np.float64) * theta ** (2 * i / D))
        m = np.sqrt(1 + np.log(131072 / 4) / np.log(4))
        lo = m * (np.cos(ang) * x[:, :D // 2] - np.sin(ang) * x[:, D // 2:])
        hi = m * (np.cos(ang) * x[:, D // 2:] + np.sin(ang) * x[:, :D // 2])
        assert_close(q[:, 0], np.concatenate([lo, hi], axis=1).astype(np.float16), atol=2e-3, rtol=2e-3, what="longrope q")


# ------------------------------------------------- frequency variants inside the attention kernels
LONGROPE = {"rope_type": "longrope", "max_position_embeddings": 131072, "original_max_position_embeddings": 4096}
GPTJ = {"rope_type": "gptj"}
LLAMA4 = {"rope_type": "llama4", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}


def rotate_whole_head(x, positions, rope_scaling, theta=1e4, scale=1.0):
    """What the reference's attention kernels do to a row before they use it (_kernel_common.py:115-127):
    element d of the WHOLE head gets cos * x[d] + sin * (-x[d + D/2] or x[d - D/2]) at the angle the variant
    gives element d (ok.rope_angle, pinned above), rounded to fp16.  x: (rows, heads, D)."""
    rows, heads, D = x.shape
    out = np.zeros_like(x)
    xf = x.astype(np.float32)
    for r in range(rows):
        for d in range(D):
            angle, mag = ok.rope_angle(rope_scaling, np.float32(positions[r]) * np.float32(scale), d, D, theta)
            c = np.float32(np.cos(np.float32(angle))) * np.float32(mag)
            s_ = np.float32(np.sin(np.float32(angle))) * np.float32(mag)
            other = -xf[r, :, d + D // 2] if d < D // 2 else xf[r, :, d - D // 2]
            out[r, :, d] = (c * xf[r, :, d] + s_ * other).astype(np.float16)
    return out


@pytest.mark.parametrize("rope_scaling", [LLAMA3, YARN, LONGROPE, GPTJ, LLAMA4], ids=lambda sc: sc["rope_type"])
def test_inline_rope_variants_equal_attention_over_rotated_rows(rope_scaling):
    """The oracle's attention kernels with rotary_mode = 1 and a frequency variant in force equal the same kernels
    with rotary_mode = 0 on rows rotated beforehand: decode (keys at k_rope_pos_offset + t, the query at its
    position) and the ragged kernel (queries and keys of a chunk)."""
    rng = np.random.default_rng(123)
    hq, hkv, d, ps = 4, 2, 64, 16
    kv_lens = [37, 5]
    pages, ip, pv, last, ks, vs = build_paged_kv(rng, kv_lens, 6, hkv, ps, d)
    k_off = np.array([100, 3], np.int32)
    q_pos = np.array([100 + 36, 3 + 4], np.int32)
    q = rng.standard_normal((2, hq, d)).astype(F16)
    z = np.zeros(2, np.int32)
    inline_o, inline_l = np.zeros((2, hq, d), F16), np.zeros((2, hq), np.float32)
    with ok.inline_rope_scaling(rope_scaling):
        ok.decode(q, pages, ip, pv, last, k_off, q_pos, inline_o, inline_l, 1, 1.0, 1e4, d ** -0.5)
    rotated_pages = pages.copy()
    for b, n in enumerate(kv_lens):
        rk = rotate_whole_head(ks[b], k_off[b] + np.arange(n), rope_scaling)
        for t in range(n):
            rotated_pages[pv[ip[b] + t // ps], 0, :, t % ps] = rk[t]
    rq = rotate_whole_head(q, q_pos, rope_scaling)
    plain_o, plain_l = np.zeros_like(inline_o), np.zeros_like(inline_l)
    ok.decode(rq, rotated_pages, ip, pv, last, z, z, plain_o, plain_l, 0, 1.0, 1e4, d ** -0.5)
    assert_close(inline_o, plain_o, atol=2e-3, rtol=2e-3, what="decode, inline variant vs rotated rows")
    assert_close(inline_l, plain_l, atol=2e-3, rtol=1e-4, what="decode lse")
    # the variant really changes something (or, for magnitude-only longrope, scales the scores)
    default_o = np.zeros_like(inline_o)
    default_l = np.zeros_like(inline_l)
    ok.decode(q, pages, ip, pv, last, k_off, q_pos, default_o, default_l, 1, 1.0, 1e4, d ** -0.5)
    assert np.abs(default_l - inline_l).max() > 1e-3
    # ragged
    lens = [9, 20]
    n = sum(lens)
    ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    qr = rng.standard_normal((n, hq, d)).astype(F16)
    kr = rng.standard_normal((n, hkv, d)).astype(F16)
    vr = rng.standard_normal((n, hkv, d)).astype(F16)
    off = np.array([50, 7], np.int32)
    pos = np.concatenate([off[i] + np.arange(lens[i]) for i in range(2)]).astype(np.int32)
    io, il = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    with ok.inline_rope_scaling(rope_scaling):
        ok.prefill_ragged(qr, ind, kr, vr, ind, pos, off, io, il, 1, 1, 1.0, 1e4, d ** -0.5)
    po, pl = np.zeros_like(io), np.zeros_like(il)
    ok.prefill_ragged(rotate_whole_head(qr, pos, rope_scaling), ind, rotate_whole_head(kr, pos, rope_scaling), vr, ind,
                      np.zeros(n, np.int32), z, po, pl, 1, 0, 1.0, 1e4, d ** -0.5)
    assert_close(io, po, atol=2e-3, rtol=2e-3, what="ragged, inline variant vs rotated rows")
    assert_close(il, pl, atol=2e-3, rtol=1e-4, what="ragged lse")
