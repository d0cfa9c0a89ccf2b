"""Pins the oracle's float32-storage build (oracle/kv_kernels.c compiled with -DORC_F32) and its kernels at page
sizes that are not a power of two.

The reference builds its kernels per storage dtype and page size; its own tests run float32 storage
(tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:269-276).  Expected values come from
oracle/closed_form.py (float64 numpy) and from special cases; with float32 storage the only roundings are those of
float32 arithmetic, so the tolerances are a hundred times tighter than for fp16 storage: a dropped cast, a
conversion left in from the fp16 build or a wrong sign in the rotation fails them.
"""
import numpy as np
import pytest

from oracle import closed_form as cf
from oracle import kernels as ok
from tests.util import REFERENCE_TREES, assert_close, build_paged_kv, random_forest, tree_order

F32 = np.float32


def test_rope_f32_matches_closed_form_and_is_a_plain_split_for_v():
    rng = np.random.default_rng(200)
    hq, hkv, d = 8, 2, 128
    positions = np.array([0, 1, 2, 17, 2047, 4095], np.int32)
    n = len(positions)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F32)
    q, k, v = np.zeros((n, hq, d), F32), np.zeros((n, hkv, d), F32), np.zeros((n, hkv, d), F32)
    ok.fused_rope(qkv, positions, q, k, v, 1)
    # float32 angles at positions up to 4095: ulp(4095) = 2.4e-4 rad on values up to ~4
    assert_close(q, cf.apply_rotary(qkv[:, :hq], positions), atol=2e-3, rtol=1e-5, what="q rope f32")
    assert_close(k, cf.apply_rotary(qkv[:, hq:hq + hkv], positions), atol=2e-3, rtol=1e-5, what="k rope f32")
    small = positions < 32
    assert_close(q[small], cf.apply_rotary(qkv[small][:, :hq], positions[small]), atol=2e-5, rtol=1e-5, what="q rope f32, small angles")
    assert np.array_equal(v, qkv[:, hq + hkv:])
    ok.fused_rope(qkv, np.zeros(n, np.int32), q, k, v, 1)
    assert np.array_equal(q, qkv[:, :hq]) and np.array_equal(k, qkv[:, hq:hq + hkv])


@pytest.mark.parametrize("ps", [16, 5, 24])
def test_append_gather_copy_round_trip_f32(ps):
    rng = np.random.default_rng(201)
    hkv, d, npages = 3, 64, 7
    pages = np.zeros((npages, 2, hkv, ps, d), F32)
    n = 2 * ps + 3
    k, v = (rng.standard_normal((n, hkv, d)).astype(F32) for _ in range(2))
    slots = rng.permutation(npages * ps)[:n].astype(np.int32)
    slots[3] = -1
    ok.transpose_append(pages, k, v, slots)
    keep = slots >= 0
    gk, gv = np.zeros((1, keep.sum(), hkv, d), F32), np.zeros((1, keep.sum(), hkv, d), F32)
    ok.debug_get_kv(pages, slots[keep], gk, gv, 0)
    assert np.array_equal(gk[0], k[keep]) and np.array_equal(gv[0], v[keep])
    assert np.count_nonzero(pages) == np.count_nonzero(k[keep]) + np.count_nonzero(v[keep])
    before = pages.copy()
    ok.copy_single_page(pages, 1, 4, ps - 2)
    assert np.array_equal(pages[4][:, :, :ps - 2], before[1][:, :, :ps - 2])
    assert np.array_equal(pages[4][:, :, ps - 2:], before[4][:, :, ps - 2:])


@pytest.mark.parametrize("dtype,ps,tol", [(F32, 16, 2e-5), (F32, 7, 2e-5), (np.float16, 24, 2e-3), (np.float16, 1, 2e-3)])
def test_decode_and_paged_prefill_match_closed_form(dtype, ps, tol):
    rng = np.random.default_rng(202)
    hq, hkv, d = 8, 2, 64
    kv_lens = [1, ps - 1 if ps > 1 else 2, ps, ps + 1, 100, 0]
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, kv_lens, 4 + sum((n + ps - 1) // ps for n in kv_lens), hkv, ps, d,
                                                       dtype=dtype)
    b = len(kv_lens)
    q = rng.standard_normal((b, hq, d)).astype(dtype)
    out, lse = np.zeros((b, hq, d), dtype), np.zeros((b, hq), F32)
    z = np.zeros(b, np.int32)
    ok.decode(q, pages, indptr, values, last, z, z, out, lse, 0, 1.0, 1e4, d ** -0.5)
    for i, n in enumerate(kv_lens):
        if n == 0:
            assert not out[i].any() and np.all(lse[i] == F32(-5e4))
            continue
        eo, el = cf.attention(q[i:i + 1], ks[i], vs[i], d ** -0.5, causal=False)
        assert_close(out[i], eo[0], atol=tol, rtol=tol, what=f"decode out seq {i}")
        assert_close(lse[i], el[0], atol=max(tol, 1e-4), rtol=1e-5, what=f"decode lse seq {i}")
    q_lens = [1, 2, 3, ps + 1, 30, 2]
    kv2 = [max(k, ql) for k, ql in zip(kv_lens, q_lens)]
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, kv2, 4 + sum((n + ps - 1) // ps for n in kv2), hkv, ps, d, dtype=dtype)
    n = sum(q_lens)
    qindptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(dtype)
    for causal in (0, 1):
        out, lse = np.zeros((n, hq, d), dtype), np.zeros((n, hq), F32)
        ok.prefill_paged(q, qindptr, pages, indptr, values, last, z, np.zeros(n, np.int32), out, lse, causal, 0, 1.0, 1e4, d ** -0.5)
        for i in range(b):
            s, e = qindptr[i], qindptr[i + 1]
            eo, el = cf.attention(q[s:e], ks[i], vs[i], d ** -0.5, causal=bool(causal))
            assert_close(out[s:e], eo, atol=tol, rtol=tol, what=f"paged out seq {i} causal {causal}")
            assert_close(lse[s:e], el, atol=max(tol, 1e-4), rtol=1e-5, what=f"paged lse seq {i} causal {causal}")


def test_ragged_tree_and_merge_f32_match_closed_forms():
    rng = np.random.default_rng(203)
    hq, hkv, d = 8, 2, 128
    lens = [1, 5, 33, 16]
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F32) for h in (hq, hkv, hkv))
    out, lse = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
    ok.prefill_ragged(q, indptr, k, v, indptr, np.zeros(n, np.int32), np.zeros(len(lens), np.int32), out, lse, 1, 0, 1.0, 1e4,
                      d ** -0.5)
    for i in range(len(lens)):
        s, e = indptr[i], indptr[i + 1]
        eo, el = cf.attention(q[s:e], k[s:e], v[s:e], d ** -0.5, causal=True)
        assert_close(out[s:e], eo, atol=2e-5, rtol=2e-5, what=f"ragged out seq {i}")
        assert_close(lse[s:e], el, atol=1e-4, rtol=1e-5, what=f"ragged lse seq {i}")
    assert np.array_equal(out[0], np.repeat(v[0], hq // hkv, axis=0))   # the first row sees only itself
    # token trees
    trees = REFERENCE_TREES + [random_forest(rng, 40)]
    tl = [len(t) for t in trees]
    n = sum(tl)
    ind = np.concatenate([[0], np.cumsum(tl)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F32) for h in (hq, hkv, hkv))
    mask = np.concatenate([tree_order(t) for t in trees])
    out, lse = np.zeros((n, hq, d), F32), np.zeros((n, hq), F32)
    ok.tree_attn_ragged(q, ind, k, v, ind, np.zeros(n, np.int32), ind, mask, out, lse, 0, 1.0, 1e4, d ** -0.5)
    for i, parents in enumerate(trees):
        s, e = ind[i], ind[i + 1]
        eo, el = cf.attention(q[s:e], k[s:e], v[s:e], d ** -0.5, mask=cf.tree_ancestor_mask(parents))
        assert_close(out[s:e], eo, atol=2e-5, rtol=2e-5, what=f"tree out seq {i}")
        assert_close(lse[s:e], el, atol=1e-4, rtol=1e-5, what=f"tree lse seq {i}")
    # merge: the two-way log-sum-exp identity, an empty side, equal weights
    nrow, h = 6, 4
    v1, v2 = (rng.standard_normal((nrow, h, d)).astype(F32) for _ in range(2))
    s1, s2 = ((rng.standard_normal((nrow, h)) * 3).astype(F32) for _ in range(2))
    s2[0] = -5e4
    s2[1] = s1[1]
    ev, es = cf.merge(v1, s1, v2, s2)
    mv, ms = v1.copy(), s1.copy()
    ok.merge_state_inplace(mv, ms, v2, s2)
    assert_close(mv, ev, atol=1e-5, rtol=1e-5, what="merge v f32")
    assert_close(ms, es, atol=1e-5, rtol=1e-6, what="merge s f32")
    assert np.array_equal(mv[0], v1[0])
    assert_close(mv[1], (v1[1].astype(np.float64) + v2[1]) / 2, atol=1e-6, rtol=1e-6)


def test_tree_attn_paged_f32_and_odd_page_size():
    from tests.test_oracle_kernels import tree_paged_case
    rng = np.random.default_rng(204)
    hq, hkv, d = 8, 2, 64
    prefix = [10, 20, 0]
    trees = [REFERENCE_TREES[0], REFERENCE_TREES[1], random_forest(rng, 30)]
    new_lens = [7, 8, 30]
    for dtype, ps, tol in ((F32, 16, 2e-5), (np.float16, 12, 2e-3)):
        kv_lens = [p + len(t) for p, t in zip(prefix, trees)]
        pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, kv_lens, 16, hkv, ps, d, dtype=dtype)
        qindptr = np.concatenate([[0], np.cumsum(new_lens)]).astype(np.int32)
        q = rng.standard_normal((int(qindptr[-1]), hq, d)).astype(dtype)
        tindptr = np.concatenate([[0], np.cumsum([len(t) for t in trees])]).astype(np.int32)
        labels = np.concatenate([tree_order(t) for t in trees])
        out, lse = np.zeros_like(q), np.zeros(q.shape[:2], F32)
        zb = np.zeros(len(trees), np.int32)
        ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, np.zeros(len(q), np.int32), out, lse, 0, 1.0, 1e4,
                           d ** -0.5, tindptr, labels)
        for i, (p, t, nq) in enumerate(zip(prefix, trees, new_lens)):
            m = np.ones((nq, p + len(t)), bool)
            m[:, p:] = cf.tree_ancestor_mask(t)[len(t) - nq:]
            s, e = qindptr[i], qindptr[i + 1]
            eo, el = cf.attention(q[s:e], ks[i], vs[i], d ** -0.5, mask=m)
            assert_close(out[s:e], eo, atol=tol, rtol=tol, what=f"tree paged out seq {i} {dtype.__name__}")
            assert_close(lse[s:e], el, atol=max(tol, 1e-4), rtol=1e-5, what=f"tree paged lse seq {i}")


def test_inline_rope_variant_and_sliding_cache_in_the_f32_build():
    """rotary_mode 1 with a frequency variant and the (3, batch) length_info of a sliding-window cache in the float32
    build: the variant is a library setting that both builds must receive (without it the float32 build rotates
    with the default frequencies), and the float32 build must agree with the fp16 build on the same values up to
    the fp16 roundings of that build."""
    rng = np.random.default_rng(210)
    hq, hkv, d, ps = 8, 2, 64, 16
    spec = [(100, 4, 20), (57, 0, 0), (33, 2, 2)]  # physical length, sink, window offset
    pages, indptr, values, last, _, _ = build_paged_kv(rng, [x[0] for x in spec], 16, hkv, ps, d, dtype=F32)
    info = np.array([last, [x[2] for x in spec], [x[1] for x in spec]], np.int32)
    b = len(spec)
    q = rng.standard_normal((b, hq, d)).astype(F32)
    k_off = np.array([0, 300, 4000], np.int32)
    q_pos = (k_off + np.array([n - off + sink for n, sink, off in spec]) - 1).astype(np.int32)
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 64}
    outs = {}
    for name, sc in (("default", None), ("llama3", scaling)):
        with ok.inline_rope_scaling(sc):
            o32, l32 = np.zeros((b, hq, d), F32), np.zeros((b, hq), F32)
            ok.decode(q, pages, indptr, values, info, k_off, q_pos, o32, l32, 1, 1.0, 1e4, d ** -0.5)
            o16, l16 = np.zeros((b, hq, d), np.float16), np.zeros((b, hq), F32)
            ok.decode(q.astype(np.float16), pages.astype(np.float16), indptr, values, info, k_off, q_pos, o16, l16, 1, 1.0, 1e4,
                      d ** -0.5)
        assert_close(o32, o16, atol=1e-2, rtol=1e-2, what=f"f32 build vs fp16 build, {name}")
        assert_close(l32, l16, atol=5e-2, rtol=1e-3, what=f"f32 build vs fp16 build lse, {name}")
        outs[name] = o32
    # the variant changes the result: long positions rotate differently
    assert np.abs(outs["default"] - outs["llama3"]).max() > 1e-2
