"""GPU parity of every HIP kernel launcher against the CPU oracle on identical seeded inputs.

Integer/byte work (append scatter, gathers, page copies) must be bit-exact; attention outputs
are fp16 with fp32 accumulation and must agree within atol = rtol = 1e-2 (the tolerance the
path is specified to); RoPE outputs are compared at one fp16 ulp."""
import ctypes

import numpy as np
import pytest
import torch

import tvm_amd
from oracle import kernels as ok
from tests.gpu_util import DEV, dev, host, i32
from tests.util import ATOL, RTOL, assert_close, assert_close_where_keys, build_paged_kv, rows_without_keys
from tvm_amd import KVError
from tvm_amd import kernels as K

pytestmark = pytest.mark.gpu
F16 = np.float16


# ------------------------------------------------------------------------------ RoPE / append
@pytest.mark.parametrize("d,hq,hkv", [(128, 32, 8), (64, 8, 2), (256, 4, 4), (80, 8, 2), (96, 32, 8), (112, 4, 4)])
@pytest.mark.parametrize("apply_rope", [1, 0])
def test_fused_rope(d, hq, hkv, apply_rope):
    rng = np.random.default_rng(0)
    pos = np.array([0, 1, 2, 3, 100, 511, 2047, 4096, 65535, 131071, 7, 9, 33], np.int32)
    n = len(pos)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    eq, ek, ev = np.zeros((n, hq, d), F16), np.zeros((n, hkv, d), F16), np.zeros((n, hkv, d), F16)
    ok.fused_rope(qkv, pos, eq, ek, ev, apply_rope)
    q, k, v = (torch.zeros(a.shape, dtype=torch.float16, device=DEV) for a in (eq, ek, ev))
    K.fused_rope(dev(qkv), i32(pos), q, k, v, apply_rope, 1.0, 1e4)
    assert np.array_equal(host(v), ev)
    if not apply_rope:
        assert np.array_equal(host(q), eq) and np.array_equal(host(k), ek)
        return
    # same fp32 formula on both sides; device cos/sin may differ from libm in the last ulp, which
    # can flip the fp16 rounding: allow one fp16 ulp (2^-10 relative) plus fp16 denormal spacing
    assert_close(host(q), eq, atol=1e-3, rtol=2e-3, what="rope q")
    assert_close(host(k), ek, atol=1e-3, rtol=2e-3, what="rope k")
    exact = np.mean(host(q) == eq)
    assert exact > 0.99, f"only {exact:.4f} of the rotated q elements are bit-identical to the oracle"


@pytest.mark.parametrize("rope_scaling", [
    {"rope_type": "default", "rotary_dim": 32}, {"rope_type": "default", "rotary_dim": 40},
    {"rope_type": "gptj", "rotary_dim": 64}, {"rope_type": "gptj", "rotary_dim": 32},
    {"rope_type": "llama4", "rotary_dim": 64, "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
     "original_max_position_embeddings": 8192},
    {"rope_type": "llama4", "rotary_dim": 64, "factor": 16.0, "low_freq_factor": 1.0, "high_freq_factor": 1.0,
     "original_max_position_embeddings": 8192},
    {"rope_type": "llama3", "rotary_dim": 64, "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
     "original_max_position_embeddings": 8192},
    {"rope_type": "yarn", "rotary_dim": 64, "factor": 40.0, "beta_fast": 32, "beta_slow": 1,
     "original_max_position_embeddings": 4096}])
@pytest.mark.parametrize("d", [128, 64])
def test_fused_rope_partial_rotation(d, rope_scaling):
    """rotary_dim < head_dim: only the first features rotate (position_embedding.py:507-520), with any
    frequency variant; the rest of q and k, and v, pass through bit for bit."""
    rng = np.random.default_rng(91)
    hq, hkv = 8, 2
    r = rope_scaling["rotary_dim"]
    pos = np.array([0, 1, 2, 3, 100, 511, 2047, 4096, 65535, 7, 9, 33], np.int32)
    n = len(pos)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    eq, ek, ev = np.zeros((n, hq, d), F16), np.zeros((n, hkv, d), F16), np.zeros((n, hkv, d), F16)
    ok.fused_rope_scaled(qkv, pos, eq, ek, ev, 1, rope_scaling)
    q, k, v = (torch.full(a.shape, 7.0, dtype=torch.float16, device=DEV) for a in (eq, ek, ev))
    K.fused_rope_scaled(dev(qkv), i32(pos), q, k, v, 1, rope_scaling)
    assert np.array_equal(host(v), ev)
    assert np.array_equal(host(q)[..., r:], qkv[:, :hq, r:]) and np.array_equal(host(k)[..., r:], qkv[:, hq:hq + hkv, r:])
    assert_close(host(q), eq, atol=1e-3, rtol=2e-3, what="partial rope q")
    assert_close(host(k), ek, atol=1e-3, rtol=2e-3, what="partial rope k")


def test_fused_rope_append_equals_rope_then_append():
    """One launch for split + RoPE + append: bit-identical q, k, v and pages to the two kernels."""
    rng = np.random.default_rng(42)
    hq, hkv, d, ps, npages, n = 32, 8, 128, 16, 12, 70
    qkv = dev(rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16))
    pos = i32(rng.integers(0, 5000, size=n))
    slots = rng.permutation(npages * ps)[:n].astype(np.int32)
    slots[[3, 17]] = -1
    pages0 = rng.standard_normal((npages, 2, hkv, ps, d)).astype(F16)
    outs = []
    for fused in (False, True):
        q = torch.zeros((n, hq, d), dtype=torch.float16, device=DEV)
        k = torch.zeros((n, hkv, d), dtype=torch.float16, device=DEV)
        v = torch.zeros((n, hkv, d), dtype=torch.float16, device=DEV)
        pages = dev(pages0)
        if fused:
            K.fused_rope_append(qkv, pos, q, k, v, 1, pages, i32(slots), 1.0, 1e4)
        else:
            K.fused_rope(qkv, pos, q, k, v, 1, 1.0, 1e4)
            K.tir_kv_cache_transpose_append(pages, k, v, i32(slots))
        outs.append([host(t) for t in (q, k, v, pages)])
    for a, b, name in zip(outs[0], outs[1], ("q", "k", "v", "pages")):
        assert np.array_equal(a, b), name


def test_transpose_append_bit_exact_with_skips():
    rng = np.random.default_rng(1)
    hkv, ps, d, npages, n = 8, 16, 128, 64, 300
    pages0 = rng.standard_normal((npages, 2, hkv, ps, d)).astype(F16)
    slots = rng.permutation(npages * ps)[:n].astype(np.int32)
    slots[[3, 77, 299]] = -1
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    expect = pages0.copy()
    ok.transpose_append(expect, k, v, slots)
    pages = dev(pages0)
    K.tir_kv_cache_transpose_append(pages, dev(k), dev(v), i32(slots))
    assert np.array_equal(host(pages), expect)
    # gather back
    keep = slots[slots >= 0]
    kd = torch.zeros((3, len(keep), hkv, d), dtype=torch.float16, device=DEV)
    vd = torch.zeros_like(kd)
    K.tir_kv_cache_debug_get_kv(pages, i32(keep), kd, vd, 2)
    assert np.array_equal(host(kd)[2], k[slots >= 0]) and np.array_equal(host(vd)[2], v[slots >= 0])
    assert not host(kd)[:2].any()
    K.tir_kv_cache_transpose_append(pages, dev(k[:0]), dev(v[:0]), i32(slots[:0]))  # empty append is a no-op
    assert np.array_equal(host(pages), expect)


def test_transpose_append_mla_and_gather_bit_exact():
    rng = np.random.default_rng(2)
    ps, d, npages, n = 64, 576, 6, 200
    pages0 = rng.standard_normal((npages, ps, d)).astype(F16)
    slots = rng.permutation(npages * ps)[:n].astype(np.int32)
    slots[0] = -1
    kv = rng.standard_normal((n, d)).astype(F16)
    expect = pages0.copy()
    ok.transpose_append_mla(expect, kv, slots)
    pages = dev(pages0)
    K.tir_kv_cache_transpose_append_mla(pages, dev(kv), i32(slots))
    assert np.array_equal(host(pages), expect)
    out = torch.zeros((2, n - 1, d), dtype=torch.float16, device=DEV)
    K.tir_kv_cache_debug_get_kv_mla(pages, i32(slots[1:]), out, 1)
    assert np.array_equal(host(out)[1], kv[1:])


def test_copy_single_page_and_compact_copy_bit_exact():
    rng = np.random.default_rng(3)
    hkv, ps, d, npages = 8, 16, 128, 12
    pages0 = rng.standard_normal((npages, 2, hkv, ps, d)).astype(F16)
    expect = pages0.copy()
    pages = dev(pages0)
    for src, tgt, n in [(1, 3, 7), (0, 11, 16), (5, 6, 1), (2, 4, 0)]:
        ok.copy_single_page(expect, src, tgt, n)
        K.copy_single_page(pages, src, tgt, n)
    assert np.array_equal(host(pages), expect)
    indptr = np.array([0, 2, 2, 5], np.int32)
    src_dst = np.array([[20, 21, 70, 71, 72], [17, 20, 65, 70, 71]], np.int32)  # later dst = earlier src
    ok.compact_kv_copy(expect, indptr, src_dst, 3)
    K.compact_kv_copy(pages, i32(indptr), i32(src_dst), 3)
    assert np.array_equal(host(pages), expect)
    mla0 = rng.standard_normal((5, 64, 576)).astype(F16)
    em = mla0.copy()
    ok.copy_single_page_mla(em, 4, 1, 33)
    mp = dev(mla0)
    K.copy_single_page_mla(mp, 4, 1, 33)
    assert np.array_equal(host(mp), em)
    with pytest.raises(KVError, match="out of range"):
        K.copy_single_page(pages, 0, npages, 3)


# ------------------------------------------------------------------------------ merge
@pytest.mark.parametrize("h,d", [(32, 128), (8, 64), (128, 512), (8, 80), (32, 96), (4, 112), (3, 40)])
def test_merge_state_inplace(h, d):
    rng = np.random.default_rng(4)
    n = 37
    v1 = rng.standard_normal((n, h, d)).astype(F16)
    v2 = rng.standard_normal((n, h, d)).astype(F16)
    s1 = (rng.standard_normal((n, h)) * 4).astype(np.float32)
    s2 = (rng.standard_normal((n, h)) * 4).astype(np.float32)
    s2[0] = -5e4
    s1[1] = -5e4
    ev, es = v1.copy(), s1.copy()
    ok.merge_state_inplace(ev, es, v2, s2)
    gv, gs = dev(v1), dev(s1)
    K.merge_state_inplace(gv, gs, dev(v2), dev(s2))
    assert_close(host(gv), ev, atol=1e-3, rtol=1e-3, what="merge v")
    assert_close(host(gs), es, atol=1e-4, rtol=1e-6, what="merge s")
    assert np.array_equal(host(gv)[0], v1[0])  # empty other side leaves the row untouched


# ------------------------------------------------------------------------------ decode
def _decode_both(rng, kv_lens, hq, hkv, d, npages, scale=1.0, page_size=16):
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, kv_lens, npages, hkv, page_size, d, scale=scale)
    b = len(kv_lens)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
    z = np.zeros(b, np.int32)
    ok.decode(q, pages, indptr, values, last, z, z, eo, el, 0, 1.0, 1e4, d ** -0.5)
    go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_decode_paged_kv(dev(q), dev(pages), i32(indptr), i32(values), i32(last), i32(z), i32(z), go, gl, 0,
                            1.0, 1e4, d ** -0.5)
    return host(go), host(gl), eo, el


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (64, 8, 128), (8, 8, 128), (8, 4, 64), (16, 2, 64), (8, 2, 256),
                                      (16, 16, 256), (8, 2, 80), (32, 8, 96), (6, 2, 112), (32, 1, 96), (40, 1, 80)])
def test_decode_ragged_lengths_against_oracle(hq, hkv, d):
    rng = np.random.default_rng(5)
    # empty, single token, page boundaries, several chunks, spare slots
    kv_lens = [0, 1, 15, 16, 17, 63, 64, 65, 100, 257, 0, 700, 33]
    go, gl, eo, el = _decode_both(rng, kv_lens, hq, hkv, d, npages=160)
    assert_close(go, eo, what="decode out")
    assert_close(gl, el, atol=1e-3, rtol=1e-4, what="decode lse")
    for i, n in enumerate(kv_lens):
        if n == 0:
            assert not go[i].any() and np.all(gl[i] == np.float32(-5e4))


@pytest.mark.parametrize("page_size", [32, 64, 128])
@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 4, 64)])
def test_decode_other_page_sizes(page_size, hq, hkv, d):
    """Pages of 32, 64 and 128 tokens (the kernel walks them as runs of 16-token pages): partly filled
    last pages at every position inside a page, several chunks, empty sequences."""
    rng = np.random.default_rng(50 + page_size)
    kv_lens = [0, 1, 15, 16, 17, page_size - 1, page_size, page_size + 1, 3 * page_size + 5, 700, 2500, 33]
    go, gl, eo, el = _decode_both(rng, kv_lens, hq, hkv, d, npages=3 + sum((n + page_size - 1) // page_size for n in kv_lens),
                                  page_size=page_size)
    assert_close(go, eo, what=f"decode out, page size {page_size}")
    assert_close(gl, el, atol=1e-3, rtol=1e-4, what=f"decode lse, page size {page_size}")


def test_decode_cfg1_shapes_against_oracle():
    """BASELINE configs[0]: 4 sequences, contexts 512/1024/1500/2048 (+1 appended), 32/8 heads."""
    rng = np.random.default_rng(6)
    go, gl, eo, el = _decode_both(rng, [513, 1025, 1501, 2049], 32, 8, 128, npages=1024)
    assert_close(go, eo, what="cfg1 decode out")
    assert_close(gl, el, atol=1e-3, rtol=1e-4, what="cfg1 decode lse")


def test_decode_long_sequence_many_chunks():
    rng = np.random.default_rng(7)
    go, gl, eo, el = _decode_both(rng, [9000, 5], 32, 8, 128, npages=600)
    assert_close(go, eo, what="long decode out")
    assert_close(gl, el, atol=1e-3, rtol=1e-4, what="long decode lse")


@pytest.mark.parametrize("batch", [65, 130, 700, 5000])
def test_decode_many_short_sequences(batch):
    """Every work item finds its sequence by a 64-ary search over page_indptr: batches that need one,
    two and three rounds of it, sequences of 0 to 3 pages and a few long ones with several chunks."""
    rng = np.random.default_rng(80 + batch)
    hq, hkv, d = 8, 2, 64
    kv_lens = [int(x) for x in rng.integers(0, 40, size=batch)]
    for i in rng.integers(0, batch, size=5):
        kv_lens[int(i)] = int(rng.integers(300, 900))
    go, gl, eo, el = _decode_both(rng, kv_lens, hq, hkv, d, npages=8 + sum((n + 15) // 16 for n in kv_lens))
    assert_close(go, eo, what=f"decode out, {batch} sequences")
    assert_close(gl, el, atol=1e-3, rtol=1e-4, what=f"decode lse, {batch} sequences")


def test_decode_ignores_garbage_beyond_last_page_len():
    """Slots of the last page beyond last_page_len may hold NaN/Inf bit patterns."""
    rng = np.random.default_rng(8)
    hq, hkv, d = 8, 2, 128
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, [21], 4, hkv, 16, d)
    pages[values[1], :, :, 5:, :] = np.float16(np.nan)
    q = rng.standard_normal((1, hq, d)).astype(F16)
    eo, el = np.zeros((1, hq, d), F16), np.zeros((1, hq), np.float32)
    z = np.zeros(1, np.int32)
    clean = pages.copy()
    clean[values[1], :, :, 5:, :] = 0
    ok.decode(q, clean, indptr, values, last, z, z, eo, el, 0, 1.0, 1e4, d ** -0.5)
    go = torch.zeros((1, hq, d), dtype=torch.float16, device=DEV)
    gl = torch.zeros((1, hq), dtype=torch.float32, device=DEV)
    K.batch_decode_paged_kv(dev(q), dev(pages), i32(indptr), i32(values), i32(last), i32(z), i32(z), go, gl, 0, 1.0,
                            1e4, d ** -0.5)
    assert np.isfinite(host(go)).all()
    assert_close(host(go), eo, what="decode with NaN padding")


@pytest.mark.parametrize("rotary", [0, 1])
@pytest.mark.parametrize("hq,hkv", [(32, 8), (8, 8), (16, 1)])
def test_decode_sliding_window_cache_and_inline_rope(hq, hkv, rotary):
    """length_info (3, B) = [last_page_len; window offset; sink size] and rotary_mode = 1."""
    from tests.test_oracle_kernels import SLIDING_SPEC, sliding_case
    rng = np.random.default_rng(22)
    d = 128
    spec = SLIDING_SPEC + [(2300, 8, 40)]  # several chunks
    pages, indptr, values, info, k_log, _ = sliding_case(rng, spec, hkv, d, npages=260)
    b = len(spec)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    k_off = rng.integers(0, 300, size=b).astype(np.int32)
    q_pos = (k_off + np.array([len(k) for k in k_log]) - 1).astype(np.int32)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
    ok.decode(q, pages, indptr, values, info, k_off, q_pos, eo, el, rotary, 1.0, 1e4, d ** -0.5)
    go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_decode_paged_kv(dev(q), dev(pages), i32(indptr), i32(values), i32(info), i32(k_off), i32(q_pos), go, gl,
                            rotary, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="sliding decode out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="sliding decode lse")


def test_decode_inline_rope_plain_cache_and_scaled_positions():
    rng = np.random.default_rng(23)
    hq, hkv, d = 32, 8, 128
    pages, indptr, values, last, ks, vs = build_paged_kv(rng, [5, 130, 1000], 80, hkv, 16, d)
    q = rng.standard_normal((3, hq, d)).astype(F16)
    k_off = np.array([0, 7, 3000], np.int32)
    q_pos = np.array([4, 136, 3999], np.int32)
    for scale, theta in ((1.0, 1e4), (0.5, 5e5)):
        eo, el = np.zeros((3, hq, d), F16), np.zeros((3, hq), np.float32)
        ok.decode(q, pages, indptr, values, last, k_off, q_pos, eo, el, 1, scale, theta, d ** -0.5)
        go = torch.zeros((3, hq, d), dtype=torch.float16, device=DEV)
        gl = torch.zeros((3, hq), dtype=torch.float32, device=DEV)
        K.batch_decode_paged_kv(dev(q), dev(pages), i32(indptr), i32(values), i32(last), i32(k_off), i32(q_pos), go,
                                gl, 1, scale, theta, d ** -0.5)
        assert_close(host(go), eo, what=f"inline rope decode out, scale {scale}")
        assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"inline rope decode lse, scale {scale}")


def test_decode_rejects_what_is_not_built():
    # head dims outside the tuned set run on the generic kernel, which takes multiples of 8 (fp16) up to 256, and
    # multiples of 16 with rotation inside the kernel
    t = torch.zeros((1, 8, 68), dtype=torch.float16, device=DEV)
    pages = torch.zeros((2, 2, 2, 16, 68), dtype=torch.float16, device=DEV)
    lse = torch.zeros((1, 8), dtype=torch.float32, device=DEV)
    one = i32([0, 1])
    with pytest.raises(KVError, match="head_dim 68 is not built") as info:
        K.batch_decode_paged_kv(t, pages, one, i32([0]), i32([1]), i32([0]), i32([0]), t, lse, 0, 1.0, 1e4, 1.0)
    assert info.value.code == -2
    t = torch.zeros((1, 8, 72), dtype=torch.float16, device=DEV)
    pages = torch.zeros((2, 2, 2, 16, 72), dtype=torch.float16, device=DEV)
    with pytest.raises(KVError, match="multiple of 16, got 72") as info:
        K.batch_decode_paged_kv(t, pages, one, i32([0]), i32([1]), i32([0]), i32([0]), t, lse, 1, 1.0, 1e4, 1.0)
    assert info.value.code == -2


def test_decode_large_gqa_groups_plain_cache():
    """Multi-query shapes (one kv head for 32 or 12 query heads) on a plain cache: groups above 16 heads
    are walked in blocks of 16, groups that are not a power of two leave columns of the tile empty."""
    for hq, hkv, d in ((32, 1, 128), (12, 1, 64), (24, 2, 64), (40, 1, 128), (80, 2, 64)):
        rng = np.random.default_rng(27)
        # 5000 tokens: several chunks, merged per block of 16 heads by the last workgroup to arrive
        go, gl, eo, el = _decode_both(rng, [5, 130, 5000, 16], hq, hkv, d, 330)
        assert_close(go, eo, what=f"decode out {hq}/{hkv}/{d}")
        assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"decode lse {hq}/{hkv}/{d}")


@pytest.mark.parametrize("rotary", [0, 1])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 64), (16, 16, 64), (32, 1, 128), (8, 2, 256)])
def test_decode_sliding_cache_and_inline_rope_other_shapes(hq, hkv, d, rotary):
    """Head dim 64 and GQA groups above 16 through the sliding-window / inline-RoPE form of the decode kernel."""
    from tests.test_oracle_kernels import SLIDING_SPEC, sliding_case
    rng = np.random.default_rng(26)
    pages, pindptr, pvalues, length_info, ks, vs = sliding_case(rng, SLIDING_SPEC, hkv, d)
    b = len(SLIDING_SPEC)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    k_off = np.arange(b, dtype=np.int32) * 3
    q_pos = np.array([k_off[i] + len(ks[i]) - 1 for i in range(b)], np.int32)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
    ok.decode(q, pages, pindptr, pvalues, length_info, k_off, q_pos, eo, el, rotary, 1.0, 1e4, d ** -0.5)
    go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_decode_paged_kv(dev(q), dev(pages), i32(pindptr), i32(pvalues), i32(length_info), i32(k_off), i32(q_pos),
                            go, gl, rotary, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="decode (prefill path) out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="decode (prefill path) lse")


# ------------------------------------------------------------------------------ prefill
def _ragged_both(rng, lens, hq, hkv, dqk, dv, causal, scale=1.0):
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q = (rng.standard_normal((n, hq, dqk)) * scale).astype(F16)
    k = (rng.standard_normal((n, hkv, dqk)) * scale).astype(F16)
    v = (rng.standard_normal((n, hkv, dv)) * scale).astype(F16)
    eo, el = np.zeros((n, hq, dv), F16), np.zeros((n, hq), np.float32)
    zq, zb = np.zeros(n, np.int32), np.zeros(len(lens), np.int32)
    ok.prefill_ragged(q, indptr, k, v, indptr, zq, zb, eo, el, causal, 0, 1.0, 1e4, dqk ** -0.5)
    go = torch.full((n, hq, dv), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_ragged_kv(dev(q), i32(indptr), dev(k), dev(v), i32(indptr), i32(zq), i32(zb), go, gl, causal, 0,
                              1.0, 1e4, dqk ** -0.5)
    return host(go), host(gl), eo, el


@pytest.mark.parametrize("hq,hkv,dqk,dv", [(32, 8, 128, 128), (8, 8, 128, 128), (8, 2, 64, 64), (16, 16, 192, 128),
                                           (8, 2, 256, 256), (8, 2, 80, 80), (32, 8, 96, 96), (6, 2, 112, 112)])
@pytest.mark.parametrize("causal", [1, 0])
def test_ragged_prefill_against_oracle(hq, hkv, dqk, dv, causal):
    rng = np.random.default_rng(9)
    lens = [1, 2, 31, 32, 33, 63, 64, 65, 130, 7]
    go, gl, eo, el = _ragged_both(rng, lens, hq, hkv, dqk, dv, causal)
    assert_close(go, eo, what="ragged out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="ragged lse")


def test_ragged_prefill_longer_chunk():
    rng = np.random.default_rng(10)
    go, gl, eo, el = _ragged_both(rng, [300, 5, 200], 32, 8, 128, 128, 1)
    assert_close(go, eo, what="ragged out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="ragged lse")


@pytest.mark.parametrize("causal", [1, 0])
def test_ragged_prefill_scores_that_keep_growing(causal):
    """The running softmax moves its reference point (and rescales O) only when a score exceeds it by
    more than 2^8; random inputs do that in the first tile only.  Here the score grows by ~10 in the
    exponent per 32 keys, so the rescale runs in every tile."""
    rng = np.random.default_rng(19)
    hq, hkv, d = 8, 2, 128
    lens = [300, 64, 130]
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    q[:, :, :16] = 1
    for b in range(len(lens)):
        k[indptr[b]:indptr[b + 1], :, :16] = (0.153 * np.arange(lens[b], dtype=np.float32))[:, None, None].astype(F16)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    zq, zb = np.zeros(n, np.int32), np.zeros(len(lens), np.int32)
    ok.prefill_ragged(q, indptr, k, v, indptr, zq, zb, eo, el, causal, 0, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_ragged_kv(dev(q), i32(indptr), dev(k), dev(v), i32(indptr), i32(zq), i32(zb), go, gl, causal, 0,
                              1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="ragged growing scores out")
    assert_close(host(gl), el, atol=5e-3, rtol=1e-4, what="ragged growing scores lse")


def _paged_both(rng, kv_lens, q_lens, hq, hkv, d, causal, npages, page_size=16):
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, kv_lens, npages, hkv, page_size, d)
    n = sum(q_lens)
    qindptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    zb, zq = np.zeros(len(kv_lens), np.int32), np.zeros(n, np.int32)
    ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, eo, el, causal, 0, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb),
                             i32(zq), go, gl, causal, 0, 1.0, 1e4, d ** -0.5)
    return host(go), host(gl), eo, el


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (8, 2, 256), (8, 2, 80), (32, 8, 96), (6, 2, 112)])
@pytest.mark.parametrize("causal", [0, 1])
@pytest.mark.parametrize("rows", ["one row tile per sequence", "several row tiles per sequence"])
def test_paged_prefill_against_oracle(hq, hkv, d, causal, rows):
    """Both forms of the paged kernel: launches with at most one row tile per sequence and kv head on
    average copy K/V with the streaming hint, the others without."""
    rng = np.random.default_rng(11)
    kv_lens = [40, 16, 0, 75, 200, 64, 1]
    q_lens = [7, 16, 3, 30, 64, 1, 1]
    if rows.startswith("several"):
        kv_lens = [300, 0, 75, 130]
        q_lens = [290, 5, 64, 129]
    if causal:  # causal paged calls see a KV that already holds the queries' own tokens
        kv_lens = [max(k, q) for k, q in zip(kv_lens, q_lens)]
    go, gl, eo, el = _paged_both(rng, kv_lens, q_lens, hq, hkv, d, causal, npages=64)
    assert_close(go, eo, what="paged out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="paged lse")


@pytest.mark.parametrize("page_size", [32, 64, 128])
@pytest.mark.parametrize("hq,hkv,d", [(16, 4, 128), (8, 2, 64)])
def test_paged_kernels_with_other_page_sizes(page_size, hq, hkv, d):
    """Pages of 32, 64 and 128 tokens through every kernel that reads the page pool with 16-token steps:
    plain and causal paged prefill, the sliding-window / inline-RoPE forms of prefill and decode, the
    tree-masked kernel, and the one-pass chunked prefill."""
    from tests.test_oracle_kernels import sliding_case, tree_paged_case
    from tests.util import REFERENCE_TREES, random_forest
    rng = np.random.default_rng(60 + page_size)
    ps = page_size
    # last pages filled to every kind of boundary: one token, a 16-token run, a tile of 64, the page
    kv_lens = [40, 16, 0, 75, 200, ps, 1, ps + 1, 2 * ps - 1, 700]
    q_lens = [7, 16, 3, 30, 64, 1, 1, 20, 5, 130]
    need = lambda lens: 4 + sum((n + ps - 1) // ps for n in lens)
    for causal in (0, 1):
        lens = [max(k, q) for k, q in zip(kv_lens, q_lens)] if causal else kv_lens
        go, gl, eo, el = _paged_both(rng, lens, q_lens, hq, hkv, d, causal, need(lens), page_size=ps)
        assert_close(go, eo, what=f"paged out, page size {ps}, causal {causal}")
        assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"paged lse, page size {ps}, causal {causal}")

    # sliding-window cache + inline RoPE: prefill with the per-layer window mask, and decode
    spec = [(100, 4, 20), (257, 0, 0), (330, 16, 48), (33, 2, 2), (ps, 16, 32), (90, 0, 17), (2300, 8, 40)]
    sq_lens = [7, 64, 33, 3, 1, 30, 40]
    pages, pindptr, pvalues, info, k_log, _ = sliding_case(rng, spec, hkv, d, ps=ps, npages=need([x[0] for x in spec]))
    n = sum(sq_lens)
    qindptr = np.concatenate([[0], np.cumsum(sq_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k_off = rng.integers(0, 200, size=len(spec)).astype(np.int32)
    q_pos = np.concatenate([k_off[i] + len(k_log[i]) - sq_lens[i] + np.arange(sq_lens[i]) for i in range(len(spec))])
    q_pos = q_pos.astype(np.int32)
    for causal, window in ((0, 0), (1, 40)):
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
        ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, info, k_off, q_pos, eo, el, causal, 1, 1.0, 1e4,
                         d ** -0.5, sliding_window_size=window)
        go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(info), i32(k_off),
                                 i32(q_pos), go, gl, causal, 1, 1.0, 1e4, d ** -0.5, sliding_window_size=window)
        assert_close_where_keys(host(go), host(gl), eo, el, rows_without_keys(sq_lens, causal, window), 2e-3,
                                f"sliding paged, page size {ps}, window {window}")
    b = len(spec)
    qd = rng.standard_normal((b, hq, d)).astype(F16)
    qd_pos = (k_off + np.array([len(k) for k in k_log]) - 1).astype(np.int32)
    for rotary in (0, 1):
        eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
        ok.decode(qd, pages, pindptr, pvalues, info, k_off, qd_pos, eo, el, rotary, 1.0, 1e4, d ** -0.5)
        go = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_decode_paged_kv(dev(qd), dev(pages), i32(pindptr), i32(pvalues), i32(info), i32(k_off), i32(qd_pos),
                                go, gl, rotary, 1.0, 1e4, d ** -0.5)
        assert_close(host(go), eo, what=f"sliding decode out, page size {ps}, rotary {rotary}")
        assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"sliding decode lse, page size {ps}, rotary {rotary}")

    # token trees behind a cached prefix
    prefix = [10, 20, 30, 40, 0, 700, ps - 3]
    trees = REFERENCE_TREES + [random_forest(rng, 50), random_forest(rng, 256), random_forest(rng, 31)]
    new_lens = [7, 8, 10, 7, 50, 256, 16]
    (pages, pindptr, pvalues, last, ks, vs, qindptr, q, tindptr, labels, masks) = tree_paged_case(
        rng, prefix, trees, new_lens, hq, hkv, d, ps=ps, npages=need([a + len(t) for a, t in zip(prefix, trees)]))
    n = len(q)
    zb, zq = np.zeros(len(trees), np.int32), np.zeros(n, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, eo, el, 0, 1.0, 1e4, d ** -0.5,
                       tindptr, labels)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.tree_attn_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb), i32(zq),
                         go, gl, 0, 1.0, 1e4, d ** -0.5, i32(tindptr), i32(labels))
    assert_close(host(go), eo, what=f"tree paged out, page size {ps}")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"tree paged lse, page size {ps}")

    # cached prefix + new chunk in one pass, against ragged + paged + merge of the oracle
    prefix = [0, 1, 63, 64, 65, ps, ps + 1, 700, 16, 330]
    chunk = [5, 130, 1, 64, 33, 300, 2, 40, 129, 64]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, prefix, need(prefix), hkv, ps, d)
    n = sum(chunk)
    ind = np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    zq, zb = np.zeros(n, np.int32), np.zeros(len(prefix), np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    to, tl = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, d ** -0.5)
    ok.prefill_paged(q, ind, pages, pindptr, pvalues, last, zb, zq, to, tl, 0, 0, 1.0, 1e4, d ** -0.5)
    ok.merge_state_inplace(eo, el, to, tl)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_cached_and_new_kv(dev(q), i32(ind), dev(k), dev(v), dev(pages), i32(pindptr), i32(pvalues),
                                      i32(last), go, gl, d ** -0.5)
    assert_close(host(go), eo, what=f"one-pass chunked prefill out, page size {ps}")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"one-pass chunked prefill lse, page size {ps}")


@pytest.mark.parametrize("hq,hkv,d,splits", [(16, 4, 128, 0), (16, 4, 128, 3), (8, 2, 64, 5), (8, 2, 64, 64), (8, 2, 256, 2)])
def test_prefill_split_over_the_keys(hq, hkv, d, splits):
    """Launches with few row tiles split every row tile's keys over several workgroups and merge the
    states: the derived split (few queries against long cached sequences) and forced ones (more shares
    than some sequences have tiles, so that shares are empty; sequences without cached tokens; rows that
    see no key), through the paged kernel with every mask, the tree-masked kernel and the one-pass
    chunked prefill."""
    import tvm_amd
    from tests.test_oracle_kernels import sliding_case, tree_paged_case
    from tests.util import REFERENCE_TREES, random_forest
    rng = np.random.default_rng(70 + splits)
    prev = tvm_amd.set_option("prefill_kv_splits", splits)
    try:
        if splits == 0:  # long enough for the derived split: 8 shares
            go, gl, eo, el = _paged_both(rng, [6000, 3000], [5, 3], hq, hkv, d, 1, 600)
            assert_close(go, eo, what="paged out, derived split")
            assert_close(gl, el, atol=2e-3, rtol=1e-4, what="paged lse, derived split")
        kv_lens = [1500, 16, 0, 75, 700, 64, 1, 65, 400, 129]
        q_lens = [7, 16, 3, 30, 64, 1, 1, 20, 5, 40]
        for causal in (0, 1):
            lens = [max(k, q) for k, q in zip(kv_lens, q_lens)] if causal else kv_lens
            go, gl, eo, el = _paged_both(rng, lens, q_lens, hq, hkv, d, causal, 8 + sum((n + 15) // 16 for n in lens))
            assert_close(go, eo, what=f"paged out, {splits} splits, causal {causal}")
            assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"paged lse, {splits} splits, causal {causal}")

        spec = [(100, 4, 20), (1300, 0, 0), (800, 16, 48), (33, 2, 2), (64, 16, 32), (500, 0, 17)]
        sq_lens = [7, 64, 33, 3, 1, 50]
        pages, pindptr, pvalues, info, k_log, _ = sliding_case(rng, spec, hkv, d, npages=8 + sum((x[0] + 15) // 16 for x in spec))
        n = sum(sq_lens)
        qindptr = np.concatenate([[0], np.cumsum(sq_lens)]).astype(np.int32)
        q = rng.standard_normal((n, hq, d)).astype(F16)
        k_off = rng.integers(0, 200, size=len(spec)).astype(np.int32)
        q_pos = np.concatenate([k_off[i] + len(k_log[i]) - sq_lens[i] + np.arange(sq_lens[i]) for i in range(len(spec))])
        q_pos = q_pos.astype(np.int32)
        for causal, window, rotary in ((0, 0, 1), (1, 40, 0), (1, 0, 1)):
            eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
            ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, info, k_off, q_pos, eo, el, causal, rotary, 1.0, 1e4,
                             d ** -0.5, sliding_window_size=window)
            go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
            gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
            K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(info), i32(k_off),
                                     i32(q_pos), go, gl, causal, rotary, 1.0, 1e4, d ** -0.5, sliding_window_size=window)
            assert_close_where_keys(host(go), host(gl), eo, el, rows_without_keys(sq_lens, causal, window), 2e-3,
                                    f"sliding paged, {splits} splits, window {window}")

        prefix = [10, 1200, 30, 640, 0, 300]
        trees = REFERENCE_TREES + [random_forest(rng, 50), random_forest(rng, 15)]
        new_lens = [7, 8, 10, 7, 50, 15]
        (pages, pindptr, pvalues, last, ks, vs, qindptr, q, tindptr, labels, masks) = tree_paged_case(
            rng, prefix, trees, new_lens, hq, hkv, d, npages=8 + sum((a + len(t) + 15) // 16 for a, t in zip(prefix, trees)))
        n = len(q)
        zb, zq = np.zeros(len(trees), np.int32), np.zeros(n, np.int32)
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
        ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, eo, el, 0, 1.0, 1e4, d ** -0.5,
                           tindptr, labels)
        go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
        K.tree_attn_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb), i32(zq),
                             go, gl, 0, 1.0, 1e4, d ** -0.5, i32(tindptr), i32(labels))
        assert_close(host(go), eo, what=f"tree paged out, {splits} splits")
        assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"tree paged lse, {splits} splits")

        prefix = [0, 1, 63, 64, 65, 1500, 200, 700]
        chunk = [5, 130, 1, 64, 33, 40, 2, 129]
        pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, prefix, 8 + sum((x + 15) // 16 for x in prefix), hkv, 16, d)
        n = sum(chunk)
        ind = np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32)
        q = rng.standard_normal((n, hq, d)).astype(F16)
        k = rng.standard_normal((n, hkv, d)).astype(F16)
        v = rng.standard_normal((n, hkv, d)).astype(F16)
        zq, zb = np.zeros(n, np.int32), np.zeros(len(prefix), np.int32)
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
        to, tl = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
        ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, d ** -0.5)
        ok.prefill_paged(q, ind, pages, pindptr, pvalues, last, zb, zq, to, tl, 0, 0, 1.0, 1e4, d ** -0.5)
        ok.merge_state_inplace(eo, el, to, tl)
        go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_prefill_cached_and_new_kv(dev(q), i32(ind), dev(k), dev(v), dev(pages), i32(pindptr), i32(pvalues),
                                          i32(last), go, gl, d ** -0.5)
        assert_close(host(go), eo, what=f"one-pass chunked prefill out, {splits} splits")
        assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what=f"one-pass chunked prefill lse, {splits} splits")
        # the same step as the cache composes it for forked sequences: the ragged kernel's state, then the paged
        # kernel merged into it (split: the merge kernel folds the caller's state in with the shares)
        go2 = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
        gl2 = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
        K.batch_prefill_ragged_kv(dev(q), i32(ind), dev(k), dev(v), i32(ind), i32(zq), i32(zb), go2, gl2, 1, 0, 1.0, 1e4,
                                  d ** -0.5)
        K.batch_prefill_paged_kv(dev(q), i32(ind), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb), i32(zq), go2,
                                 gl2, 0, 0, 1.0, 1e4, d ** -0.5, merge_into=True)
        assert_close(host(go2), eo, what=f"paged merged into ragged out, {splits} splits")
        assert_close(host(gl2), el, atol=2e-3, rtol=1e-4, what=f"paged merged into ragged lse, {splits} splits")
    finally:
        tvm_amd.set_option("prefill_kv_splits", prev)


def test_prefill_more_than_64_sequences():
    """Up to 64 sequences the kernels rank the sequences by length themselves; beyond that they
    take them in batch order.  Both orders on one ragged and one paged call."""
    rng = np.random.default_rng(43)
    hq, hkv, d = 8, 2, 128
    for nseq in (64, 70):
        kv_lens = [int(x) for x in rng.integers(0, 90, size=nseq)]
        q_lens = [int(x) for x in rng.integers(1, 40, size=nseq)]
        go, gl, eo, el = _paged_both(rng, kv_lens, q_lens, hq, hkv, d, 0, 512)
        assert_close(go, eo, what=f"paged out, {nseq} sequences")
        assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"paged lse, {nseq} sequences")
        go, gl, eo, el = _ragged_both(rng, q_lens, hq, hkv, d, d, 1)
        assert_close(go, eo, what=f"ragged out, {nseq} sequences")
        assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"ragged lse, {nseq} sequences")


def test_layer_sliding_window_mask_known_answer_on_the_gpu():
    """The reference's known-answer vector for the paged prefill kernel with sliding_window_size = 3
    (tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_tir.py:98-156)."""
    hq, hkv, d = 4, 2, 64
    q = np.zeros((2, hq, d), F16)
    pages = np.zeros((1, 2, hkv, 16, d), F16)
    for position, value in enumerate([1, 3, 5]):
        pages[0, 1, :, position, :] = value
    go = torch.full((2, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.zeros((2, hq), dtype=torch.float32, device=DEV)
    K.batch_prefill_paged_kv(dev(q), i32([0, 2]), dev(pages), i32([0, 1]), i32([0]), i32([[3], [0], [0]]), i32([0]),
                             i32([3, 4]), go, gl, 1, 0, 1.0, 1e4, d ** -0.5, sliding_window_size=3)
    assert_close(host(go)[:, 0, 0], np.array([4, 5], F16), atol=1e-3, rtol=1e-3, what="sliding window known answer")


@pytest.mark.parametrize("hq,hkv,d", [(16, 4, 128), (8, 2, 64), (8, 2, 256)])
@pytest.mark.parametrize("rotary", [0, 1])
@pytest.mark.parametrize("causal,window", [(0, 1024), (1, 0), (1, 5), (1, 40)])
@pytest.mark.parametrize("long_q", [False, True])
def test_paged_prefill_sliding_cache_layer_window_and_inline_rope(hq, hkv, d, rotary, causal, window, long_q):
    """length_info (3, B), the per-layer window mask (window > 0 together with causal; with
    window = 0 or without causal the reference falls back to the plain masks) and rotary_mode = 1.
    long_q: several row tiles per sequence, the form of the kernel that copies K/V without the
    streaming hint."""
    from tests.test_oracle_kernels import sliding_case
    rng = np.random.default_rng(24)
    spec = [(100, 4, 20), (257, 0, 0), (330, 16, 48), (33, 2, 2), (64, 16, 32), (90, 0, 17)]
    q_lens = [70, 250, 290, 3, 1, 30] if long_q else [7, 64, 33, 3, 1, 30]
    pages, pindptr, pvalues, info, k_log, _ = sliding_case(rng, spec, hkv, d, npages=64)
    n = sum(q_lens)
    qindptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k_off = rng.integers(0, 200, size=len(spec)).astype(np.int32)
    q_pos = np.concatenate([k_off[i] + len(k_log[i]) - q_lens[i] + np.arange(q_lens[i]) for i in range(len(spec))])
    q_pos = q_pos.astype(np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_paged(q, qindptr, pages, pindptr, pvalues, info, k_off, q_pos, eo, el, causal, rotary, 1.0, 1e4,
                     d ** -0.5, sliding_window_size=window)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(info), i32(k_off),
                             i32(q_pos), go, gl, causal, rotary, 1.0, 1e4, d ** -0.5, sliding_window_size=window)
    assert_close_where_keys(host(go), host(gl), eo, el, rows_without_keys(q_lens, causal, window), 2e-3, "sliding paged")


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (8, 2, 256)])
@pytest.mark.parametrize("causal", [1, 0])
def test_prefill_inline_rope_plain_cache(hq, hkv, d, causal):
    rng = np.random.default_rng(25)
    # ragged
    lens = [1, 33, 64, 130, 7]
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    k_off = np.array([0, 17, 500, 3, 1000], np.int32)
    q_pos = np.concatenate([k_off[i] + np.arange(lens[i]) for i in range(len(lens))]).astype(np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_ragged(q, indptr, k, v, indptr, q_pos, k_off, eo, el, causal, 1, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_ragged_kv(dev(q), i32(indptr), dev(k), dev(v), i32(indptr), i32(q_pos), i32(k_off), go, gl,
                              causal, 1, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="inline rope ragged out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="inline rope ragged lse")
    # paged, plain length_info
    kv_lens = [max(40, lens[0]), 75, 200, 130, 64]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, kv_lens, 48, hkv, 16, d)
    q_pos = np.concatenate([k_off[i] + kv_lens[i] - lens[i] + np.arange(lens[i]) for i in range(len(lens))])
    q_pos = q_pos.astype(np.int32)
    ok.prefill_paged(q, indptr, pages, pindptr, pvalues, last, k_off, q_pos, eo, el, causal, 1, 0.5, 5e5, d ** -0.5)
    K.batch_prefill_paged_kv(dev(q), i32(indptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(k_off),
                             i32(q_pos), go, gl, causal, 1, 0.5, 5e5, d ** -0.5)
    assert_close(host(go), eo, what="inline rope paged out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="inline rope paged lse")


# ------------------------------------------------------------------------------ token trees
@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (8, 2, 256)])
@pytest.mark.parametrize("rotary", [0, 1])
def test_tree_attn_ragged_against_oracle(hq, hkv, d, rotary):
    from tests.util import REFERENCE_TREES, random_forest, tree_order
    rng = np.random.default_rng(40)
    trees = REFERENCE_TREES + [random_forest(rng, 200), [-1], list(range(-1, 69))]
    lens = [len(t) for t in trees]
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    mask = np.concatenate([tree_order(t) for t in trees])
    # positions: the depth of the node in its tree on top of a per-sequence offset, as the cache hands out
    depth = []
    for i, t in enumerate(trees):
        dep = []
        for parent in t:
            dep.append(0 if parent == -1 else dep[parent] + 1)
        depth += [100 * i + x for x in dep]
    q_pos = np.array(depth, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.tree_attn_ragged(q, indptr, k, v, indptr, q_pos, indptr, mask, eo, el, rotary, 1.0, 1e4, d ** -0.5)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_tree_attn(dev(q), i32(indptr), dev(k), dev(v), i32(indptr), i32(q_pos), i32(indptr), i32(mask), go, gl,
                      rotary, 1.0, 1e4, d ** -0.5)
    assert_close(host(go), eo, what="tree ragged out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="tree ragged lse")


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (8, 2, 256)])
def test_tree_attn_paged_against_oracle(hq, hkv, d):
    from tests.test_oracle_kernels import tree_paged_case
    from tests.util import REFERENCE_TREES, random_forest
    rng = np.random.default_rng(41)
    prefix = [10, 20, 30, 40, 0, 700, 129]
    trees = REFERENCE_TREES + [random_forest(rng, 50), random_forest(rng, 256), random_forest(rng, 31)]
    new_lens = [7, 8, 10, 7, 50, 256, 16]  # some trees already had nodes from earlier steps
    (pages, pindptr, pvalues, last, ks, vs, qindptr, q, tindptr, labels, masks) = tree_paged_case(
        rng, prefix, trees, new_lens, hq, hkv, d, npages=128)
    n = len(q)
    zb, zq = np.zeros(len(trees), np.int32), np.zeros(n, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, eo, el, 0, 1.0, 1e4, d ** -0.5,
                       tindptr, labels)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.tree_attn_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb), i32(zq),
                         go, gl, 0, 1.0, 1e4, d ** -0.5, i32(tindptr), i32(labels))
    assert_close(host(go), eo, what="tree paged out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="tree paged lse")
    with pytest.raises(KVError, match="inline rotary mode is not supported in tree attention"):
        K.tree_attn_paged_kv(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb),
                             i32(zq), go, gl, 1, 1.0, 1e4, d ** -0.5, i32(tindptr), i32(labels))


def test_chunked_prefill_composition_matches_oracle():
    """ragged(causal) + paged(non-causal) + merge_state: the chunked-prefill path of the cache."""
    rng = np.random.default_rng(12)
    hq, hkv, d = 32, 8, 128
    prefix, chunk = [100, 0, 333], [50, 20, 129]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, prefix, 64, hkv, 16, d)
    n = sum(chunk)
    ind = np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    zq, zb = np.zeros(n, np.int32), np.zeros(3, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    to, tl = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, d ** -0.5)
    ok.prefill_paged(q, ind, pages, pindptr, pvalues, last, zb, zq, to, tl, 0, 0, 1.0, 1e4, d ** -0.5)
    ok.merge_state_inplace(eo, el, to, tl)
    go = torch.zeros((n, hq, d), dtype=torch.float16, device=DEV)
    gl = torch.zeros((n, hq), dtype=torch.float32, device=DEV)
    ho = torch.zeros((n, hq, d), dtype=torch.float16, device=DEV)
    hl = torch.zeros((n, hq), dtype=torch.float32, device=DEV)
    qd = dev(q)
    K.batch_prefill_ragged_kv(qd, i32(ind), dev(k), dev(v), i32(ind), i32(zq), i32(zb), go, gl, 1, 0, 1.0, 1e4, d ** -0.5)
    K.batch_prefill_paged_kv(qd, i32(ind), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb), i32(zq), ho, hl,
                             0, 0, 1.0, 1e4, d ** -0.5)
    go2, gl2 = go.clone(), gl.clone()
    K.merge_state_inplace(go, gl, ho, hl)
    assert_close(host(go), eo, what="chunked prefill out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="chunked prefill lse")
    # the same with the merge done in the paged kernel's epilogue (sequence 1 has no pages: unchanged)
    K.batch_prefill_paged_kv(qd, i32(ind), dev(pages), i32(pindptr), i32(pvalues), i32(last), i32(zb), i32(zq), go2,
                             gl2, 0, 0, 1.0, 1e4, d ** -0.5, merge_into=True)
    assert_close(host(go2), eo, what="chunked prefill out, merged in the epilogue")
    assert_close(host(gl2), el, atol=2e-3, rtol=1e-4, what="chunked prefill lse, merged in the epilogue")
    assert_close(host(go2), host(go), atol=2e-3, rtol=2e-3, what="epilogue merge vs separate merge")
    # and as one pass over the cached and the new tokens
    go3 = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl3 = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_cached_and_new_kv(qd, i32(ind), dev(k), dev(v), dev(pages), i32(pindptr), i32(pvalues), i32(last),
                                      go3, gl3, d ** -0.5)
    assert_close(host(go3), eo, what="chunked prefill out, one pass")
    assert_close(host(gl3), el, atol=2e-3, rtol=1e-4, what="chunked prefill lse, one pass")


@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (8, 8, 128), (8, 2, 256)])
def test_prefill_cached_and_new_in_one_pass(hq, hkv, d):
    """Prefix lengths around the tile size (the padded end of the cached part), no prefix, chunks of one
    token and of several row tiles; against ragged + paged + merge of the oracle."""
    rng = np.random.default_rng(44)
    prefix = [0, 1, 63, 64, 65, 128, 200, 700, 16, 330]
    chunk = [5, 130, 1, 64, 33, 300, 2, 40, 129, 64]
    if d == 64:  # more than 64 sequences: the kernel takes them in batch order
        prefix += [int(x) for x in rng.integers(0, 100, size=60)]
        chunk += [int(x) for x in rng.integers(1, 50, size=60)]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, prefix, 512, hkv, 16, d)
    n = sum(chunk)
    ind = np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    k = rng.standard_normal((n, hkv, d)).astype(F16)
    v = rng.standard_normal((n, hkv, d)).astype(F16)
    zq, zb = np.zeros(n, np.int32), np.zeros(len(prefix), np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    to, tl = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, d ** -0.5)
    ok.prefill_paged(q, ind, pages, pindptr, pvalues, last, zb, zq, to, tl, 0, 0, 1.0, 1e4, d ** -0.5)
    ok.merge_state_inplace(eo, el, to, tl)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_cached_and_new_kv(dev(q), i32(ind), dev(k), dev(v), dev(pages), i32(pindptr), i32(pvalues),
                                      i32(last), go, gl, d ** -0.5)
    assert_close(host(go), eo, what="one-pass chunked prefill out")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="one-pass chunked prefill lse")


@pytest.mark.parametrize("apply_rope", [1, 0])
@pytest.mark.parametrize("hq,hkv,d", [(32, 8, 128), (8, 2, 64), (8, 2, 256)])
def test_prefill_one_pass_with_queries_from_the_fused_qkv(hq, hkv, d, apply_rope):
    """The step of the cache object for a chunked prefill: k rotated and appended without writing q
    (fused_rope_append with q = None), then the one-pass kernel that reads q from qkv and rotates it
    itself.  Against the oracle from the raw qkv (fused_rope, ragged + paged + merge), with positions
    that continue each sequence's prefix, a scaled position and a theta other than the default; the
    appended slots against the k / v rows bit for bit."""
    rng = np.random.default_rng(45)
    prefix = [0, 63, 200, 700, 16]
    chunk = [130, 1, 33, 40, 129]
    pages, pindptr, pvalues, last, ks, vs = build_paged_kv(rng, prefix, 512, hkv, 16, d)
    n = sum(chunk)
    ind = np.concatenate([[0], np.cumsum(chunk)]).astype(np.int32)
    qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
    pos = np.concatenate([p0 + np.arange(c) for p0, c in zip(prefix, chunk)]).astype(np.int32)
    scale, theta = 0.5, 5e5
    # free slots for the new rows: pages beyond the ones the prefixes use
    used = set(int(x) for x in pvalues)
    free = [pg for pg in range(512) if pg not in used]
    slots = np.array([free[i // 16] * 16 + i % 16 for i in range(n)], np.int32)
    q, k, v = np.zeros((n, hq, d), F16), np.zeros((n, hkv, d), F16), np.zeros((n, hkv, d), F16)
    ok.fused_rope(qkv, pos, q, k, v, apply_rope, theta=theta, scale=scale)
    zq, zb = np.zeros(n, np.int32), np.zeros(len(prefix), np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    to, tl = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_ragged(q, ind, k, v, ind, zq, zb, eo, el, 1, 0, 1.0, 1e4, d ** -0.5)
    ok.prefill_paged(q, ind, pages, pindptr, pvalues, last, zb, zq, to, tl, 0, 0, 1.0, 1e4, d ** -0.5)
    ok.merge_state_inplace(eo, el, to, tl)
    gp, gqkv = dev(pages), dev(qkv)
    gk = torch.zeros((n, hkv, d), dtype=torch.float16, device=DEV)
    gv = torch.zeros_like(gk)
    go = torch.full((n, hq, d), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, hq), 7.0, dtype=torch.float32, device=DEV)
    K.fused_rope_append(gqkv, i32(pos), None, gk, gv, apply_rope, gp, i32(slots), scale, theta)
    K.batch_prefill_cached_and_new_kv_fused_q(gqkv, i32(pos), apply_rope, scale, theta, i32(ind), gk, gv, gp,
                                              i32(pindptr), i32(pvalues), i32(last), go, gl, d ** -0.5)
    assert_close(host(go), eo, what="one-pass chunked prefill with fused q, out")
    assert_close(host(gl), el, atol=4e-3, rtol=1e-4, what="one-pass chunked prefill with fused q, lse")
    assert np.array_equal(host(gv), v)
    assert_close(host(gk), k, atol=2e-3, rtol=2e-3, what="rotated k")
    flat = gp.permute(0, 3, 1, 2, 4).reshape(-1, 2, hkv, d)
    sl = torch.tensor(slots, dtype=torch.int64, device=DEV)
    assert torch.equal(flat[sl, 0], gk) and torch.equal(flat[sl, 1], gv)
    assert torch.equal(gqkv, dev(qkv)), "qkv must be left alone"


def test_measurement_utilities():
    """The calibration kernels of the benchmark (libtvmkv_bench.so): the copy copies, the reads leave their
    input alone, and the MFMA loop adds up what its instruction count says (integers in fp32, so exactly)."""
    from tvm_amd import bench_aids as A

    src = torch.arange(1 << 16, dtype=torch.int32, device=DEV)
    dst = torch.zeros_like(src)
    sink = torch.zeros(4, dtype=torch.int32, device=DEV)
    A.stream_copy(src, dst)
    A.stream_read(src, sink)
    A.stream_read_nt(src, sink)
    torch.cuda.synchronize()
    assert torch.equal(src, dst) and torch.equal(src, torch.arange(1 << 16, dtype=torch.int32, device=DEV))
    ops = torch.full((256, 16), 0.5, dtype=torch.float16, device=DEV)
    out = torch.zeros((3, 256), dtype=torch.float32, device=DEV)
    iters = 5
    A.mfma_loop(ops, out, iters)
    torch.cuda.synchronize()
    # one instruction adds 16 * 0.5 * 0.5 = 4 to each of its 16 results per lane; 8 instructions a round
    assert torch.all(out == 4.0 * 16 * 8 * iters)


def test_scratch_epoch_wrap_and_release():
    """Split-KV launches across the wrap of the 32-bit epoch that tags their arrival counters (the launch
    count is set just below 2^32), through the pooled buffer and through the built-in one of the entry
    point that allocates nothing; then the pooled buffers of the stream are released and the next call
    allocates afresh.  Every output equals the one before."""
    from tvm_amd._lib import check, lib

    rng = np.random.default_rng(5)
    kv = [700, 33, 1500, 260]
    pages, ip, pv, last, _, _ = build_paged_kv(rng, kv, 170, 8, 16, 128)
    q = rng.standard_normal((4, 32, 128)).astype(F16)
    z = np.zeros(4, np.int32)
    args = (dev(q), dev(pages), i32(ip), i32(pv), i32(last), i32(z), i32(z))

    def run(noalloc):
        o = torch.zeros((4, 32, 128), dtype=torch.float16, device=DEV)
        s = torch.zeros((4, 32), dtype=torch.float32, device=DEV)
        K.batch_decode_paged_kv(*args, o, s, 0, 1.0, 1e4, 128 ** -0.5, noalloc=noalloc)
        return host(o), host(s)

    prev = tvm_amd.set_option("decode_chunk_pages", 8)  # several chunks per sequence: the fused merge counts arrivals
    try:
        base = run(False)
        base_noalloc = run(True)
        assert np.array_equal(base[0], base_noalloc[0])
        check(lib().tvmkv_debug_set_scratch_launches((1 << 32) - 3))
        for _ in range(6):  # epochs 0xfffffffe, 0xffffffff, then 1, 2, ... from cleared counters
            for noalloc in (False, True):
                o, s = run(noalloc)
                assert np.array_equal(o, base[0]) and np.array_equal(s, base[1])
        check(lib().tvmkv_release_scratch(ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        o, s = run(False)
        assert np.array_equal(o, base[0]) and np.array_equal(s, base[1])
    finally:
        tvm_amd.set_option("decode_chunk_pages", prev)


# ------------------------------------------------------------------------------ fused decode step
@pytest.mark.parametrize("hq,hkv,d,ps,apply_rope", [(32, 8, 128, 16, 1), (32, 8, 128, 16, 0), (8, 2, 64, 32, 1),
                                                    (32, 1, 128, 16, 1), (64, 1, 128, 16, 1), (20, 1, 64, 16, 1),
                                                    (16, 8, 256, 16, 1), (64, 8, 128, 64, 1)])
def test_fused_decode_step(hq, hkv, d, ps, apply_rope):
    """Split + RoPE + append + decode attention of a step in one launch (tvmkv_fused_decode_step) against
    the oracle's three kernels, and against the library's own two launches: the slot of the new token holds
    NaN patterns before the call, so a work item that attended before the append landed would show."""
    rng = np.random.default_rng(90 + hq + d)
    kv_lens = [1, 16, 17, 33, 700, 2500, 64, ps + 1, 3 * ps]   # the new token included
    b = len(kv_lens)
    npages = 4 + sum((n + ps - 1) // ps for n in kv_lens)
    pages, ip, pv, last, _, _ = build_paged_kv(rng, kv_lens, npages, hkv, ps, d)
    slots = np.array([pv[ip[i] + (n - 1) // ps] * ps + (n - 1) % ps for i, n in enumerate(kv_lens)], np.int32)
    q_pos = (rng.integers(0, 3000, size=b) + np.array(kv_lens) - 1).astype(np.int32)
    qkv = rng.standard_normal((b, hq + 2 * hkv, d)).astype(F16)
    # oracle: split + RoPE, append, decode
    eq, ek, ev = np.zeros((b, hq, d), F16), np.zeros((b, hkv, d), F16), np.zeros((b, hkv, d), F16)
    ok.fused_rope(qkv, q_pos, eq, ek, ev, apply_rope)
    epages = pages.copy()
    ok.transpose_append(epages, ek, ev, slots)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
    z = np.zeros(b, np.int32)
    ok.decode(eq, epages, ip, pv, last, z, z, eo, el, 0, 1.0, 1e4, d ** -0.5)
    # the new token's slot is poisoned on the device side
    poisoned = pages.copy()
    for s in slots:
        poisoned[s // ps, :, :, s % ps, :] = np.float16(np.nan)
    # the library's two launches
    p2 = dev(poisoned)
    q2, k2, v2 = (torch.zeros(a.shape, dtype=torch.float16, device=DEV) for a in (eq, ek, ev))
    o2 = torch.zeros((b, hq, d), dtype=torch.float16, device=DEV)
    l2 = torch.zeros((b, hq), dtype=torch.float32, device=DEV)
    K.fused_rope_append(dev(qkv), i32(q_pos), q2, k2, v2, apply_rope, p2, i32(slots), 1.0, 1e4)
    K.batch_decode_paged_kv(q2, p2, i32(ip), i32(pv), i32(last), i32(z), i32(z), o2, l2, 0, 1.0, 1e4, d ** -0.5)
    # one launch
    p1 = dev(poisoned)
    o1 = torch.full((b, hq, d), 7.0, dtype=torch.float16, device=DEV)
    l1 = torch.full((b, hq), 7.0, dtype=torch.float32, device=DEV)
    K.fused_decode_step(dev(qkv), p1, i32(ip), i32(pv), i32(last), i32(q_pos), i32(slots), o1, l1, apply_rope, 1.0, 1e4,
                        d ** -0.5)
    assert torch.equal(p1, p2), "the fused step must leave the pool as split + RoPE + append does"
    gp = host(p1)
    assert np.array_equal(gp[:, 1], epages[:, 1])                      # V rows: a copy
    assert_close(gp[:, 0], epages[:, 0], atol=2e-3, rtol=1e-3, what="appended K rows vs oracle")  # one fp16 ulp
    assert_close(host(o1), eo, what="fused step out vs oracle")
    assert_close(host(l1), el, atol=1e-3, rtol=1e-4, what="fused step lse vs oracle")
    assert_close(host(o1), host(o2), atol=2e-3, rtol=2e-3, what="fused step out vs two launches")


def test_decode_group_of_64_heads():
    """One kv head for 64 query heads: two work items of 32 heads per chunk; 16 kv heads x 64: the same at head dim 64."""
    for hq, hkv, d in ((64, 1, 128), (128, 2, 64)):
        rng = np.random.default_rng(28)
        go, gl, eo, el = _decode_both(rng, [5, 130, 3000, 16, 0], hq, hkv, d, 220)
        assert_close(go, eo, what=f"decode out {hq}/{hkv}/{d}")
        assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"decode lse {hq}/{hkv}/{d}")


def test_head_dims_between_64_and_128_refuse_what_they_do_not_have():
    """Head dims 80, 96 and 112 run on the head dim 128 kernels of the plain cache and on the generic kernels in
    the sliding-window / inline-RoPE forms (tests/test_gpu_generic.py); the one-pass chunked prefill and RoPE inside
    the kernel at a head dim that is not a multiple of 16 are not built and say so."""
    t = torch.zeros((1, 8, 96), dtype=torch.float16, device=DEV)
    pages = torch.zeros((2, 2, 2, 16, 96), dtype=torch.float16, device=DEV)
    lse = torch.zeros((1, 8), dtype=torch.float32, device=DEV)
    one, z = i32([0, 1]), i32([0])
    kv = torch.zeros((1, 2, 96), dtype=torch.float16, device=DEV)
    with pytest.raises(KVError, match="is not built") as info:
        K.batch_prefill_cached_and_new_kv(t, one, kv, kv, pages, one, z, i32([1]), t, lse, 1.0)
    assert info.value.code == -2
    t = torch.zeros((1, 8, 72), dtype=torch.float16, device=DEV)
    pages = torch.zeros((2, 2, 2, 16, 72), dtype=torch.float16, device=DEV)
    with pytest.raises(KVError, match="multiple of 16") as info:
        K.batch_decode_paged_kv(t, pages, one, z, i32([1]), z, z, t, lse, 1, 1.0, 1e4, 1.0)
    assert info.value.code == -2


# ------------------------------------------------------------------------------ frequency variants in the kernels
ROPE_VARIANTS = [
    {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
     "original_max_position_embeddings": 8192},
    {"rope_type": "yarn", "factor": 40.0, "beta_fast": 32, "beta_slow": 1, "original_max_position_embeddings": 4096},
    {"rope_type": "longrope", "max_position_embeddings": 131072, "original_max_position_embeddings": 4096},
    {"rope_type": "gptj"},
    {"rope_type": "llama4", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
     "original_max_position_embeddings": 8192},
]


@pytest.mark.parametrize("rope_scaling", ROPE_VARIANTS, ids=lambda sc: sc["rope_type"])
@pytest.mark.parametrize("hq,hkv,d", [(8, 2, 128), (4, 2, 64), (20, 1, 128)])
def test_inline_rope_frequency_variants(rope_scaling, hq, hkv, d):
    """rotary_mode = 1 with the model's frequency variant (the *_scaled launchers) in the decode, paged prefill,
    ragged prefill and ragged tree-attention kernels, against the oracle with the same variant in force."""
    from tests.util import random_forest, tree_order
    rng = np.random.default_rng(300 + d + hq)
    sm = d ** -0.5
    # (the oracle recomputes the rotation for every score element: the shapes are small)
    # decode over a sliding-window cache (sinks, an evicted gap) and a plain one
    kv = [5, 130, 600, 64]
    pages, ip, pv, last, _, _ = build_paged_kv(rng, kv, 60, hkv, 16, d)
    info = np.array([last, [2, 40, 300, 0], [1, 4, 0, 0]], np.int32)  # window offsets, sink sizes
    q = rng.standard_normal((4, hq, d)).astype(F16)
    k_off = np.array([0, 7, 3000, 11], np.int32)
    logical = np.array([kv[i] - info[1][i] + info[2][i] for i in range(4)])
    q_pos = (k_off + logical - 1).astype(np.int32)
    for length_info in (last, info):
        eo, el = np.zeros((4, hq, d), F16), np.zeros((4, hq), np.float32)
        with ok.inline_rope_scaling(rope_scaling):
            ok.decode(q, pages, ip, pv, length_info, k_off, q_pos, eo, el, 1, 1.0, 1e4, sm)
        go = torch.zeros((4, hq, d), dtype=torch.float16, device=DEV)
        gl = torch.zeros((4, hq), dtype=torch.float32, device=DEV)
        K.batch_decode_paged_kv(dev(q), dev(pages), i32(ip), i32(pv), i32(length_info), i32(k_off), i32(q_pos), go, gl, 1,
                                1.0, 1e4, sm, rope_scaling=rope_scaling)
        assert_close(host(go), eo, what="decode out, frequency variant")
        assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="decode lse, frequency variant")
    # paged prefill, causal
    ql = [7, 33, 70, 1]
    kvp = [5, 130, 200, 64]
    kvp = [max(a, b) for a, b in zip(kvp, ql)]
    pages, ip, pv, last, _, _ = build_paged_kv(rng, kvp, 40, hkv, 16, d)
    n = sum(ql)
    ind = np.concatenate([[0], np.cumsum(ql)]).astype(np.int32)
    qp = rng.standard_normal((n, hq, d)).astype(F16)
    pos = np.concatenate([k_off[i] + kvp[i] - ql[i] + np.arange(ql[i]) for i in range(4)]).astype(np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    with ok.inline_rope_scaling(rope_scaling):
        ok.prefill_paged(qp, ind, pages, ip, pv, last, k_off, pos, eo, el, 1, 1, 1.0, 1e4, sm)
    go = torch.zeros((n, hq, d), dtype=torch.float16, device=DEV)
    gl = torch.zeros((n, hq), dtype=torch.float32, device=DEV)
    K.batch_prefill_paged_kv(dev(qp), i32(ind), dev(pages), i32(ip), i32(pv), i32(last), i32(k_off), i32(pos), go, gl, 1, 1,
                             1.0, 1e4, sm, rope_scaling=rope_scaling)
    assert_close(host(go), eo, what="paged out, frequency variant")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="paged lse, frequency variant")
    # ragged prefill
    kr = rng.standard_normal((n, hkv, d)).astype(F16)
    vr = rng.standard_normal((n, hkv, d)).astype(F16)
    off = np.array([0, 50, 900, 3], np.int32)
    rpos = np.concatenate([off[i] + np.arange(ql[i]) for i in range(4)]).astype(np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    with ok.inline_rope_scaling(rope_scaling):
        ok.prefill_ragged(qp, ind, kr, vr, ind, rpos, off, eo, el, 1, 1, 1.0, 1e4, sm)
    go.zero_()
    gl.zero_()
    K.batch_prefill_ragged_kv(dev(qp), i32(ind), dev(kr), dev(vr), i32(ind), i32(rpos), i32(off), go, gl, 1, 1, 1.0, 1e4,
                              sm, rope_scaling=rope_scaling)
    assert_close(host(go), eo, what="ragged out, frequency variant")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="ragged lse, frequency variant")
    # ragged tree attention: positions are depths
    trees = [random_forest(rng, s_) for s_ in (7, 15, 33)]
    sizes = [len(t) for t in trees]
    nt = sum(sizes)
    tind = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    qt = rng.standard_normal((nt, hq, d)).astype(F16)
    kt = rng.standard_normal((nt, hkv, d)).astype(F16)
    vt = rng.standard_normal((nt, hkv, d)).astype(F16)
    mask = np.concatenate([tree_order(t) for t in trees])
    depth = []
    for i, t in enumerate(trees):
        dep = []
        for parent in t:
            dep.append(0 if parent == -1 else dep[parent] + 1)
        depth += [200 * i + x for x in dep]
    tpos = np.array(depth, np.int32)
    eo, el = np.zeros((nt, hq, d), F16), np.zeros((nt, hq), np.float32)
    with ok.inline_rope_scaling(rope_scaling):
        ok.tree_attn_ragged(qt, tind, kt, vt, tind, tpos, tind, mask, eo, el, 1, 1.0, 1e4, sm)
    go = torch.zeros((nt, hq, d), dtype=torch.float16, device=DEV)
    gl = torch.zeros((nt, hq), dtype=torch.float32, device=DEV)
    K.batch_tree_attn(dev(qt), i32(tind), dev(kt), dev(vt), i32(tind), i32(tpos), i32(tind), i32(mask), go, gl, 1, 1.0,
                      1e4, sm, rope_scaling=rope_scaling)
    assert_close(host(go), eo, what="tree out, frequency variant")
    assert_close(host(gl), el, atol=2e-3, rtol=1e-4, what="tree lse, frequency variant")
