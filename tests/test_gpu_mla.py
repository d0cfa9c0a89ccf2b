"""GPU parity of the MLA latent-cache path: the paged MLA kernel against the CPU oracle on
identical inputs (decode-shaped calls take the split-KV route, prefill-shaped calls do not), and
the cache-level flow of the reference's MLA test (append_mla_kv, self_attention on expanded
192/128-dim heads, cross_attention on the absorbed query, merge) against the definition of MLA:
expand the latent with w_kv and run plain multi-head attention
(tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_mla_tir.py:293-398).

Relative to "the reference's llvm kernels" MLA parity is unpinned by construction: the reference
has no llvm MLA kernel; the oracle function is pinned to the closed form in
tests/test_oracle_kernels.py."""
import numpy as np
import pytest
import torch

from oracle import closed_form as cf
from oracle import kernels as ok
from tests.gpu_util import DEV, GpuCache, dev, host, i32
from tests.util import assert_close
from tvm_amd import kernels as K

pytestmark = pytest.mark.gpu
F16 = np.float16
H, D_LAT, D_ROPE, D_NOPE, D_V = 128, 512, 64, 128, 128
D_QK = D_LAT + D_ROPE


def _latent_pool(rng, kv_lens, ps, npages, ramp=0.0):
    """ramp > 0: the rope part of token t is ramp * t in every feature, so that against a query
    whose rope part is all ones the scores grow along the sequence without bound."""
    pages = np.zeros((npages, ps, D_QK), F16)
    order = rng.permutation(npages)
    indptr, values, last, rows = [0], [], [], []
    cursor = 0
    for n in kv_lens:
        npg = (n + ps - 1) // ps
        ids = order[cursor:cursor + npg]
        cursor += npg
        lat = (rng.standard_normal((n, D_QK)) * 0.5).astype(F16)
        if ramp:
            lat[:, D_LAT:] = (ramp * np.arange(n, dtype=np.float32))[:, None].astype(F16)
        for t in range(n):
            pages[ids[t // ps], t % ps] = lat[t]
        values.extend(int(x) for x in ids)
        indptr.append(len(values))
        last.append(0 if n == 0 else (n - 1) % ps + 1)
        rows.append(lat)
    return pages, np.array(indptr, np.int32), np.array(values, np.int32), np.array(last, np.int32), rows


def _mla_both(rng, kv_lens, q_lens, ps, npages, causal=0, heads=H, ramp=0.0):
    pages, pindptr, pvalues, last, _ = _latent_pool(rng, kv_lens, ps, npages, ramp)
    n = sum(q_lens)
    qindptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = (rng.standard_normal((n, heads, D_QK)) * 0.5).astype(F16)
    if ramp:
        q[:, :, D_LAT:] = 1
    eo, el = np.zeros((n, heads, D_LAT), F16), np.zeros((n, heads), np.float32)
    sm = (D_NOPE + D_ROPE) ** -0.5
    ok.prefill_paged_mla(q, qindptr, pages, pindptr, pvalues, last, eo, el, causal, sm, d_latent=D_LAT)
    go = torch.full((n, heads, D_LAT), 7.0, dtype=torch.float16, device=DEV)
    gl = torch.full((n, heads), 7.0, dtype=torch.float32, device=DEV)
    K.batch_prefill_paged_kv_mla(dev(q), i32(qindptr), dev(pages), i32(pindptr), i32(pvalues), i32(last), go, gl,
                                 causal, sm)
    return host(go), host(gl), eo, el


@pytest.mark.parametrize("ps", [64, 16])
def test_mla_decode_shaped_split_kv(ps):
    rng = np.random.default_rng(30)
    kv_lens = [1, 63, 64, 65, 200, 1000, 0, 129]
    go, gl, eo, el = _mla_both(rng, kv_lens, [1] * len(kv_lens), ps, npages=(40 if ps == 64 else 130))
    assert_close(go, eo, what="mla decode out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla decode lse")
    assert not go[6].any() and np.all(gl[6] == np.float32(-5e4))


def test_mla_decode_one_long_sequence_many_chunks():
    """One sequence over all workgroups: more than a hundred chunks, merged several at a time."""
    rng = np.random.default_rng(31)
    go, gl, eo, el = _mla_both(rng, [20000], [1], 64, npages=320)
    assert_close(go, eo, what="mla long decode out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla long decode lse")


def test_mla_decode_batch_beyond_one_sequence_per_lane():
    """100 sequences: the split plan keeps two sequences per lane; lengths from empty to a few chunks."""
    rng = np.random.default_rng(32)
    kv_lens = [int(x) for x in rng.integers(0, 700, size=100)]
    kv_lens[3], kv_lens[64], kv_lens[99] = 0, 1, 2500
    go, gl, eo, el = _mla_both(rng, kv_lens, [1] * 100, 64, npages=700)
    assert_close(go, eo, what="mla wide decode out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla wide decode lse")
    assert not go[3].any() and np.all(gl[3] == np.float32(-5e4))


def test_mla_decode_batch_beyond_one_split_launch():
    """200 long sequences: more than one split launch plans, so the step is cut into two split launches
    over slices of the index arrays; a few empty and short sequences among them."""
    rng = np.random.default_rng(38)
    kv_lens = [int(x) for x in rng.integers(1030, 1300, size=200)]
    kv_lens[0], kv_lens[99], kv_lens[100], kv_lens[199] = 0, 1, 2600, 7
    go, gl, eo, el = _mla_both(rng, kv_lens, [1] * 200, 64, npages=8 + sum((n + 63) // 64 for n in kv_lens), heads=16)
    assert_close(go, eo, what="mla two-launch decode out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla two-launch decode lse")
    assert not go[0].any() and np.all(gl[0] == np.float32(-5e4))


@pytest.mark.parametrize("causal", [1, 0])
def test_mla_draft_verification_beyond_one_split_launch(causal):
    """60 long sequences with 1 to 5 tokens each, about 190 tokens: more one-token sequences than one split
    launch plans, so the call is cut into parts of consecutive tokens (sequences straddle the parts)."""
    rng = np.random.default_rng(39 + causal)
    kv_lens = [int(x) for x in rng.integers(1030, 1300, size=60)]
    q_lens = [int(x) for x in rng.integers(1, 6, size=60)]
    kv_lens[7], q_lens[7] = 2600, 5
    go, gl, eo, el = _mla_both(rng, kv_lens, q_lens, 64, npages=8 + sum((n + 63) // 64 for n in kv_lens), causal=causal,
                               heads=16)
    assert 128 < sum(q_lens) <= 512
    assert_close(go, eo, what="mla verify in parts out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla verify in parts lse")


def test_mla_as_many_tokens_as_sequences_but_not_a_decode_step():
    """total_q == batch makes the launcher split the KV; sequences that do not have exactly one
    query token must still come out right (they are done unsplit by the workgroups of chunk 0)."""
    rng = np.random.default_rng(33)
    kv_lens, q_lens = [700, 50, 300, 420], [2, 0, 1, 1]
    go, gl, eo, el = _mla_both(rng, kv_lens, q_lens, 64, npages=30)
    assert_close(go, eo, what="mla mixed out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla mixed lse")


@pytest.mark.parametrize("causal", [1, 0])
def test_mla_few_tokens_per_sequence_split_kv(causal):
    """A draft to verify (a few tokens per sequence) and a short chunk late in a long sequence have as few
    row tiles as a decode step: the launcher plans every token as a one-token sequence of its own (under
    the causal mask token j of n sees the first L - n + j + 1 keys) and splits the KV."""
    rng = np.random.default_rng(36 + causal)
    for kv_lens, q_lens in (([1500, 64, 700, 65, 4, 900, 130, 33], [4, 4, 4, 4, 4, 4, 4, 4]),   # verify
                            ([3000], [64]),                                                       # one short chunk
                            ([900, 5, 300, 0, 420, 77], [3, 5, 0, 2, 1, 7])):                    # ragged, empty sequences
        if causal:
            kv_lens = [max(k, q) for k, q in zip(kv_lens, q_lens)]
        heads = 64 if len(kv_lens) == 1 else 128   # the long single chunk is most of the oracle's time
        go, gl, eo, el = _mla_both(rng, kv_lens, q_lens, 64, npages=8 + sum((n + 63) // 64 for n in kv_lens), causal=causal,
                                   heads=heads)
        assert_close(go, eo, what=f"mla few tokens out, q_lens {q_lens}")
        assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"mla few tokens lse, q_lens {q_lens}")


def test_mla_decode_heads_not_a_multiple_of_the_row_tile():
    rng = np.random.default_rng(34)
    kv_lens = [900, 33, 257]
    for heads in (16, 160):
        go, gl, eo, el = _mla_both(rng, kv_lens, [1, 1, 1], 16, npages=80, heads=heads)
        assert_close(go, eo, what=f"mla decode out, {heads} heads")
        assert_close(gl, el, atol=2e-3, rtol=1e-4, what=f"mla decode lse, {heads} heads")


@pytest.mark.parametrize("causal", [0, 1])
def test_mla_prefill_shaped(causal):
    rng = np.random.default_rng(31)
    kv_lens, q_lens = [300, 40, 0, 77], [33, 5, 2, 77]
    if causal:
        kv_lens = [max(k, q) for k, q in zip(kv_lens, q_lens)]
    go, gl, eo, el = _mla_both(rng, kv_lens, q_lens, 64, npages=16, causal=causal, heads=16)
    assert_close(go, eo, what="mla prefill out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla prefill lse")


@pytest.mark.parametrize("causal", [0, 1])
def test_mla_scores_that_keep_growing_move_the_reference_point(causal):
    """The running softmax only moves its reference point (and rescales O, which the kernel does on
    the accumulation registers from assembly) when a score exceeds it by more than 2^8.  Random
    inputs do that in the first tile only; here the score grows by ~10 in the exponent per 32-token
    tile, so every tile rescales, in prefill- and in decode-shaped (split-KV) calls."""
    rng = np.random.default_rng(35)
    kv_lens, q_lens = [330, 96, 64, 200], [40, 1, 3, 200]
    go, gl, eo, el = _mla_both(rng, kv_lens, q_lens, 64, npages=16, causal=causal, heads=16, ramp=0.047)
    assert_close(go, eo, what="mla growing scores out")
    assert_close(gl, el, atol=5e-3, rtol=1e-4, what="mla growing scores lse")
    kv_lens = [700, 1300, 129]
    go, gl, eo, el = _mla_both(rng, kv_lens, [1, 1, 1], 64, npages=40, ramp=0.02)
    assert_close(go, eo, what="mla growing scores decode out")
    assert_close(gl, el, atol=5e-3, rtol=1e-4, what="mla growing scores decode lse")


def test_mla_page_size_that_is_not_a_power_of_two():
    rng = np.random.default_rng(36)
    kv_lens, q_lens = [300, 47, 0, 100], [33, 5, 2, 100]
    go, gl, eo, el = _mla_both(rng, kv_lens, q_lens, 24, npages=24, causal=1, heads=16)
    assert_close(go, eo, what="mla page 24 out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla page 24 lse")
    go, gl, eo, el = _mla_both(rng, [500, 90], [1, 1], 40, npages=20)
    assert_close(go, eo, what="mla page 40 decode out")
    assert_close(gl, el, atol=2e-3, rtol=1e-4, what="mla page 40 decode lse")


def test_mla_cache_flow_matches_the_definition():
    """Prefill a chunk on a cached prefix, then decode one token, through the cache verbs."""
    rng = np.random.default_rng(32)
    heads, layers, ps = 16, 1, 64
    sm = (D_NOPE + D_ROPE) ** -0.5
    w_kv = (rng.standard_normal((D_LAT, heads * (D_NOPE + D_V))) * 0.04).astype(np.float64)
    w = w_kv.reshape(D_LAT, heads, D_NOPE + D_V)
    w_uk, w_uv = w[..., :D_NOPE], w[..., D_NOPE:]
    cache = GpuCache([4, 1024, 256, ps, 0], layers, heads, 1, D_QK, D_LAT, attn_kinds=[1], rope_mode=0)
    cached = {0: np.zeros((0, D_QK), F16), 1: np.zeros((0, D_QK), F16)}
    cache.add_sequence(0)
    cache.add_sequence(1)
    for lens in ([70, 3], [37, 90], [1, 1]):
        ids = [0, 1]
        cache.begin_forward(ids, lens)
        total = sum(lens)
        q = (rng.standard_normal((total, heads, D_NOPE + D_ROPE)) * 0.5).astype(F16)
        kv = (rng.standard_normal((total, D_QK)) * 0.5).astype(F16)
        is_decode = all(n == 1 for n in lens)
        all_new = all(cached[s].shape[0] == 0 for s in ids)
        cache.append_mla_kv(0, kv)
        o1 = np.zeros((total, heads, D_V), F16)
        l1 = np.zeros((total, heads), np.float32)
        if not is_decode:
            k_full, v_full = cf.mla_expand(kv, w_kv, heads, D_NOPE, D_V)
            cache.self_attention(0, sm, q, k_full.astype(F16), v_full.astype(F16), o1, l1)
        if not all_new or is_decode:
            q_abs = np.concatenate([np.einsum("qhn,lhn->qhl", q[..., :D_NOPE].astype(np.float64), w_uk),
                                    q[..., D_NOPE:].astype(np.float64)], axis=-1).astype(F16)
            o2 = np.zeros((total, heads, D_LAT), F16)
            l2 = np.zeros((total, heads), np.float32)
            cache.cross_attention(0, sm, q_abs, o2, l2)
            cross = np.einsum("qhl,lhv->qhv", o2.astype(np.float64), w_uv).astype(F16)
            if is_decode:
                o1 = cross
            else:
                cache.merge_attn_output_inplace(o1, l1, cross, l2)
        cache.end_forward()
        cursor = 0
        for sid, n in zip(ids, lens):
            cached[sid] = np.concatenate([cached[sid], kv[cursor:cursor + n]])
            k_seq, v_seq = cf.mla_expand(cached[sid], w_kv, heads, D_NOPE, D_V)
            k_seq = k_seq.astype(F16) if not is_decode else k_seq
            expected, _ = cf.attention(q[cursor:cursor + n], k_seq, v_seq, sm, causal=True)
            assert_close(o1[cursor:cursor + n], expected, atol=1e-2, rtol=2e-2, what=f"mla flow seq {sid} lens {lens}")
            back = np.zeros((layers, cached[sid].shape[0], D_QK), F16)
            cache.debug_get_kv_mla(sid, 0, cached[sid].shape[0], back)
            assert np.array_equal(back[0], cached[sid])
            cursor += n
