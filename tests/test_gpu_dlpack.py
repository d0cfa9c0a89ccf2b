"""The DLPack-level entry points on the GPU, called the way the reference's cache calls its kernels:
every int32 auxiliary array is a view at a non-zero, 16-byte aligned byte_offset into ONE merged device
buffer (src/runtime/vm/attn_utils.h:1027-1035 of the reference), fp16 tensors are views into larger
allocations, and shapes travel in the tensors.  Results are checked against the CPU oracle with the
tolerances of tests/test_gpu_kernels.py; integer / byte work bit for bit."""
import numpy as np
import pytest
import torch

from oracle import kernels as ok
from tests.gpu_util import DEV, dev, host
from tests.util import REFERENCE_TREES, assert_close, build_paged_kv, random_forest, tree_order
from tvm_amd import KVError
from tvm_amd import dlpack as dl

pytestmark = pytest.mark.gpu
F16 = np.float16


class Merged:
    """One int32 device buffer holding every auxiliary array of a call at 16-byte aligned offsets,
    the first of them not at the start of the buffer."""

    def __init__(self, **arrays):
        cursor = 4  # in int32 elements: nothing sits at byte offset 0
        self.offsets, self.shapes = {}, {}
        parts = []
        for name, a in arrays.items():
            a = np.ascontiguousarray(a, dtype=np.int32)
            self.offsets[name] = cursor * 4
            self.shapes[name] = a.shape
            parts.append((cursor, a.reshape(-1)))
            cursor = (cursor + a.size + 3) // 4 * 4
        flat = np.full(cursor + 4, -12345, np.int32)
        for at, a in parts:
            flat[at:at + a.size] = a
        self.buffer = torch.from_numpy(flat).to(DEV)

    def __getitem__(self, name):
        assert self.offsets[name] > 0 and self.offsets[name] % 16 == 0
        return dl.view(self.buffer, self.offsets[name], self.shapes[name])


def offset_f16(a, pad=24):
    """An fp16 array as a view `pad` elements (48 bytes) into a larger device allocation."""
    a = np.ascontiguousarray(a, dtype=F16)
    flat = torch.zeros(a.size + 2 * pad, dtype=torch.float16, device=DEV)
    flat[pad:pad + a.size] = torch.from_numpy(a.reshape(-1)).to(DEV)
    return dl.view(flat, pad * 2, a.shape), flat, pad


def read_back(flat, pad, shape):
    n = int(np.prod(shape))
    return host(flat[pad:pad + n]).reshape(shape)


def outputs(rows, hq, d):
    out, out_flat, pad = offset_f16(np.full((rows, hq, d), 7.0, F16))
    lse = torch.full((rows, hq), 7.0, dtype=torch.float32, device=DEV)
    return out, lse, lambda: read_back(out_flat, pad, (rows, hq, d))


def test_decode_and_paged_prefill_through_merged_aux_views():
    rng = np.random.default_rng(100)
    hq, hkv, d = 32, 8, 128
    kv_lens = [0, 1, 16, 17, 300, 1000, 64]
    b = len(kv_lens)
    pages, indptr, values, last, _, _ = build_paged_kv(rng, kv_lens, 128, hkv, 16, d)
    # decode: one query per sequence
    q = rng.standard_normal((b, hq, d)).astype(F16)
    z = np.zeros(b, np.int32)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
    ok.decode(q, pages, indptr, values, last, z, z, eo, el, 0, 1.0, 1e4, d ** -0.5)
    aux = Merged(page_indptr=indptr, page_indices=values, length_info=last, k_rope_pos_offset=z, q_rope_position=z)
    q_dl, _, _ = offset_f16(q)
    pages_dl, _, _ = offset_f16(pages, pad=64)
    out, lse, get_out = outputs(b, hq, d)
    dl.call("batch_decode_paged_kv", q_dl, pages_dl, aux["page_indptr"], aux["page_indices"], aux["length_info"],
            aux["k_rope_pos_offset"], aux["q_rope_position"], out, dl.tensor(lse), 0, 1.0, 1e4, d ** -0.5)
    assert_close(get_out(), eo, what="dl decode out")
    assert_close(host(lse), el, atol=1e-3, rtol=1e-4, what="dl decode lse")
    # paged prefill: ragged query lengths, non-causal
    q_lens = [3, 1, 16, 5, 64, 30, 2]
    n = sum(q_lens)
    qo_indptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    q = rng.standard_normal((n, hq, d)).astype(F16)
    zq = np.zeros(n, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_paged(q, qo_indptr, pages, indptr, values, last, z, zq, eo, el, 0, 0, 1.0, 1e4, d ** -0.5)
    aux = Merged(q_rope_position=zq, qo_indptr=qo_indptr, page_indptr=indptr, page_indices=values, length_info=last,
                 k_rope_pos_offset=z)
    q_dl, _, _ = offset_f16(q)
    out, lse, get_out = outputs(n, hq, d)
    dl.call("batch_prefill_paged_kv", q_dl, aux["qo_indptr"], pages_dl, aux["page_indptr"], aux["page_indices"],
            aux["length_info"], aux["k_rope_pos_offset"], aux["q_rope_position"], out, dl.tensor(lse), 0, 0, 1.0, 1e4,
            d ** -0.5, 0)
    assert_close(get_out(), eo, what="dl paged prefill out")
    assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl paged prefill lse")


def test_sliding_window_form_is_selected_by_the_rank_of_length_info():
    """(3, batch) length_info = [last_page_len; sliding_window_offset; sink_size] -> the sliding-window kernels."""
    from tests.test_oracle_kernels import SLIDING_SPEC, sliding_case
    rng = np.random.default_rng(101)
    hq, hkv, d = 8, 2, 128
    pages, indptr, values, length_info, k_log, _ = sliding_case(rng, SLIDING_SPEC, hkv, d, npages=100)
    b = len(SLIDING_SPEC)
    q = rng.standard_normal((b, hq, d)).astype(F16)
    k_off = rng.integers(0, 300, size=b).astype(np.int32)
    q_pos = (k_off + np.array([len(k) for k in k_log]) - 1).astype(np.int32)
    eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
    ok.decode(q, pages, indptr, values, length_info, k_off, q_pos, eo, el, 1, 1.0, 1e4, d ** -0.5)
    aux = Merged(page_indptr=indptr, page_indices=values, length_info=length_info, k_rope_pos_offset=k_off,
                 q_rope_position=q_pos)
    assert aux.shapes["length_info"] == (3, b)
    q_dl, _, _ = offset_f16(q)
    pages_dl, _, _ = offset_f16(pages)
    out, lse, get_out = outputs(b, hq, d)
    dl.call("batch_decode_paged_kv", q_dl, pages_dl, aux["page_indptr"], aux["page_indices"], aux["length_info"],
            aux["k_rope_pos_offset"], aux["q_rope_position"], out, dl.tensor(lse), 1, 1.0, 1e4, d ** -0.5)
    assert_close(get_out(), eo, what="dl sliding decode out")
    assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl sliding decode lse")


def test_ragged_prefill_and_merge():
    rng = np.random.default_rng(102)
    hq, hkv, d = 8, 2, 64
    lens = [5, 64, 1, 130]
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F16) for h in (hq, hkv, hkv))
    zq, zb = np.zeros(n, np.int32), np.zeros(len(lens), np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.prefill_ragged(q, indptr, k, v, indptr, zq, zb, eo, el, 1, 0, 1.0, 1e4, d ** -0.5)
    aux = Merged(qo_indptr=indptr, kv_indptr=indptr, q_rope_position=zq, k_rope_pos_offset=zb)
    out, lse, get_out = outputs(n, hq, d)
    dl.call("batch_prefill_ragged_kv", offset_f16(q)[0], aux["qo_indptr"], offset_f16(k)[0], offset_f16(v)[0],
            aux["kv_indptr"], aux["q_rope_position"], aux["k_rope_pos_offset"], out, dl.tensor(lse), 1, 0, 1.0, 1e4,
            d ** -0.5)
    assert_close(get_out(), eo, what="dl ragged out")
    assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl ragged lse")
    # merge a second state into it, in place
    o2 = rng.standard_normal((n, hq, d)).astype(F16)
    l2 = rng.standard_normal((n, hq)).astype(np.float32)
    mo, ml = eo.copy(), el.copy()
    ok.merge_state_inplace(mo, ml, o2, l2)
    v_dl, v_flat, pad = offset_f16(eo)
    s = dev(el)
    dl.call("merge_state_inplace", v_dl, dl.tensor(s), offset_f16(o2)[0], dl.tensor(dev(l2)))
    assert_close(read_back(v_flat, pad, eo.shape), mo, what="dl merge out")
    assert_close(host(s), ml, atol=1e-3, rtol=1e-4, what="dl merge lse")


def test_tree_attention_slots():
    from tests.test_oracle_kernels import tree_paged_case
    rng = np.random.default_rng(103)
    hq, hkv, d = 8, 2, 128
    # slot 21: ragged
    trees = REFERENCE_TREES + [random_forest(rng, 40)]
    lens = [len(t) for t in trees]
    n = sum(lens)
    indptr = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    q, k, v = (rng.standard_normal((n, h, d)).astype(F16) for h in (hq, hkv, hkv))
    mask = np.concatenate([tree_order(t) for t in trees])
    q_pos = np.arange(n, dtype=np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.tree_attn_ragged(q, indptr, k, v, indptr, q_pos, indptr, mask, eo, el, 0, 1.0, 1e4, d ** -0.5)
    aux = Merged(qo_indptr=indptr, kv_indptr=indptr, q_rope_position=q_pos, mn_indptr=indptr, mask=np.asarray(mask).reshape(-1))
    out, lse, get_out = outputs(n, hq, d)
    dl.call("batch_tree_attn", offset_f16(q)[0], aux["qo_indptr"], offset_f16(k)[0], offset_f16(v)[0], aux["kv_indptr"],
            aux["q_rope_position"], aux["mn_indptr"], aux["mask"], out, dl.tensor(lse), 0, 1.0, 1e4, d ** -0.5)
    assert_close(get_out(), eo, what="dl tree ragged out")
    assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl tree ragged lse")
    # slot 20: paged
    prefix = [10, 0, 129]
    trees = [REFERENCE_TREES[0], REFERENCE_TREES[3], random_forest(rng, 31)]
    new_lens = [7, 14, 16]
    (pages, pindptr, pvalues, last, ks, vs, qindptr, q, tindptr, labels, masks) = tree_paged_case(
        rng, prefix, trees, new_lens, hq, hkv, d, npages=32)
    n = len(q)
    zb, zq = np.zeros(len(trees), np.int32), np.zeros(n, np.int32)
    eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
    ok.tree_attn_paged(q, qindptr, pages, pindptr, pvalues, last, zb, zq, eo, el, 0, 1.0, 1e4, d ** -0.5, tindptr, labels)
    aux = Merged(qo_indptr=qindptr, page_indptr=pindptr, page_indices=pvalues, length_info=last, k_rope_pos_offset=zb,
                 q_rope_position=zq, mn_indptr=tindptr, mask=np.asarray(labels).reshape(-1))
    out, lse, get_out = outputs(n, hq, d)
    dl.call("tree_attn_paged_kv", offset_f16(q)[0], aux["qo_indptr"], offset_f16(pages)[0], aux["page_indptr"],
            aux["page_indices"], aux["length_info"], aux["k_rope_pos_offset"], aux["q_rope_position"], out, dl.tensor(lse),
            0, 1.0, 1e4, d ** -0.5, aux["mn_indptr"], aux["mask"])
    assert_close(get_out(), eo, what="dl tree paged out")
    assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl tree paged lse")


def test_page_slots_bit_exact():
    """Slots 13, 25, 26, 27 and 24 -> 13 on one pool: append, partial page copy, compaction, gather."""
    rng = np.random.default_rng(104)
    hkv, d, ps, npages = 2, 128, 16, 12
    pages = rng.standard_normal((npages, 2, hkv, ps, d)).astype(F16)
    n = 9
    k, v = (rng.standard_normal((n, hkv, d)).astype(F16) for _ in range(2))
    pos = np.array([0, 17, -1, 33, 34, 35, 191, 100, -1], np.int32)
    expect = pages.copy()
    ok.transpose_append(expect, k, v, pos)
    pages_dl, pages_flat, pad = offset_f16(pages, pad=8)
    aux = Merged(position_map=pos)
    dl.call("transpose_append", pages_dl, offset_f16(k)[0], offset_f16(v)[0], aux["position_map"])
    assert np.array_equal(read_back(pages_flat, pad, pages.shape), expect)
    ok.copy_single_page(expect, 2, 7, 5)
    dl.call("copy_single_page", pages_dl, 2, 7, 5)
    assert np.array_equal(read_back(pages_flat, pad, pages.shape), expect)
    copy_indptr = np.array([0, 2, 2, 5], np.int32)
    src_dst = np.array([[33, 35, 100, 17, 191], [32, 33, 96, 97, 98]], np.int32)
    ok.compact_kv_copy(expect, copy_indptr, src_dst, 3)
    aux = Merged(copy_length_indptr=copy_indptr, copy_src_dst_pos=src_dst)
    dl.call("compact_kv_copy", pages_dl, aux["copy_length_indptr"], aux["copy_src_dst_pos"], 3)
    assert np.array_equal(read_back(pages_flat, pad, pages.shape), expect)
    gather = np.array([32, 33, 96, 97, 98, 0, 17], np.int32)
    ek, ev = np.zeros((3, len(gather), hkv, d), F16), np.zeros((3, len(gather), hkv, d), F16)
    ok.debug_get_kv(expect, gather, ek, ev, 1)
    k_dl, k_flat, kpad = offset_f16(np.zeros_like(ek))
    v_dl, v_flat, vpad = offset_f16(np.zeros_like(ev))
    aux = Merged(position_map=gather)
    dl.call("debug_get_kv", pages_dl, aux["position_map"], k_dl, v_dl, 1)
    assert np.array_equal(read_back(k_flat, kpad, ek.shape), ek) and np.array_equal(read_back(v_flat, vpad, ev.shape), ev)
    with pytest.raises(KVError, match="layer_id 3 is outside k_data's 3 layers"):
        dl.call("debug_get_kv", pages_dl, aux["position_map"], k_dl, v_dl, 3)


def test_mla_slots():
    rng = np.random.default_rng(105)
    hq, d_latent, d_rope, ps, npages = 16, 512, 64, 64, 8
    dqk = d_latent + d_rope
    pages = np.zeros((npages, ps, dqk), F16)
    kv_lens = [70, 128, 5]
    n_new = sum(kv_lens)
    kv = (rng.standard_normal((n_new, dqk)) * 0.5).astype(F16)
    order = rng.permutation(npages)
    indptr, values, last, pos, cursor = [0], [], [], [], 0
    for n in kv_lens:
        ids = order[cursor:cursor + (n + ps - 1) // ps]
        cursor += len(ids)
        values += [int(x) for x in ids]
        indptr.append(len(values))
        last.append((n - 1) % ps + 1)
        pos += [int(ids[t // ps]) * ps + t % ps for t in range(n)]
    expect = pages.copy()
    ok.transpose_append_mla(expect, kv, np.array(pos, np.int32))
    pages_dl, pages_flat, pad = offset_f16(pages, pad=8)
    aux = Merged(position_map=pos, qo_indptr=[0, 2, 3, 6], page_indptr=indptr, page_indices=values, length_info=last)
    dl.call("transpose_append_mla", pages_dl, offset_f16(kv)[0], aux["position_map"])
    assert np.array_equal(read_back(pages_flat, pad, pages.shape), expect)
    q = (rng.standard_normal((6, hq, dqk)) * 0.5).astype(F16)
    eo, el = np.zeros((6, hq, d_latent), F16), np.zeros((6, hq), np.float32)
    ok.prefill_paged_mla(q, np.array([0, 2, 3, 6], np.int32), expect, np.array(indptr, np.int32), np.array(values, np.int32),
                         np.array(last, np.int32), eo, el, 0, dqk ** -0.5)
    out, lse, get_out = outputs(6, hq, d_latent)
    dl.call("batch_prefill_paged_kv_mla", offset_f16(q)[0], aux["qo_indptr"], pages_dl, aux["page_indptr"],
            aux["page_indices"], aux["length_info"], out, dl.tensor(lse), 0, dqk ** -0.5)
    assert_close(get_out(), eo, what="dl mla out")
    assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl mla lse")
    gather = np.array(pos[:9], np.int32)
    ekv = np.zeros((2, 9, dqk), F16)
    ok.debug_get_kv_mla(expect, gather, ekv, 1)
    kv_dl, kv_flat, kpad = offset_f16(np.zeros_like(ekv))
    dl.call("debug_get_kv_mla", pages_dl, Merged(position_map=gather)["position_map"], kv_dl, 1)
    assert np.array_equal(read_back(kv_flat, kpad, ekv.shape), ekv)
    dl.call("copy_single_page", pages_dl, int(order[0]), int(order[7]), 9)
    ok.copy_single_page_mla(expect, int(order[0]), int(order[7]), 9)
    assert np.array_equal(read_back(pages_flat, pad, pages.shape), expect)


LLAMA3 = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 8192}
YARN = {"rope_type": "yarn", "factor": 40.0, "beta_fast": 32, "beta_slow": 1, "original_max_position_embeddings": 4096}
LONGROPE = {"rope_type": "longrope", "max_position_embeddings": 131072, "original_max_position_embeddings": 8}


@pytest.mark.parametrize("scaling,theta", [({}, 1e4), (LLAMA3, 5e5), (YARN, 1e4), (LONGROPE, 1e4)])
@pytest.mark.parametrize("d", [128, 64])
def test_fused_rope_slot_with_frequency_variants(scaling, theta, d):
    """Slot 24 with what the reference bakes into the kernel of a model; longrope also with its factor tensor,
    short factors for a call of up to original_max rows and long ones beyond."""
    rng = np.random.default_rng(106)
    hq, hkv = 8, 2
    longrope = scaling.get("rope_type") == "longrope"
    ext = np.concatenate([np.linspace(1.0, 8.0, d // 2), np.linspace(1.0, 1.3, d // 2)]).astype(np.float32)
    for n in (5, 13):
        pos = np.array([0, 1, 2, 3, 100, 511, 2047, 4096, 65535, 131071, 7, 9, 33], np.int32)[:n]
        qkv = rng.standard_normal((n, hq + 2 * hkv, d)).astype(F16)
        eq, ek, ev = np.zeros((n, hq, d), F16), np.zeros((n, hkv, d), F16), np.zeros((n, hkv, d), F16)
        ok.fused_rope_scaled(qkv, pos, eq, ek, ev, 1, scaling, theta=theta, scale=0.5, ext_factors=ext if longrope else None)
        aux = Merged(q_rope_position_map=pos)
        q, q_flat, qp = offset_f16(np.zeros_like(eq))
        k, k_flat, kp = offset_f16(np.zeros_like(ek))
        v, v_flat, vp = offset_f16(np.zeros_like(ev))
        dl.call("fused_rope", offset_f16(qkv)[0], aux["q_rope_position_map"], q, k, v, 1,
                dl.tensor(dev(ext)) if longrope else None, dl.RopeScaling.from_dict(scaling), 0.5, theta)
        assert np.array_equal(read_back(v_flat, vp, ev.shape), ev)
        gq, gk = read_back(q_flat, qp, eq.shape), read_back(k_flat, kp, ek.shape)
        assert_close(gq, eq, atol=2e-3, rtol=2e-3, what="rope q")
        assert_close(gk, ek, atol=2e-3, rtol=2e-3, what="rope k")
        assert np.mean(gq == eq) > 0.98, np.mean(gq == eq)


@pytest.mark.parametrize("scaling,theta", [(LLAMA3, 5e5), (YARN, 1e4)])
def test_attention_slots_with_a_frequency_variant_inside_the_kernel(scaling, theta):
    """Slots 17, 16, 15 and 21 as a model with inline RoPE and a frequency variant gets them: the variant is a
    property of the kernel function (the reference compiles it in), here an argument of the *_scaled entry
    points.  The oracle's kernels rotate with the same variant."""
    rng = np.random.default_rng(107)
    hq, hkv, d = 8, 2, 128
    rs = dl.RopeScaling.from_dict(scaling)
    kv_lens = [1, 17, 300, 64]
    b = len(kv_lens)
    pages, indptr, values, last, _, _ = build_paged_kv(rng, kv_lens, 40, hkv, 16, d)
    pages_dl = offset_f16(pages, pad=64)[0]
    k_off = rng.integers(0, 3000, size=b).astype(np.int32)
    with ok.inline_rope_scaling(scaling):
        # slot 17
        q = rng.standard_normal((b, hq, d)).astype(F16)
        q_pos = (k_off + np.array(kv_lens) - 1).astype(np.int32)
        eo, el = np.zeros((b, hq, d), F16), np.zeros((b, hq), np.float32)
        ok.decode(q, pages, indptr, values, last, k_off, q_pos, eo, el, 1, 0.5, theta, d ** -0.5)
        aux = Merged(page_indptr=indptr, page_indices=values, length_info=last, k_rope_pos_offset=k_off, q_rope_position=q_pos)
        out, lse, get_out = outputs(b, hq, d)
        dl.call("batch_decode_paged_kv_scaled", offset_f16(q)[0], pages_dl, aux["page_indptr"], aux["page_indices"],
                aux["length_info"], aux["k_rope_pos_offset"], aux["q_rope_position"], out, dl.tensor(lse), 1, 0.5, theta,
                d ** -0.5, rs)
        assert_close(get_out(), eo, what="dl scaled decode out")
        assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl scaled decode lse")
        # slot 16, causal
        q_lens = [1, 5, 40, 64]
        n = sum(q_lens)
        qo_indptr = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
        q = rng.standard_normal((n, hq, d)).astype(F16)
        q_pos = np.concatenate([k_off[i] + kv_lens[i] - q_lens[i] + np.arange(q_lens[i]) for i in range(b)]).astype(np.int32)
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
        ok.prefill_paged(q, qo_indptr, pages, indptr, values, last, k_off, q_pos, eo, el, 1, 1, 0.5, theta, d ** -0.5)
        aux = Merged(q_rope_position=q_pos, qo_indptr=qo_indptr, page_indptr=indptr, page_indices=values, length_info=last,
                     k_rope_pos_offset=k_off)
        out, lse, get_out = outputs(n, hq, d)
        dl.call("batch_prefill_paged_kv_scaled", offset_f16(q)[0], aux["qo_indptr"], pages_dl, aux["page_indptr"],
                aux["page_indices"], aux["length_info"], aux["k_rope_pos_offset"], aux["q_rope_position"], out, dl.tensor(lse),
                1, 1, 0.5, theta, d ** -0.5, 0, rs)
        assert_close(get_out(), eo, what="dl scaled paged prefill out")
        assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl scaled paged prefill lse")
        # slot 15, causal
        lens = [33, 1, 70]
        n = sum(lens)
        ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        q = rng.standard_normal((n, hq, d)).astype(F16)
        k, v = (rng.standard_normal((n, hkv, d)).astype(F16) for _ in range(2))
        off = rng.integers(0, 3000, size=len(lens)).astype(np.int32)
        q_pos = np.concatenate([off[i] + np.arange(lens[i]) for i in range(len(lens))]).astype(np.int32)
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
        ok.prefill_ragged(q, ind, k, v, ind, q_pos, off, eo, el, 1, 1, 0.5, theta, d ** -0.5)
        aux = Merged(qo_indptr=ind, kv_indptr=ind, q_rope_position=q_pos, k_rope_pos_offset=off)
        out, lse, get_out = outputs(n, hq, d)
        dl.call("batch_prefill_ragged_kv_scaled", offset_f16(q)[0], aux["qo_indptr"], offset_f16(k)[0], offset_f16(v)[0],
                aux["kv_indptr"], aux["q_rope_position"], aux["k_rope_pos_offset"], out, dl.tensor(lse), 1, 1, 0.5, theta,
                d ** -0.5, rs)
        assert_close(get_out(), eo, what="dl scaled ragged out")
        assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl scaled ragged lse")
        # slot 21
        trees = [REFERENCE_TREES[0], random_forest(rng, 20)]
        lens = [len(t) for t in trees]
        n = sum(lens)
        ind = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        q, k, v = (rng.standard_normal((n, h, d)).astype(F16) for h in (hq, hkv, hkv))
        mask = np.concatenate([tree_order(t) for t in trees])
        q_pos = rng.integers(0, 3000, size=n).astype(np.int32)
        eo, el = np.zeros((n, hq, d), F16), np.zeros((n, hq), np.float32)
        ok.tree_attn_ragged(q, ind, k, v, ind, q_pos, ind, mask, eo, el, 1, 0.5, theta, d ** -0.5)
        aux = Merged(qo_indptr=ind, kv_indptr=ind, q_rope_position=q_pos, mn_indptr=ind, mask=np.asarray(mask).reshape(-1))
        out, lse, get_out = outputs(n, hq, d)
        dl.call("batch_tree_attn_scaled", offset_f16(q)[0], aux["qo_indptr"], offset_f16(k)[0], offset_f16(v)[0],
                aux["kv_indptr"], aux["q_rope_position"], aux["mn_indptr"], aux["mask"], out, dl.tensor(lse), 1, 0.5, theta,
                d ** -0.5, rs)
        assert_close(get_out(), eo, what="dl scaled tree out")
        assert_close(host(lse), el, atol=2e-3, rtol=1e-4, what="dl scaled tree lse")
