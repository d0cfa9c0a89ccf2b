"""Python face of the kernel launchers of libtvmkv.so.

Function names and positional arguments are those of the reference's kernels
(python/tvm/relax/frontend/nn/llm/_page_kernels.py, _decode_kernels.py, _prefill_kernels.py,
position_embedding.py) as the cache calls them (src/runtime/vm/attn_backend.h:239-242,
:392-395, :511-514; src/runtime/vm/paged_kv_cache.cc:728, :1361-1372, :1550, :1718, :2292).
Tensors are torch tensors in device memory; shapes are read from them the way the reference's
``T.match_buffer`` does.  Launches go to torch's current stream.
"""
import ctypes

import torch

from ._lib import KVError, check, lib


def _p(t):
    if t is None:
        return ctypes.c_void_p(0)
    if not t.is_contiguous():
        raise KVError(-1, "kernel arguments must be contiguous")
    if not t.is_cuda:
        raise KVError(-4, "kernel arguments must live in device memory")
    return ctypes.c_void_p(t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _f16(*tensors):
    for t in tensors:
        if t.dtype != torch.float16:
            raise KVError(-2, f"only float16 K/V/Q data is built, got {t.dtype}")


def _i32(*tensors):
    for t in tensors:
        if t is not None and t.dtype != torch.int32:
            raise KVError(-1, f"index arrays must be int32, got {t.dtype}")


def fused_rope(qkv, position_map, q, k, v, apply_rope, rope_scale=1.0, rope_theta=1e4):
    _f16(qkv, q, k, v)
    _i32(position_map)
    n, _, d = qkv.shape
    check(lib().tvmkv_fused_rope(_p(qkv), _p(position_map), _p(q), _p(k), _p(v), int(apply_rope), n, q.shape[1],
                                 k.shape[1], d, float(rope_scale), float(rope_theta), _stream()))


def fused_rope_scaled(qkv, position_map, q, k, v, apply_rope, rope_scaling, rope_scale=1.0, rope_theta=1e4,
                      rope_ext_factors=None):
    """fused_rope with one of the reference's frequency variants: rope_scaling is the reference's dictionary
    (rope_type llama3 / longrope / yarn and its parameters, position_embedding.py:258-299); rope_ext_factors the
    float32 device tensor of a longrope model (long factors, then short ones)."""
    from .dlpack import RopeScaling
    _f16(qkv, q, k, v)
    _i32(position_map)
    if rope_ext_factors is not None and rope_ext_factors.dtype != torch.float32:
        raise KVError(-1, "rope_ext_factors must be float32")
    n, _, d = qkv.shape
    scaling = RopeScaling.from_dict(rope_scaling)
    check(lib().tvmkv_fused_rope_scaled(_p(qkv), _p(position_map), _p(q), _p(k), _p(v), int(apply_rope),
                                        _p(rope_ext_factors), ctypes.c_void_p(ctypes.addressof(scaling)), n, q.shape[1],
                                        k.shape[1], d, float(rope_scale), float(rope_theta), _stream()))


def fused_rope_append(qkv, position_map, q, k, v, apply_rope, pages, append_position_map, rope_scale=1.0,
                      rope_theta=1e4):
    """fused_rope and tir_kv_cache_transpose_append in one launch.  q=None: the q rows are not written
    (batch_prefill_cached_and_new_kv_fused_q reads and rotates them from qkv)."""
    _f16(qkv, k, v, pages)
    if q is not None:
        _f16(q)
    _i32(position_map, append_position_map)
    n, _, d = qkv.shape
    num_pages, _, hkv, ps, _ = pages.shape
    check(lib().tvmkv_fused_rope_append(_p(qkv), _p(position_map), _p(q), _p(k), _p(v), int(apply_rope), _p(pages),
                                        _p(append_position_map), n, qkv.shape[1] - 2 * k.shape[1], k.shape[1], d,
                                        num_pages, ps, float(rope_scale), float(rope_theta), _stream()))


def tir_kv_cache_transpose_append(pages, k_data, v_data, position_map):
    _f16(pages, k_data, v_data)
    _i32(position_map)
    num_pages, _, hkv, ps, d = pages.shape
    check(lib().tvmkv_kv_cache_transpose_append(_p(pages), _p(k_data), _p(v_data), _p(position_map),
                                                position_map.shape[0], num_pages, hkv, ps, d, _stream()))


def tir_kv_cache_transpose_append_mla(pages, kv_data, position_map):
    _f16(pages, kv_data)
    _i32(position_map)
    num_pages, ps, d = pages.shape
    check(lib().tvmkv_kv_cache_transpose_append_mla(_p(pages), _p(kv_data), _p(position_map),
                                                    position_map.shape[0], num_pages, ps, d, _stream()))


def _scaling_arg(rope_scaling):
    """The reference's rope_scaling dictionary (position_embedding.py:258-299) as the C description, kept
    alive by the caller for the duration of the call; None = the default frequencies."""
    from .dlpack import RopeScaling
    scaling = RopeScaling.from_dict(rope_scaling)
    return scaling, ctypes.c_void_p(ctypes.addressof(scaling))


def batch_prefill_ragged_kv(q, q_indptr, k, v, kv_indptr, q_rope_position, k_rope_pos_offset, output, lse,
                            causal, rotary_mode, rope_scale, rope_theta, sm_scale, rope_scaling=None):
    """rope_scaling: the frequency variant of the in-kernel RoPE (rotary_mode = 1), the reference's dictionary."""
    _f16(q, k, v, output)
    _i32(q_indptr, kv_indptr, q_rope_position, k_rope_pos_offset)
    args = (_p(q), _p(q_indptr), _p(k), _p(v), _p(kv_indptr), _p(q_rope_position), _p(k_rope_pos_offset), _p(output),
            _p(lse), int(causal), int(rotary_mode), float(rope_scale), float(rope_theta), float(sm_scale),
            q_indptr.shape[0] - 1, q.shape[0], q.shape[1], k.shape[1], q.shape[2], v.shape[2])
    if rope_scaling:
        keep, ptr = _scaling_arg(rope_scaling)
        check(lib().tvmkv_batch_prefill_ragged_kv_scaled(*args, ptr, _stream()))
    else:
        check(lib().tvmkv_batch_prefill_ragged_kv(*args, _stream()))


def batch_prefill_paged_kv(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset,
                           q_rope_position, output, lse, causal, rotary_mode, rope_scale, rope_theta, sm_scale,
                           sliding_window_size=1024, merge_into=False, rope_scaling=None):
    """merge_into: output / lse hold an attention state of the same rows; merge into it instead of
    overwriting (one launch for the paged kernel and merge_state_inplace).  rope_scaling: the frequency
    variant of the in-kernel RoPE (rotary_mode = 1), the reference's dictionary."""
    _f16(q, pages, output)
    _i32(q_indptr, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position)
    num_pages, _, hkv, ps, d = pages.shape
    args = (_p(q), _p(q_indptr), _p(pages), _p(page_indptr), _p(page_values), _p(length_info), _p(k_rope_pos_offset),
            _p(q_rope_position), _p(output), _p(lse), int(causal), int(rotary_mode), float(rope_scale),
            float(rope_theta), float(sm_scale), q_indptr.shape[0] - 1, q.shape[0], page_values.shape[0], num_pages,
            q.shape[1], hkv, d, ps, int(length_info.dim() == 2), int(sliding_window_size))
    if rope_scaling:
        keep, ptr = _scaling_arg(rope_scaling)
        check(lib().tvmkv_batch_prefill_paged_kv_scaled(*args, int(bool(merge_into)), ptr, _stream()))
    else:
        fn = lib().tvmkv_batch_prefill_paged_kv_merge if merge_into else lib().tvmkv_batch_prefill_paged_kv
        check(fn(*args, _stream()))


def batch_prefill_cached_and_new_kv(q, q_indptr, k, v, pages, page_indptr, page_values, last_page_len, output, lse,
                                    sm_scale):
    """Ragged causal self-attention over the new tokens, paged attention over the cached ones and
    the merge of the two, in one pass."""
    _f16(q, k, v, pages, output)
    _i32(q_indptr, page_indptr, page_values, last_page_len)
    num_pages, _, hkv, ps, d = pages.shape
    check(lib().tvmkv_batch_prefill_cached_and_new_kv(
        _p(q), _p(q_indptr), _p(k), _p(v), _p(pages), _p(page_indptr), _p(page_values), _p(last_page_len),
        _p(output), _p(lse), float(sm_scale), q_indptr.shape[0] - 1, q.shape[0], page_values.shape[0], num_pages,
        q.shape[1], hkv, d, ps, _stream()))


def batch_prefill_cached_and_new_kv_fused_q(qkv, q_rope_position, apply_rope, rope_scale, rope_theta, q_indptr, k, v,
                                            pages, page_indptr, page_values, last_page_len, output, lse, sm_scale):
    """batch_prefill_cached_and_new_kv with the queries read from the fused qkv tensor and rotated inside
    the kernel."""
    _f16(qkv, k, v, pages, output)
    _i32(q_rope_position, q_indptr, page_indptr, page_values, last_page_len)
    num_pages, _, hkv, ps, d = pages.shape
    hq = qkv.shape[1] - 2 * hkv
    check(lib().tvmkv_batch_prefill_cached_and_new_kv_fused_q(
        _p(qkv), _p(q_rope_position), int(apply_rope), float(rope_scale), float(rope_theta), _p(q_indptr), _p(k),
        _p(v), _p(pages), _p(page_indptr), _p(page_values), _p(last_page_len), _p(output), _p(lse), float(sm_scale),
        q_indptr.shape[0] - 1, qkv.shape[0], page_values.shape[0], num_pages, hq, hkv, d, ps, _stream()))


def fused_decode_step(qkv, pages, page_indptr, page_values, last_page_len, q_rope_position, append_position_map,
                      output, lse, apply_rope, rope_scale, rope_theta, sm_scale):
    """One launch for the decode step of a layer: split of qkv, RoPE, append of the new k / v rows and
    decode attention (tvmkv_fused_decode_step); the page table covers the new tokens."""
    _f16(qkv, pages, output)
    _i32(page_indptr, page_values, last_page_len, q_rope_position, append_position_map)
    num_pages, _, hkv, ps, d = pages.shape
    hq = qkv.shape[1] - 2 * hkv
    check(lib().tvmkv_fused_decode_step(
        _p(qkv), _p(pages), _p(page_indptr), _p(page_values), _p(last_page_len), _p(q_rope_position),
        _p(append_position_map), _p(output), _p(lse), int(apply_rope), float(rope_scale), float(rope_theta),
        float(sm_scale), qkv.shape[0], page_values.shape[0], num_pages, hq, hkv, d, ps, _stream()))


def batch_decode_paged_kv(q, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position,
                          output, lse, rotary_mode, rope_scale, rope_theta, sm_scale, noalloc=False, rope_scaling=None):
    """noalloc=True calls the entry point that takes its scratch memory from the library's built-in
    per-device array instead of allocating (tvmkv_batch_decode_paged_kv_noalloc).  rope_scaling: the
    frequency variant of the in-kernel RoPE (rotary_mode = 1), the reference's dictionary."""
    _f16(q, pages, output)
    _i32(page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position)
    num_pages, _, hkv, ps, d = pages.shape
    args = (_p(q), _p(pages), _p(page_indptr), _p(page_values), _p(length_info), _p(k_rope_pos_offset),
            _p(q_rope_position), _p(output), _p(lse), int(rotary_mode), float(rope_scale), float(rope_theta),
            float(sm_scale), q.shape[0], page_values.shape[0], num_pages, q.shape[1], hkv, d, ps,
            int(length_info.dim() == 2))
    if rope_scaling:
        keep, ptr = _scaling_arg(rope_scaling)
        check(lib().tvmkv_batch_decode_paged_kv_scaled(*args, ptr, _stream()))
        return
    entry = lib().tvmkv_batch_decode_paged_kv_noalloc if noalloc else lib().tvmkv_batch_decode_paged_kv
    check(entry(*args, _stream()))


def batch_tree_attn(q, q_indptr, k, v, kv_indptr, q_rope_position, mn_indptr, mask, output, lse, rotary_mode,
                    rope_scale, rope_theta, sm_scale, rope_scaling=None):
    _f16(q, k, v, output)
    _i32(q_indptr, kv_indptr, q_rope_position, mn_indptr, mask)
    args = (_p(q), _p(q_indptr), _p(k), _p(v), _p(kv_indptr), _p(q_rope_position), _p(mn_indptr), _p(mask), _p(output),
            _p(lse), int(rotary_mode), float(rope_scale), float(rope_theta), float(sm_scale), q_indptr.shape[0] - 1,
            q.shape[0], q.shape[1], k.shape[1], q.shape[2])
    if rope_scaling:
        keep, ptr = _scaling_arg(rope_scaling)
        check(lib().tvmkv_batch_tree_attn_scaled(*args, ptr, _stream()))
    else:
        check(lib().tvmkv_batch_tree_attn(*args, _stream()))


def tree_attn_paged_kv(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset,
                       q_rope_position, output, lse, rotary_mode, rope_scale, rope_theta, sm_scale,
                       tree_order_indptr, tree_order):
    _f16(q, pages, output)
    _i32(q_indptr, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position, tree_order_indptr,
         tree_order)
    num_pages, _, hkv, ps, d = pages.shape
    check(lib().tvmkv_tree_attn_paged_kv(
        _p(q), _p(q_indptr), _p(pages), _p(page_indptr), _p(page_values), _p(length_info), _p(k_rope_pos_offset),
        _p(q_rope_position), _p(output), _p(lse), int(rotary_mode), float(rope_scale), float(rope_theta),
        float(sm_scale), _p(tree_order_indptr), _p(tree_order), q_indptr.shape[0] - 1, q.shape[0],
        page_values.shape[0], num_pages, q.shape[1], hkv, d, ps, int(length_info.dim() == 2), _stream()))


def batch_prefill_paged_kv_mla(q, q_indptr, pages, page_indptr, page_values, length_info, output, lse, causal,
                               sm_scale):
    _f16(q, pages, output)
    _i32(q_indptr, page_indptr, page_values, length_info)
    num_pages, ps, d_qk = pages.shape
    d_latent = output.shape[2]
    check(lib().tvmkv_batch_prefill_paged_kv_mla(
        _p(q), _p(q_indptr), _p(pages), _p(page_indptr), _p(page_values), _p(length_info), _p(output), _p(lse),
        int(causal), float(sm_scale), q_indptr.shape[0] - 1, q.shape[0], page_values.shape[0], num_pages,
        q.shape[1], d_latent, d_qk - d_latent, ps, _stream()))


def merge_state_inplace(v, s, v_other, s_other):
    _f16(v, v_other)
    n, h, d = v.shape
    check(lib().tvmkv_merge_state_inplace(_p(v), _p(s), _p(v_other), _p(s_other), n, h, d, _stream()))


def copy_single_page(pages, src_page_id, tgt_page_id, copy_length):
    _f16(pages)
    num_pages, _, hkv, ps, d = pages.shape
    check(lib().tvmkv_copy_single_page(_p(pages), src_page_id, tgt_page_id, copy_length, num_pages, hkv, ps, d,
                                       _stream()))


def copy_single_page_mla(pages, src_page_id, tgt_page_id, copy_length):
    _f16(pages)
    num_pages, ps, d = pages.shape
    check(lib().tvmkv_copy_single_page_mla(_p(pages), src_page_id, tgt_page_id, copy_length, num_pages, ps, d,
                                           _stream()))


def tir_kv_cache_debug_get_kv(pages, position_map, k_data, v_data, layer_id):
    _f16(pages, k_data, v_data)
    _i32(position_map)
    num_pages, _, hkv, ps, d = pages.shape
    check(lib().tvmkv_kv_cache_debug_get_kv(_p(pages), _p(position_map), _p(k_data), _p(v_data), layer_id,
                                            position_map.shape[0], num_pages, hkv, ps, d, _stream()))


def tir_kv_cache_debug_get_kv_mla(pages, position_map, kv_data, layer_id):
    _f16(pages, kv_data)
    _i32(position_map)
    num_pages, ps, d = pages.shape
    check(lib().tvmkv_kv_cache_debug_get_kv_mla(_p(pages), _p(position_map), _p(kv_data), layer_id,
                                                position_map.shape[0], num_pages, ps, d, _stream()))


def compact_kv_copy(pages, copy_length_indptr, copy_src_dst_pos, batch_size):
    _f16(pages)
    _i32(copy_length_indptr, copy_src_dst_pos)
    num_pages, _, hkv, ps, d = pages.shape
    check(lib().tvmkv_compact_kv_copy(_p(pages), _p(copy_length_indptr), _p(copy_src_dst_pos), batch_size,
                                      copy_src_dst_pos.shape[1], num_pages, hkv, ps, d, _stream()))
