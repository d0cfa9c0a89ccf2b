"""ctypes front end of the CPU oracle kernels (``oracle/kv_kernels.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py``; the shipped package never imports it.

Every wrapper takes numpy arrays (K/V/q storage as ``np.float16`` or, for the MHA kernels, ``np.float32``:
the dtype of the first array picks the build of the C file; indices as ``np.int32``) in the
argument order of the reference kernel it restates and writes its outputs in place, like
the destination-passing kernels of the reference.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liborc_kernels.so")
_LIB_PATH_F32 = os.path.join(_HERE, "liborc_kernels_f32.so")   # the same file compiled for float32 storage
_lib = None
_lib_f32 = None


def build(force=False):
    """Compile the C oracle with the committed Makefile (both storage types)."""
    for path in (_LIB_PATH, _LIB_PATH_F32):
        if force and os.path.exists(path):
            os.remove(path)
    subprocess.check_call(["make", "-C", _HERE, "all"], stdout=subprocess.DEVNULL)


def lib(like=None):
    """The oracle library; `like`: an array whose dtype selects the storage type (float32 or, by default, float16)."""
    global _lib, _lib_f32
    if like is not None and like.dtype == np.float32:
        if _lib_f32 is None:
            if not os.path.exists(_LIB_PATH_F32):
                build()
            _lib_f32 = ctypes.CDLL(_LIB_PATH_F32)
        return _lib_f32
    assert like is None or like.dtype == np.float16, like.dtype
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _p(a):
    assert a.flags["C_CONTIGUOUS"], "oracle kernels need contiguous arrays"
    return ctypes.c_void_p(a.ctypes.data)


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a


_c_int, _c_i64, _c_f = ctypes.c_int, ctypes.c_int64, ctypes.c_float


def fused_rope(qkv, position_map, q, k, v, apply_rope, *, theta=1e4, scale=1.0, rotary_dim=None):
    n, fused, d = qkv.shape
    hq, hkv = q.shape[1], k.shape[1]
    assert fused == hq + 2 * hkv
    pm = _i32(position_map)
    lib(qkv).orc_fused_rope(_p(qkv), _p(pm), _p(q), _p(k), _p(v), _c_i64(n), _c_int(hq), _c_int(hkv),
                         _c_int(d), _c_int(rotary_dim or d), _c_i64(int(apply_rope)), _c_f(theta),
                         _c_f(scale))


class RopeScaling(ctypes.Structure):
    """orc_rope_scaling; `from_dict` takes the reference's rope_scaling dictionary (position_embedding.py:258-299)."""
    _fields_ = [("rope_type", ctypes.c_int32), ("rotary_dim", ctypes.c_int32), ("factor", ctypes.c_double),
                ("low_freq_factor", ctypes.c_double), ("high_freq_factor", ctypes.c_double),
                ("beta_fast", ctypes.c_double), ("beta_slow", ctypes.c_double),
                ("max_position_embeddings", ctypes.c_int64), ("original_max_position_embeddings", ctypes.c_int64)]
    TYPES = {"default": 0, "llama3": 1, "longrope": 2, "yarn": 3, "gptj": 4, "llama4": 5}

    @classmethod
    def from_dict(cls, rope_scaling):
        out = cls()
        out.rope_type = cls.TYPES[rope_scaling.get("rope_type", "default")]
        for key in ("rotary_dim", "factor", "low_freq_factor", "high_freq_factor", "beta_fast", "beta_slow",
                    "max_position_embeddings", "original_max_position_embeddings"):
            if key in rope_scaling:
                setattr(out, key, rope_scaling[key])
        return out


def rope_angle(rope_scaling, pos_scaled, d, rotary_dim, theta, ext=None):
    """(angle, magnitude) of element d at scaled position pos_scaled, float32 as the reference computes it."""
    sc = RopeScaling.from_dict(rope_scaling)
    fn = lib().orc_rope_angle
    fn.restype = ctypes.c_float
    mag = ctypes.c_float()
    ext_p = None if ext is None else _p(np.ascontiguousarray(ext, dtype=np.float32))
    angle = fn(ctypes.byref(sc), _c_f(pos_scaled), _c_int(d), _c_int(rotary_dim), _c_f(theta), ext_p, ctypes.byref(mag))
    return float(angle), float(mag.value)


class inline_rope_scaling:
    """`with inline_rope_scaling(rope_scaling):` -- inside the block the attention kernels' own RoPE (rotary_mode 1)
    uses this frequency variant, the way the reference bakes the model's rope_scaling dictionary into the kernels it
    builds (_decode_kernels.py:49,138,150; _prefill_kernels.py:54-60,159,171,677,752,758).  A library setting."""

    def __init__(self, rope_scaling):
        self.sc = None if not rope_scaling else RopeScaling.from_dict(rope_scaling)

    def __enter__(self):
        for each in (lib(), lib(np.empty(0, np.float32))):  # both builds: the storage type of the call decides later
            each.orc_set_inline_rope_scaling(None if self.sc is None else ctypes.byref(self.sc))
        return self

    def __exit__(self, *exc):
        for each in (lib(), lib(np.empty(0, np.float32))):
            each.orc_set_inline_rope_scaling(None)
        return False


def fused_rope_scaled(qkv, position_map, q, k, v, apply_rope, rope_scaling, *, theta=1e4, scale=1.0, ext_factors=None):
    n, fused, d = qkv.shape
    hq, hkv = q.shape[1], k.shape[1]
    assert fused == hq + 2 * hkv
    pm = _i32(position_map)
    sc = RopeScaling.from_dict(rope_scaling)
    ext = None if ext_factors is None else np.ascontiguousarray(ext_factors, dtype=np.float32)
    lib(qkv).orc_fused_rope_scaled(_p(qkv), _p(pm), _p(q), _p(k), _p(v), _c_i64(n), _c_int(hq), _c_int(hkv), _c_int(d),
                                _c_i64(int(apply_rope)), _c_f(theta), _c_f(scale), ctypes.byref(sc),
                                None if ext is None else _p(ext))


def transpose_append(pages, k_data, v_data, position_map):
    _, two, hkv, ps, d = pages.shape
    assert two == 2
    pm = _i32(position_map)
    lib(pages).orc_transpose_append(_p(pages), _p(k_data), _p(v_data), _p(pm), _c_i64(len(pm)),
                               _c_int(hkv), _c_int(ps), _c_int(d))


def transpose_append_mla(pages, kv_data, position_map):
    _, ps, d = pages.shape
    pm = _i32(position_map)
    lib().orc_transpose_append_mla(_p(pages), _p(kv_data), _p(pm), _c_i64(len(pm)), _c_int(ps),
                                   _c_int(d))


def debug_get_kv(pages, position_map, k_data, v_data, layer_id):
    _, _, hkv, ps, d = pages.shape
    pm = _i32(position_map)
    lib(pages).orc_debug_get_kv(_p(pages), _p(pm), _p(k_data), _p(v_data), _c_i64(layer_id),
                           _c_i64(len(pm)), _c_int(hkv), _c_int(ps), _c_int(d))


def debug_get_kv_mla(pages, position_map, kv_data, layer_id):
    _, ps, d = pages.shape
    pm = _i32(position_map)
    lib().orc_debug_get_kv_mla(_p(pages), _p(pm), _p(kv_data), _c_i64(layer_id), _c_i64(len(pm)),
                               _c_int(ps), _c_int(d))


def copy_single_page(pages, src_page_id, tgt_page_id, copy_length):
    _, _, hkv, ps, d = pages.shape
    lib(pages).orc_copy_single_page(_p(pages), _c_i64(src_page_id), _c_i64(tgt_page_id),
                               _c_i64(copy_length), _c_int(hkv), _c_int(ps), _c_int(d))


def copy_single_page_mla(pages, src_page_id, tgt_page_id, copy_length):
    _, ps, d = pages.shape
    lib().orc_copy_single_page_mla(_p(pages), _c_i64(src_page_id), _c_i64(tgt_page_id),
                                   _c_i64(copy_length), _c_int(ps), _c_int(d))


def compact_kv_copy(pages, copy_length_indptr, copy_src_dst_pos, batch_size):
    _, _, hkv, ps, d = pages.shape
    ip = _i32(copy_length_indptr)
    sd = _i32(copy_src_dst_pos)
    lib(pages).orc_compact_kv_copy(_p(pages), _p(ip), _p(sd), _c_int(batch_size), _c_int(sd.shape[1]),
                              _c_int(hkv), _c_int(ps), _c_int(d))


def decode(q, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position,
           output, lse, rotary_mode, rope_scale, rope_theta, sm_scale):
    b, hq, d = q.shape
    _, _, hkv, ps, _ = pages.shape
    li = _i32(length_info)
    args = [_i32(page_indptr), _i32(page_values), li, _i32(k_rope_pos_offset), _i32(q_rope_position)]
    lib(q).orc_decode(_p(q), _p(pages), *[_p(a) for a in args], _p(output), _p(lse), _c_int(b),
                     _c_int(hq), _c_int(hkv), _c_int(d), _c_int(ps), _c_int(int(li.ndim == 2)),
                     _c_int(rotary_mode), _c_f(rope_scale), _c_f(rope_theta), _c_f(sm_scale))


def decode_range(q, pages, page_indptr, page_values, length_info, k_rope_pos_offset,
                 q_rope_position, output, lse, b_begin, b_end, sm_scale):
    b, hq, d = q.shape
    _, _, hkv, ps, _ = pages.shape
    args = [_i32(page_indptr), _i32(page_values), _i32(length_info), _i32(k_rope_pos_offset),
            _i32(q_rope_position)]
    lib(q).orc_decode_range(_p(q), _p(pages), *[_p(a) for a in args], _p(output), _p(lse),
                           _c_int(b_begin), _c_int(b_end), _c_int(b), _c_int(hq), _c_int(hkv),
                           _c_int(d), _c_int(ps), _c_f(sm_scale))


def merge_state_inplace(v, s, v_other, s_other):
    n, h, d = v.shape
    lib(v).orc_merge_state_inplace(_p(v), _p(s), _p(v_other), _p(s_other), _c_i64(n), _c_int(h),
                                  _c_int(d))


def prefill_paged(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset,
                  q_rope_position, output, lse, causal, rotary_mode, rope_scale, rope_theta,
                  sm_scale, sliding_window_size=1024):
    _, hq, d = q.shape
    _, _, hkv, ps, _ = pages.shape
    qi = _i32(q_indptr)
    li = _i32(length_info)
    args = [_i32(page_indptr), _i32(page_values), li, _i32(k_rope_pos_offset), _i32(q_rope_position)]
    lib(q).orc_prefill_paged(_p(q), _p(qi), _p(pages), *[_p(a) for a in args], _p(output), _p(lse),
                            _c_int(len(qi) - 1), _c_int(hq), _c_int(hkv), _c_int(d), _c_int(ps),
                            _c_int(int(li.ndim == 2)), _c_int(sliding_window_size),
                            _c_int(int(causal)), _c_int(rotary_mode), _c_f(rope_scale),
                            _c_f(rope_theta), _c_f(sm_scale))


def prefill_ragged(q, q_indptr, k, v, kv_indptr, q_rope_position, k_rope_pos_offset, output, lse,
                   causal, rotary_mode, rope_scale, rope_theta, sm_scale):
    _, hq, dqk = q.shape
    _, hkv, dv = v.shape
    qi, ki = _i32(q_indptr), _i32(kv_indptr)
    qp, ko = _i32(q_rope_position), _i32(k_rope_pos_offset)
    lib(q).orc_prefill_ragged(_p(q), _p(qi), _p(k), _p(v), _p(ki), _p(qp), _p(ko), _p(output),
                             _p(lse), _c_int(len(qi) - 1), _c_int(hq), _c_int(hkv), _c_int(dqk),
                             _c_int(dv), _c_int(int(causal)), _c_int(rotary_mode),
                             _c_f(rope_scale), _c_f(rope_theta), _c_f(sm_scale))


def tree_attn_ragged(q, q_indptr, k, v, kv_indptr, q_rope_position, mn_indptr, mask, output, lse,
                     rotary_mode, rope_scale, rope_theta, sm_scale):
    """tree_attn_cpu; mask is (tree nodes, 2) int32 = (DFS order, end of the subtree's range)."""
    _, hq, d = q.shape
    _, hkv, _ = v.shape
    qi, ki, qp = _i32(q_indptr), _i32(kv_indptr), _i32(q_rope_position)
    mi, mk = _i32(mn_indptr), _i32(mask)
    lib(q).orc_tree_attn_ragged(_p(q), _p(qi), _p(k), _p(v), _p(ki), _p(qp), _p(mi), _p(mk), _p(output),
                               _p(lse), _c_int(len(qi) - 1), _c_int(hq), _c_int(hkv), _c_int(d),
                               _c_int(rotary_mode), _c_f(rope_scale), _c_f(rope_theta), _c_f(sm_scale))


def tree_attn_paged(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset,
                    q_rope_position, output, lse, rotary_mode, rope_scale, rope_theta, sm_scale,
                    tree_order_indptr, tree_order):
    """tree_attn_paged_kv_cpu, argument order of the reference kernel."""
    _, hq, d = q.shape
    _, _, hkv, ps, _ = pages.shape
    qi = _i32(q_indptr)
    li = _i32(length_info)
    args = [_i32(page_indptr), _i32(page_values), li, _i32(k_rope_pos_offset), _i32(q_rope_position)]
    ti, to = _i32(tree_order_indptr), _i32(tree_order)
    lib(q).orc_tree_attn_paged(_p(q), _p(qi), _p(pages), *[_p(a) for a in args], _p(output), _p(lse),
                              _c_int(len(qi) - 1), _c_int(hq), _c_int(hkv), _c_int(d), _c_int(ps),
                              _c_int(int(li.ndim == 2)), _c_int(rotary_mode), _c_f(rope_scale),
                              _c_f(rope_theta), _c_f(sm_scale), _p(ti), _p(to))


def prefill_paged_mla(q, q_indptr, pages, page_indptr, page_values, length_info, output, lse,
                      causal, sm_scale, d_latent=512):
    _, hq, dqk = q.shape
    _, ps, _ = pages.shape
    qi = _i32(q_indptr)
    li = _i32(length_info)
    pi, pv = _i32(page_indptr), _i32(page_values)  # keep the converted arrays alive
    lib().orc_prefill_paged_mla(_p(q), _p(qi), _p(pages), _p(pi), _p(pv), _p(li), _p(output),
                                _p(lse),
                                _c_int(len(qi) - 1), _c_int(hq), _c_int(d_latent),
                                _c_int(dqk - d_latent), _c_int(ps), _c_int(int(li.ndim == 2)),
                                _c_int(int(causal)), _c_f(sm_scale))
