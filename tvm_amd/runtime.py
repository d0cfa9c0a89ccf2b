"""Host-side mirror of the reference's global functions for the paged KV cache.

``get_global_func(name)`` accepts the names the reference registers
(src/runtime/vm/kv_state.cc:33-116, src/runtime/vm/paged_kv_cache.cc:2532-2640) and returns a
callable with the same positional arguments.  Tensors are anything with ``data_ptr()`` and
``shape`` living in device memory (torch tensors on a ROCm device); ``Shape`` arguments are
sequences of ints.  Errors of the library surface as ``KVError`` the way failed checks of the
reference surface as ``tvm.error.InternalError``.
"""
import ctypes
import enum

import numpy as np

from . import _lib
from ._lib import KVError, check, lib


class AttnKind(enum.IntEnum):
    MHA = 0
    MLA = 1
    MHA_SLIDING = 3


class RopeMode(enum.IntEnum):
    NONE = 0
    NORMAL = 1
    INLINE = 2


def Shape(values):  # pylint: disable=invalid-name
    """Stand-in for tvm_ffi.Shape: a tuple of ints."""
    return tuple(int(v) for v in values)


def _i64_array(values):
    arr = (ctypes.c_int64 * len(values))(*[int(v) for v in values])
    return arr


def _ptr(tensor):
    return ctypes.c_void_p(tensor.data_ptr()) if tensor is not None else ctypes.c_void_p(0)


def _require_contiguous(*tensors):
    for t in tensors:
        if t is not None and not t.is_contiguous():
            raise KVError(-1, "tensors handed to the KV cache must be contiguous")


def _require_storage(cache, *tensors):
    """q / k / v / output tensors have the cache's storage type (the reference checks the same,
    src/runtime/vm/paged_kv_cache.cc:1318-1320): the library sees pointers only."""
    for t in tensors:
        element_size = getattr(t, "element_size", None)
        if t is None or element_size is None:
            continue  # not a torch tensor: the caller vouches for what the pointer holds
        if not t.is_floating_point() or element_size() * 8 != cache.dtype_bits:
            raise KVError(-1, f"the KV cache stores float{cache.dtype_bits}; got a tensor of {t.dtype}")


class PagedAttentionKVCache:
    """Handle of a cache object created by ``vm.builtin.paged_attention_kv_cache_create``."""

    def __init__(self, handle, num_layers, num_kv_heads, qk_head_dim, v_head_dim, dtype_bits=16):
        self._handle = handle
        self.dtype_bits = dtype_bits  # storage type of the K/V pages and of every q / k / v / output tensor
        self.num_layers = num_layers
        self.num_kv_heads = num_kv_heads
        self.qk_head_dim = qk_head_dim
        self.v_head_dim = v_head_dim

    def __del__(self):
        handle, self._handle = getattr(self, "_handle", None), None
        if handle:
            try:
                lib().tvmkv_cache_destroy(handle)
            except Exception:  # pylint: disable=broad-except
                pass

    @property
    def handle(self):
        if not self._handle:
            raise KVError(-1, "the KV cache has been destroyed")
        return self._handle

    # ---- introspection used by the parity tests -------------------------------------------
    def aux(self, name, depth=0):
        data = ctypes.POINTER(ctypes.c_int32)()
        size = ctypes.c_int64()
        check(lib().tvmkv_cache_get_aux(self.handle, name.encode(), depth, ctypes.byref(data), ctypes.byref(size)))
        return [data[i] for i in range(size.value)]

    def flags(self):
        buf = (ctypes.c_int64 * 9)()
        check(lib().tvmkv_cache_get_flags(self.handle, buf, 9))
        keys = ["num_depths", "append_before_attn", "is_decode_request", "use_decode_kernel_0",
                "use_decode_kernel_1", "is_chain_0", "is_chain_1", "num_total_pages", "rope_mode"]
        return dict(zip(keys, (int(v) for v in buf)))

    def state(self):
        """Pool snapshot in the format of oracle.host_cache.HostCache.state()."""
        needed = ctypes.c_int64()
        cap = 1 << 16
        while True:
            buf = (ctypes.c_int64 * cap)()
            rc = lib().tvmkv_cache_dump_state(self.handle, buf, cap, ctypes.byref(needed))
            if rc == 0:
                break
            if needed.value <= cap:
                check(rc)
            cap = needed.value
        vals = [int(buf[i]) for i in range(needed.value)]
        pos = 0

        def take(n):
            nonlocal pos
            out = vals[pos:pos + n]
            pos += n
            return out

        free_pages = take(take(1)[0])
        free_blocks = take(take(1)[0])
        blocks = []
        for _ in range(take(1)[0]):
            pages = take(take(1)[0])
            blocks.append((pages, *take(6)))
        seqs = {}
        for _ in range(take(1)[0]):
            sid, last_block, length, window, sink = take(5)
            seqs[sid] = (last_block, length, window, sink)
        return {"free_page_ids": free_pages, "free_block_idx": free_blocks, "blocks": blocks, "seqs": seqs}

    def copy_log(self):
        data = ctypes.POINTER(ctypes.c_int64)()
        n = ctypes.c_int64()
        check(lib().tvmkv_cache_get_copy_log(self.handle, ctypes.byref(data), ctypes.byref(n)))
        return [(int(data[3 * i]), int(data[3 * i + 1]), int(data[3 * i + 2])) for i in range(n.value)]

    def pages_ptr(self, local_layer):
        ptr = ctypes.c_void_p()
        nbytes = ctypes.c_int64()
        check(lib().tvmkv_cache_get_pages(self.handle, local_layer, ctypes.byref(ptr), ctypes.byref(nbytes)))
        return ptr.value, nbytes.value

    def set_stream(self, stream_handle):
        check(lib().tvmkv_cache_set_stream(self.handle, ctypes.c_void_p(stream_handle)))


def _device_index(init):
    """Device of the `init` tensor argument of the create call (None / 'host' = host-only)."""
    if init is None or init == "host":
        return -1
    device = getattr(init, "device", init)
    if getattr(device, "type", None) == "cpu":
        return -1
    index = getattr(device, "index", None)
    if index is None:
        import torch
        index = torch.cuda.current_device()
    return int(index)


def _dtype_bits(init):
    dtype = getattr(init, "dtype", None)
    if dtype is None:
        return 16
    name = str(dtype)
    if "bfloat16" in name:
        return -16  # rejected by the library with a clear message
    if "float16" in name or "half" in name:
        return 16
    if "float32" in name:
        return 32
    return 0


def _create(cache_config, layer_indptr, num_qo_heads, num_kv_heads, qk_head_dim, v_head_dim, attn_kinds,
            enable_kv_transfer, rope_mode, rope_scale, rope_theta, rope_ext_factors, init, *kernel_slots,
            rope_scaling=None):
    """(cache_config, layer_indptr, Hq, Hkv, qk_dim, v_dim, attn_kinds, enable_kv_transfer, rope_mode,
    rope_scale, rope_theta, rope_ext_factors, init_tensor, <15 kernel slots>).  The kernel slots of the
    reference's signature are accepted and ignored: the kernels are the library's own.  What the reference
    bakes into its split-rotary kernel slot travels as the keyword rope_scaling: the model's dictionary
    (rope_type llama3 / longrope / yarn and its parameters, position_embedding.py:258-299 of the reference);
    rope_ext_factors is the float32 device tensor of a longrope model."""
    if rope_ext_factors is not None and (rope_scaling or {}).get("rope_type") != "longrope":
        raise KVError(-1, "rope_ext_factors needs rope_scaling = {'rope_type': 'longrope', ...}")
    cfg = _i64_array(cache_config)
    lip = _i64_array(layer_indptr)
    kinds = _i64_array(attn_kinds)
    out = ctypes.c_void_p()
    check(lib().tvmkv_cache_create(cfg, len(cache_config), lip, len(layer_indptr), num_qo_heads, num_kv_heads,
                                   qk_head_dim, v_head_dim, kinds, len(attn_kinds), int(bool(enable_kv_transfer)),
                                   int(rope_mode), float(rope_scale), float(rope_theta), _dtype_bits(init),
                                   _device_index(init), ctypes.byref(out)))
    cache = PagedAttentionKVCache(out.value, layer_indptr[-1] - layer_indptr[0], num_kv_heads, qk_head_dim,
                                  v_head_dim, _dtype_bits(init))
    if rope_scaling:
        from .dlpack import RopeScaling
        scaling = RopeScaling.from_dict(rope_scaling)
        ext = ctypes.c_void_p(rope_ext_factors.data_ptr()) if rope_ext_factors is not None else None
        check(lib().tvmkv_cache_set_rope_scaling(cache.handle, ctypes.c_void_p(ctypes.addressof(scaling)), ext))
        cache._rope_ext_factors = rope_ext_factors  # the library keeps the pointer, not the tensor
    return cache


def _begin_forward(cache, seq_ids, append_lengths, token_tree_parent_ptr=None):
    ids, lens = _i64_array(seq_ids), _i64_array(append_lengths)
    if len(seq_ids) != len(append_lengths):
        raise KVError(-1, f"The seq_ids size ({len(seq_ids)}) and append_lengths size ({len(append_lengths)}) mismatch.")
    if token_tree_parent_ptr is None:
        check(lib().tvmkv_kv_state_begin_forward(cache.handle, ids, lens, len(seq_ids), None, 0))
    else:
        tree = _i64_array(token_tree_parent_ptr)
        check(lib().tvmkv_kv_state_begin_forward(cache.handle, ids, lens, len(seq_ids), tree, len(tree)))


def _int_query(fn_name):
    def query(cache):
        out = ctypes.c_int32()
        check(getattr(lib(), fn_name)(cache.handle, ctypes.byref(out)))
        return out.value
    return query


def _attention_with_fused_qkv(cache, layer_id, sm_scale, qkv, out):
    _require_contiguous(qkv, out)
    _require_storage(cache, qkv, out)
    check(lib().tvmkv_attention_kv_cache_attention_with_fused_qkv(
        cache.handle, layer_id, float(sm_scale), _ptr(qkv), qkv.shape[0], _ptr(out), out.shape[0]))


def _self_attention(cache, layer_id, sm_scale, q, k, v, o, lse):
    _require_contiguous(q, k, v, o, lse)
    _require_storage(cache, q, k, v, o)
    if not (q.shape[0] == k.shape[0] == v.shape[0] == o.shape[0]):
        raise KVError(-1, "self_attention: q, k, v, o must have the same number of rows")
    check(lib().tvmkv_attention_kv_cache_self_attention(
        cache.handle, layer_id, float(sm_scale), _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(lse), q.shape[0],
        k.shape[1], q.shape[2], v.shape[2]))


def _cross_attention(cache, layer_id, sm_scale, q, o, lse):
    _require_contiguous(q, o, lse)
    _require_storage(cache, q, o)
    if q.shape[0] != o.shape[0]:
        raise KVError(-1, "cross_attention: q and o must have the same number of rows")
    check(lib().tvmkv_attention_kv_cache_cross_attention(
        cache.handle, layer_id, float(sm_scale), _ptr(q), _ptr(o), _ptr(lse), q.shape[0]))


def _attention_with_shared_kv(cache, source_layer_id, sm_scale, q, current_k, current_v, o):
    _require_contiguous(q, current_k, current_v, o)
    _require_storage(cache, q, current_k, current_v, o)
    if not (q.shape[0] == current_k.shape[0] == current_v.shape[0] == o.shape[0]):
        raise KVError(-1, "attention_with_shared_kv: q, current_k, current_v, o must have the same number of rows")
    if current_k.shape[1] != cache.num_kv_heads or current_k.shape[2] != cache.qk_head_dim or \
            current_v.shape[2] != cache.v_head_dim:
        raise KVError(-1, "attention_with_shared_kv: current_k / current_v do not have the cache's head shape")
    check(lib().tvmkv_attention_kv_cache_attention_with_shared_kv(
        cache.handle, source_layer_id, float(sm_scale), _ptr(q), _ptr(current_k), _ptr(current_v), _ptr(o),
        q.shape[0]))


def _append_mla_kv(cache, layer_id, kv):
    _require_contiguous(kv)
    _require_storage(cache, kv)
    check(lib().tvmkv_attention_kv_cache_append_mla_kv(cache.handle, layer_id, _ptr(kv), kv.shape[0]))
    return cache


def _merge_attn_output_inplace(cache, o_self, lse_self, o_cross, lse_cross):
    _require_contiguous(o_self, lse_self, o_cross, lse_cross)
    _require_storage(cache, o_self, o_cross)
    check(lib().tvmkv_attention_kv_cache_merge_attn_output_inplace(
        cache.handle, _ptr(o_self), _ptr(lse_self), _ptr(o_cross), _ptr(lse_cross), o_self.shape[0],
        o_self.shape[1], o_self.shape[2]))
    return [o_self, lse_self]


def _debug_get_kv(cache, seq_id, start_pos, end_pos, k_data, v_data):
    _require_contiguous(k_data, v_data)
    _require_storage(cache, k_data, v_data)
    expect = (cache.num_layers, end_pos - start_pos, cache.num_kv_heads, cache.qk_head_dim)
    for t in (k_data, v_data):
        if tuple(t.shape) != expect:
            raise KVError(-1, "DebugGetKV expects the k_data in layout (num_layers, seq_length, num_kv_heads, "
                              f"qk_head_dim) = {expect}, got {tuple(t.shape)}")
    check(lib().tvmkv_attention_kv_cache_debug_get_kv(cache.handle, seq_id, start_pos, end_pos, _ptr(k_data),
                                                      _ptr(v_data)))


def _debug_get_kv_mla(cache, seq_id, start_pos, end_pos, kv_data):
    _require_contiguous(kv_data)
    _require_storage(cache, kv_data)
    expect = (cache.num_layers, end_pos - start_pos, cache.qk_head_dim)
    if tuple(kv_data.shape) != expect:
        raise KVError(-1, f"DebugGetKV expects the kv_data in layout (num_layers, seq_length, qk_head_dim) = {expect}")
    check(lib().tvmkv_attention_kv_cache_debug_get_kv_mla(cache.handle, seq_id, start_pos, end_pos, _ptr(kv_data)))


def _get_query_positions(cache):
    """Returns (device pointer, length) of the int32 q_rope_position_map."""
    ptr = ctypes.c_void_p()
    n = ctypes.c_int64()
    check(lib().tvmkv_attention_kv_cache_get_query_positions(cache.handle, ctypes.byref(ptr), ctypes.byref(n)))
    return ptr.value, n.value


def _commit(cache, seq_ids, leaf_indices):
    if len(seq_ids) != len(leaf_indices):
        raise KVError(-1, "The given seq_ids and leaf_indices have different size.")
    check(lib().tvmkv_attention_kv_cache_commit_accepted_token_tree_nodes(
        cache.handle, _i64_array(seq_ids), _i64_array(leaf_indices), len(seq_ids)))


_GLOBAL_FUNCS = {
    "vm.builtin.paged_attention_kv_cache_create": _create,
    "vm.builtin.kv_state_clear": lambda c: check(lib().tvmkv_kv_state_clear(c.handle)),
    "vm.builtin.kv_state_add_sequence": lambda c, s: check(lib().tvmkv_kv_state_add_sequence(c.handle, s)),
    "vm.builtin.kv_state_remove_sequence": lambda c, s: check(lib().tvmkv_kv_state_remove_sequence(c.handle, s)),
    "vm.builtin.kv_state_fork_sequence":
        lambda c, parent, child, pos=-1: check(lib().tvmkv_kv_state_fork_sequence(c.handle, parent, child, pos)),
    "vm.builtin.kv_state_popn": lambda c, s, n: check(lib().tvmkv_kv_state_popn(c.handle, s, n)),
    "vm.builtin.kv_state_begin_forward": _begin_forward,
    "vm.builtin.kv_state_end_forward": lambda c: check(lib().tvmkv_kv_state_end_forward(c.handle)),
    "vm.builtin.attention_kv_cache_enable_sliding_window_for_seq":
        lambda c, s, w, sink: check(lib().tvmkv_attention_kv_cache_enable_sliding_window_for_seq(c.handle, s, w, sink)),
    "vm.builtin.attention_kv_cache_commit_accepted_token_tree_nodes": _commit,
    "vm.builtin.attention_kv_cache_empty": lambda c: bool(_int_query("tvmkv_attention_kv_cache_empty")(c)),
    "vm.builtin.attention_kv_cache_get_num_available_pages":
        _int_query("tvmkv_attention_kv_cache_get_num_available_pages"),
    "vm.builtin.attention_kv_cache_get_total_sequence_length":
        _int_query("tvmkv_attention_kv_cache_get_total_sequence_length"),
    "vm.builtin.attention_kv_cache_get_query_positions": _get_query_positions,
    "vm.builtin.attention_kv_cache_attention_with_fused_qkv": _attention_with_fused_qkv,
    "vm.builtin.attention_kv_cache_self_attention": _self_attention,
    "vm.builtin.attention_kv_cache_cross_attention": _cross_attention,
    "vm.builtin.attention_kv_cache_attention_with_shared_kv": _attention_with_shared_kv,
    "vm.builtin.attention_kv_cache_append_mla_kv": _append_mla_kv,
    "vm.builtin.attention_kv_cache_merge_attn_output_inplace": _merge_attn_output_inplace,
    "vm.builtin.attention_kv_cache_debug_get_kv": _debug_get_kv,
    "vm.builtin.attention_kv_cache_debug_get_kv_mla": _debug_get_kv_mla,
}


def get_global_func(name):
    """Counterpart of tvm.get_global_func for the functions on the paged-KV-cache path."""
    try:
        return _GLOBAL_FUNCS[name]
    except KeyError:
        raise KVError(-2, f"global function {name!r} is not part of the paged KV-cache path") from None


def np_i32(values):
    return np.ascontiguousarray(values, dtype=np.int32)
