"""Loader of libtvmkv.so.  There is no fallback: if the library is missing or does not export
a symbol declared in include/tvmkv.h, importing this module raises."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TVMKV_LIB_PATH points the loader at another build of the same library (kernel experiments)
LIB_PATH = os.environ.get("TVMKV_LIB_PATH") or os.path.join(_HERE, "lib", "libtvmkv.so")

c_i32, c_i64, c_f64, c_vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_double, ctypes.c_void_p
p_i32, p_i64 = ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_int64)


class KVError(RuntimeError):
    """A failed call into libtvmkv; carries the library's error code and message (the text of
    the reference's failed check where one exists)."""

    def __init__(self, code, message):
        super().__init__(message)
        self.code = code


# name -> argument ctypes, in the order of include/tvmkv.h
SIGNATURES = {
    "tvmkv_fused_rope": [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i32, c_i32, c_i32, c_f64, c_f64, c_vp],
    "tvmkv_fused_rope_scaled": [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_i32, c_i32, c_i32, c_f64,
                                c_f64, c_vp],
    "tvmkv_fused_rope_append_scaled": [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_i64, c_i32, c_i32,
                                       c_i32, c_i64, c_i32, c_f64, c_f64, c_vp],
    "tvmkv_fused_rope_append": [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp, c_vp, c_i64, c_i32, c_i32, c_i32, c_i64,
                                c_i32, c_f64, c_f64, c_vp],
    "tvmkv_kv_cache_transpose_append": [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_kv_cache_transpose_append_mla": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i32, c_i32, c_vp],
    "tvmkv_batch_prefill_ragged_kv": [c_vp] * 9 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i32, c_i32,
                                                   c_i32, c_i32, c_vp],
    "tvmkv_batch_prefill_paged_kv": [c_vp] * 10 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i64, c_i64,
                                                   c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_batch_prefill_paged_kv_merge": [c_vp] * 10 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i64,
                                                         c_i64, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_batch_prefill_cached_and_new_kv": [c_vp] * 10 + [c_f64, c_i32, c_i64, c_i64, c_i64, c_i32, c_i32, c_i32,
                                                            c_i32, c_vp],
    "tvmkv_batch_prefill_cached_and_new_kv_fused_q": [c_vp, c_vp, c_i64, c_f64, c_f64] + [c_vp] * 9 + [
        c_f64, c_i32, c_i64, c_i64, c_i64, c_i32, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_batch_decode_paged_kv": [c_vp] * 9 + [c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i64, c_i32, c_i32,
                                                 c_i32, c_i32, c_i32, c_vp],
    "tvmkv_batch_decode_paged_kv_noalloc": [c_vp] * 9 + [c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i64, c_i32,
                                                         c_i32, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_batch_decode_paged_kv_scaled": [c_vp] * 9 + [c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i64, c_i32, c_i32,
                                                        c_i32, c_i32, c_i32, c_vp, c_vp],
    "tvmkv_batch_prefill_ragged_kv_scaled": [c_vp] * 9 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i32,
                                                          c_i32, c_i32, c_i32, c_vp, c_vp],
    "tvmkv_batch_prefill_paged_kv_scaled": [c_vp] * 10 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i64,
                                                          c_i64, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32, c_i32,
                                                          c_vp, c_vp],
    "tvmkv_batch_tree_attn_scaled": [c_vp] * 10 + [c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i32, c_i32, c_i32,
                                                   c_vp, c_vp],
    "tvmkv_fused_decode_step": [c_vp] * 9 + [c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i64, c_i32, c_i32, c_i32, c_i32,
                                             c_vp],
    "tvmkv_batch_tree_attn": [c_vp] * 10 + [c_i64, c_f64, c_f64, c_f64, c_i32, c_i64, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_tree_attn_paged_kv": [c_vp] * 10 + [c_i64, c_f64, c_f64, c_f64, c_vp, c_vp, c_i32, c_i64, c_i64, c_i64,
                                               c_i32, c_i32, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_batch_prefill_paged_kv_mla": [c_vp] * 8 + [c_i64, c_f64, c_i32, c_i64, c_i64, c_i64, c_i32, c_i32,
                                                      c_i32, c_i32, c_vp],
    "tvmkv_merge_state_inplace": [c_vp, c_vp, c_vp, c_vp, c_i64, c_i32, c_i32, c_vp],
    "tvmkv_copy_single_page": [c_vp, c_i64, c_i64, c_i64, c_i64, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_copy_single_page_mla": [c_vp, c_i64, c_i64, c_i64, c_i64, c_i32, c_i32, c_vp],
    "tvmkv_kv_cache_debug_get_kv": [c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_kv_cache_debug_get_kv_mla": [c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i32, c_i32, c_vp],
    "tvmkv_compact_kv_copy": [c_vp, c_vp, c_vp, c_i32, c_i32, c_i64, c_i32, c_i32, c_i32, c_vp],
    "tvmkv_set_option": [ctypes.c_char_p, c_i64],
    "tvmkv_get_option": [ctypes.c_char_p, p_i64],
    "tvmkv_release_scratch": [c_vp],
    "tvmkv_debug_set_scratch_launches": [ctypes.c_uint64],
    "tvmkv_decode_split_plan": [p_i32, c_i32, c_i64, c_i32, p_i32, p_i64, p_i32, p_i32, c_i64],
    "tvmkv_cache_create": [p_i64, c_i32, p_i64, c_i32, c_i64, c_i64, c_i64, c_i64, p_i64, c_i32, c_i32, c_i32,
                           c_f64, c_f64, c_i32, c_i32, ctypes.POINTER(c_vp)],
    "tvmkv_cache_set_stream": [c_vp, c_vp],
    "tvmkv_cache_set_rope_scaling": [c_vp, c_vp, c_vp],
    "tvmkv_kv_state_clear": [c_vp],
    "tvmkv_kv_state_add_sequence": [c_vp, c_i64],
    "tvmkv_kv_state_remove_sequence": [c_vp, c_i64],
    "tvmkv_kv_state_fork_sequence": [c_vp, c_i64, c_i64, c_i64],
    "tvmkv_kv_state_popn": [c_vp, c_i64, c_i32],
    "tvmkv_kv_state_begin_forward": [c_vp, p_i64, p_i64, c_i32, p_i64, c_i32],
    "tvmkv_kv_state_end_forward": [c_vp],
    "tvmkv_attention_kv_cache_enable_sliding_window_for_seq": [c_vp, c_i64, c_i32, c_i32],
    "tvmkv_attention_kv_cache_commit_accepted_token_tree_nodes": [c_vp, p_i64, p_i64, c_i32],
    "tvmkv_attention_kv_cache_empty": [c_vp, p_i32],
    "tvmkv_attention_kv_cache_get_num_available_pages": [c_vp, p_i32],
    "tvmkv_attention_kv_cache_get_total_sequence_length": [c_vp, p_i32],
    "tvmkv_attention_kv_cache_get_query_positions": [c_vp, ctypes.POINTER(c_vp), p_i64],
    "tvmkv_attention_kv_cache_attention_with_fused_qkv": [c_vp, c_i64, c_f64, c_vp, c_i64, c_vp, c_i64],
    "tvmkv_attention_kv_cache_self_attention": [c_vp, c_i64, c_f64, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i32,
                                                c_i32, c_i32],
    "tvmkv_attention_kv_cache_cross_attention": [c_vp, c_i64, c_f64, c_vp, c_vp, c_vp, c_i64],
    "tvmkv_attention_kv_cache_attention_with_shared_kv": [c_vp, c_i64, c_f64, c_vp, c_vp, c_vp, c_vp, c_i64],
    "tvmkv_attention_kv_cache_append_mla_kv": [c_vp, c_i64, c_vp, c_i64],
    "tvmkv_attention_kv_cache_merge_attn_output_inplace": [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i32, c_i32],
    "tvmkv_attention_kv_cache_debug_get_kv": [c_vp, c_i64, c_i64, c_i64, c_vp, c_vp],
    "tvmkv_attention_kv_cache_debug_get_kv_mla": [c_vp, c_i64, c_i64, c_i64, c_vp],
    "tvmkv_cache_get_aux": [c_vp, ctypes.c_char_p, c_i32, ctypes.POINTER(p_i32), p_i64],
    "tvmkv_cache_get_flags": [c_vp, p_i64, c_i32],
    "tvmkv_cache_dump_state": [c_vp, p_i64, c_i64, p_i64],
    "tvmkv_cache_get_copy_log": [c_vp, ctypes.POINTER(p_i64), p_i64],
    "tvmkv_cache_get_pages": [c_vp, c_i64, ctypes.POINTER(c_vp), p_i64],
    # include/tvmkv_dlpack.h: DLTensor* arguments in the order of the reference's kernel slots
    "tvmkv_dl_fused_rope": [c_vp] * 5 + [c_i64, c_vp, c_vp, c_f64, c_f64, c_vp],
    "tvmkv_dl_transpose_append": [c_vp] * 5,
    "tvmkv_dl_transpose_append_mla": [c_vp] * 4,
    "tvmkv_dl_batch_prefill_ragged_kv": [c_vp] * 9 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_vp],
    "tvmkv_dl_batch_prefill_paged_kv": [c_vp] * 10 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_i64, c_vp],
    "tvmkv_dl_batch_decode_paged_kv": [c_vp] * 9 + [c_i64, c_f64, c_f64, c_f64, c_vp],
    "tvmkv_dl_tree_attn_paged_kv": [c_vp] * 10 + [c_i64, c_f64, c_f64, c_f64, c_vp, c_vp, c_vp],
    "tvmkv_dl_batch_tree_attn": [c_vp] * 10 + [c_i64, c_f64, c_f64, c_f64, c_vp],
    "tvmkv_dl_batch_prefill_ragged_kv_scaled": [c_vp] * 9 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_vp, c_vp],
    "tvmkv_dl_batch_prefill_paged_kv_scaled": [c_vp] * 10 + [c_i64, c_i64, c_f64, c_f64, c_f64, c_i64, c_vp, c_vp],
    "tvmkv_dl_batch_decode_paged_kv_scaled": [c_vp] * 9 + [c_i64, c_f64, c_f64, c_f64, c_vp, c_vp],
    "tvmkv_dl_batch_tree_attn_scaled": [c_vp] * 10 + [c_i64, c_f64, c_f64, c_f64, c_vp, c_vp],
    "tvmkv_dl_batch_prefill_paged_kv_mla": [c_vp] * 8 + [c_i64, c_f64, c_vp],
    "tvmkv_dl_merge_state_inplace": [c_vp] * 5,
    "tvmkv_dl_copy_single_page": [c_vp, c_i64, c_i64, c_i64, c_vp],
    "tvmkv_dl_debug_get_kv": [c_vp] * 4 + [c_i64, c_vp],
    "tvmkv_dl_debug_get_kv_mla": [c_vp] * 3 + [c_i64, c_vp],
    "tvmkv_dl_compact_kv_copy": [c_vp] * 3 + [c_i64, c_vp],
}

# include/tvmkv_bench.h: the measurement aids of bench.py, a library of their own
BENCH_LIB_PATH = os.path.join(_HERE, "lib", "libtvmkv_bench.so")
BENCH_SIGNATURES = {
    "tvmkvb_stream_read": [c_vp, c_i64, c_vp, c_vp],
    "tvmkvb_stream_read_nt": [c_vp, c_i64, c_vp, c_vp],
    "tvmkvb_stream_copy": [c_vp, c_vp, c_i64, c_vp],
    "tvmkvb_mfma_loop": [c_vp, c_vp, c_i32, c_i32, c_vp],
}

_lib = None
_bench_lib = None


def bench_lib():
    """libtvmkv_bench.so (measurement aids; not part of the drop-in library) with argtypes set."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise ImportError(f"{BENCH_LIB_PATH} is missing: build it with `make -C tvm_amd/csrc`.")
        handle = ctypes.CDLL(BENCH_LIB_PATH)
        for name, argtypes in BENCH_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        _bench_lib = handle
    return _bench_lib


def lib():
    """The loaded library with argtypes set.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C tvm_amd/csrc`. There is no CPU fallback.")
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the symbol is not exported
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        handle.tvmkv_cache_destroy.argtypes = [c_vp]
        handle.tvmkv_cache_destroy.restype = None
        handle.tvmkv_last_error.restype = ctypes.c_char_p
        handle.tvmkv_version.restype = ctypes.c_char_p
        _lib = handle
    return _lib


def check(rc):
    if rc != 0:
        raise KVError(rc, lib().tvmkv_last_error().decode())


def set_option(name, value):
    """Sets a tuning option of the library (see tvmkv_set_option in include/tvmkv.h); returns the old value."""
    old = ctypes.c_int64()
    check(lib().tvmkv_get_option(name.encode(), ctypes.byref(old)))
    check(lib().tvmkv_set_option(name.encode(), int(value)))
    return old.value


def decode_split_plan(page_indptr, nnz_pages, h_kv):
    """(chunk_pages, slot_seq, slot_chunk) of a decode launch with these shapes; host arithmetic only."""
    batch = len(page_indptr) - 1
    indptr = (ctypes.c_int32 * (batch + 1))(*[int(v) for v in page_indptr])
    cp, slots = ctypes.c_int32(), ctypes.c_int64()
    check(lib().tvmkv_decode_split_plan(indptr, batch, int(nnz_pages), int(h_kv), ctypes.byref(cp),
                                        ctypes.byref(slots), None, None, 0))
    seq = (ctypes.c_int32 * max(slots.value, 1))()
    chunk = (ctypes.c_int32 * max(slots.value, 1))()
    check(lib().tvmkv_decode_split_plan(indptr, batch, int(nnz_pages), int(h_kv), ctypes.byref(cp),
                                        ctypes.byref(slots), seq, chunk, slots.value))
    return cp.value, list(seq[:slots.value]), list(chunk[:slots.value])
