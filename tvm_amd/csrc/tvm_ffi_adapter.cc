// Registration of libtvmkv's kernels as tvm-ffi global functions, one per kernel slot of
// `vm.builtin.paged_attention_kv_cache_create` (src/runtime/vm/paged_kv_cache.cc:2562-2585): a model
// builder passes them, tagged ["tirx", f], where it passes the TIR kernels today
// (python/tvm/relax/frontend/nn/llm/kv_cache.py:559-736), and the reference's C++ cache runs on this
// library's kernels unchanged.
//
// This translation unit is empty unless tvm-ffi's headers are on the include path (build inside a
// TVM tree, or with -I<tvm-ffi>/include).  Each function unpacks its tensors and hands them, in the
// slot's own order, to the DLPack-level entry point of include/tvmkv_dlpack.h, which validates them and
// applies byte_offset; the stream is the one the TVM device API reports as current for the tensor's
// device (src/runtime/device_api.cc:172).
#if defined(__has_include)
#if __has_include(<tvm/ffi/function.h>) && __has_include(<tvm/ffi/container/tensor.h>)
#define TVMKV_HAVE_TVM_FFI 1
#endif
#endif

#ifdef TVMKV_HAVE_TVM_FFI
#include <tvm/ffi/container/tensor.h>
#include <tvm/ffi/extra/c_env_api.h>
#include <tvm/ffi/function.h>
#include <tvm/ffi/reflection/registry.h>

#include "../../include/tvmkv_dlpack.h"

namespace {

using tvm::ffi::Function;
using tvm::ffi::Tensor;

inline const DLTensor* T(const Tensor& t) { return t.operator->(); }
inline void* StreamOf(const Tensor& t) { return TVMFFIEnvGetStream(t->device.device_type, t->device.device_id); }
inline void Check(int rc) { TVM_FFI_ICHECK_EQ(rc, 0) << "tvmkv: " << tvmkv_last_error(); }

tvmkv_rope_scaling Scaling(int64_t rope_type, double factor, double low_freq_factor, double high_freq_factor, double beta_fast,
                           double beta_slow, int64_t max_position_embeddings, int64_t original_max_position_embeddings,
                           int64_t rotary_dim) {
  tvmkv_rope_scaling scaling{};
  scaling.rope_type = static_cast<int32_t>(rope_type);
  scaling.rotary_dim = static_cast<int32_t>(rotary_dim);  // 0 = the whole head
  scaling.factor = factor;
  scaling.low_freq_factor = low_freq_factor;
  scaling.high_freq_factor = high_freq_factor;
  scaling.beta_fast = beta_fast;
  scaling.beta_slow = beta_slow;
  scaling.max_position_embeddings = max_position_embeddings;
  scaling.original_max_position_embeddings = original_max_position_embeddings;
  return scaling;
}

// Slot 24 for a model: RoPE scale / theta and the frequency variant are compile-time constants of the
// reference's kernel (position_embedding.py:444-667), so the kernel function is made per model.
Function MakeFusedRope(double rope_scale, double rope_theta, int64_t rope_type, double factor, double low_freq_factor,
                       double high_freq_factor, double beta_fast, double beta_slow, int64_t max_position_embeddings,
                       int64_t original_max_position_embeddings, int64_t rotary_dim) {
  const tvmkv_rope_scaling scaling = Scaling(rope_type, factor, low_freq_factor, high_freq_factor, beta_fast, beta_slow,
                                             max_position_embeddings, original_max_position_embeddings, rotary_dim);
  return Function::FromPacked([=](tvm::ffi::PackedArgs args, tvm::ffi::Any* rv) {
    // (qkv, q_rope_position_map, q, k, v, apply_rope) or (..., v, rope_ext_factors): paged_kv_cache.cc:1360-1366
    TVM_FFI_ICHECK_EQ(args.size(), 6) << "tvmkv fused_rope takes 6 arguments";
    Tensor qkv = args[0].cast<Tensor>(), pos = args[1].cast<Tensor>(), q = args[2].cast<Tensor>();
    Tensor k = args[3].cast<Tensor>(), v = args[4].cast<Tensor>();
    if (auto apply_rope = args[5].try_cast<int64_t>()) {
      Check(tvmkv_dl_fused_rope(T(qkv), T(pos), T(q), T(k), T(v), *apply_rope, nullptr, &scaling, rope_scale, rope_theta,
                                StreamOf(qkv)));
    } else {
      Tensor ext_factors = args[5].cast<Tensor>();
      Check(tvmkv_dl_fused_rope(T(qkv), T(pos), T(q), T(k), T(v), 1, T(ext_factors), &scaling, rope_scale, rope_theta,
                                StreamOf(qkv)));
    }
  });
}

void PagedPrefill(int64_t layer_window, Tensor q, Tensor qo_indptr, Tensor pages, Tensor page_indptr, Tensor page_indices,
                  Tensor length_info, Tensor k_rope_pos_offset, Tensor q_rope_position, Tensor out, Tensor lse,
                  int64_t causal, int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale) {
  Check(tvmkv_dl_batch_prefill_paged_kv(T(q), T(qo_indptr), T(pages), T(page_indptr), T(page_indices), T(length_info),
                                        T(k_rope_pos_offset), T(q_rope_position), T(out), T(lse), causal, rotary_mode,
                                        rope_scale, rope_theta, sm_scale, layer_window, StreamOf(q)));
}

// Slot 18 for a model: the per-layer window (cache_config[5]) is a compile-time constant of the
// reference's sliding-window prefill kernel (_prefill_kernels.py:217-391, sliding_window=True).
Function MakePagedPrefillSlidingWindow(int64_t layer_sliding_window_size) {
  return Function::FromTyped([=](Tensor q, Tensor qo_indptr, Tensor pages, Tensor page_indptr, Tensor page_indices,
                                 Tensor length_info, Tensor k_rope_pos_offset, Tensor q_rope_position, Tensor out,
                                 Tensor lse, int64_t causal, int64_t rotary_mode, double rope_scale, double rope_theta,
                                 double sm_scale) {
    PagedPrefill(layer_sliding_window_size, q, qo_indptr, pages, page_indptr, page_indices, length_info, k_rope_pos_offset,
                 q_rope_position, out, lse, causal, rotary_mode, rope_scale, rope_theta, sm_scale);
  });
}

// Slots 15, 16 / 18, 17 / 19 and 21 for a model whose cache rotates inside the attention kernels (rope_mode
// inline) and whose RoPE has a frequency variant: the reference compiles rope_scaling into those kernels too
// (_decode_kernels.py:138,150; _prefill_kernels.py:291-305; tree_attn.py:272-286).  slot: 15, 16, 17 or 21;
// layer_sliding_window_size as for slot 18 (0 otherwise).
Function MakeAttentionWithRopeScaling(int64_t slot, int64_t layer_sliding_window_size, int64_t rope_type, double factor,
                                      double low_freq_factor, double high_freq_factor, double beta_fast, double beta_slow,
                                      int64_t max_position_embeddings, int64_t original_max_position_embeddings) {
  const tvmkv_rope_scaling scaling = Scaling(rope_type, factor, low_freq_factor, high_freq_factor, beta_fast, beta_slow,
                                             max_position_embeddings, original_max_position_embeddings, 0);
  switch (slot) {
    case 15:
      return Function::FromTyped([=](Tensor q, Tensor qo_indptr, Tensor k, Tensor v, Tensor kv_indptr, Tensor q_rope_position,
                                     Tensor k_rope_pos_offset, Tensor out, Tensor lse, int64_t causal, int64_t rotary_mode,
                                     double rope_scale, double rope_theta, double sm_scale) {
        Check(tvmkv_dl_batch_prefill_ragged_kv_scaled(T(q), T(qo_indptr), T(k), T(v), T(kv_indptr), T(q_rope_position),
                                                      T(k_rope_pos_offset), T(out), T(lse), causal, rotary_mode, rope_scale,
                                                      rope_theta, sm_scale, &scaling, StreamOf(q)));
      });
    case 16:
      return Function::FromTyped([=](Tensor q, Tensor qo_indptr, Tensor pages, Tensor page_indptr, Tensor page_indices,
                                     Tensor length_info, Tensor k_rope_pos_offset, Tensor q_rope_position, Tensor out,
                                     Tensor lse, int64_t causal, int64_t rotary_mode, double rope_scale, double rope_theta,
                                     double sm_scale) {
        Check(tvmkv_dl_batch_prefill_paged_kv_scaled(T(q), T(qo_indptr), T(pages), T(page_indptr), T(page_indices),
                                                     T(length_info), T(k_rope_pos_offset), T(q_rope_position), T(out), T(lse),
                                                     causal, rotary_mode, rope_scale, rope_theta, sm_scale,
                                                     layer_sliding_window_size, &scaling, StreamOf(q)));
      });
    case 17:
      return Function::FromTyped([=](Tensor q, Tensor pages, Tensor page_indptr, Tensor page_indices, Tensor length_info,
                                     Tensor k_rope_pos_offset, Tensor q_rope_position, Tensor out, Tensor lse,
                                     int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale) {
        Check(tvmkv_dl_batch_decode_paged_kv_scaled(T(q), T(pages), T(page_indptr), T(page_indices), T(length_info),
                                                    T(k_rope_pos_offset), T(q_rope_position), T(out), T(lse), rotary_mode,
                                                    rope_scale, rope_theta, sm_scale, &scaling, StreamOf(q)));
      });
    case 21:
      return Function::FromTyped([=](Tensor q, Tensor qo_indptr, Tensor k, Tensor v, Tensor kv_indptr, Tensor q_rope_position,
                                     Tensor tree_attn_mn_indptr, Tensor tree_attn_mask, Tensor out, Tensor lse,
                                     int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale) {
        Check(tvmkv_dl_batch_tree_attn_scaled(T(q), T(qo_indptr), T(k), T(v), T(kv_indptr), T(q_rope_position),
                                              T(tree_attn_mn_indptr), T(tree_attn_mask), T(out), T(lse), rotary_mode,
                                              rope_scale, rope_theta, sm_scale, &scaling, StreamOf(q)));
      });
    default:
      TVM_FFI_THROW(ValueError) << "tvmkv.make_attention_with_rope_scaling: slot must be 15, 16, 17 or 21";
  }
  return Function();
}

}  // namespace

TVM_FFI_STATIC_INIT_BLOCK() {
  namespace refl = tvm::ffi::reflection;
  refl::GlobalDef()
      // slot 13 f_transpose_append_mha
      .def("tvmkv.transpose_append",
           [](Tensor pages, Tensor k_data, Tensor v_data, Tensor position_map) {
             Check(tvmkv_dl_transpose_append(T(pages), T(k_data), T(v_data), T(position_map), StreamOf(pages)));
           })
      // slot 14 f_transpose_append_mla
      .def("tvmkv.transpose_append_mla",
           [](Tensor pages, Tensor kv_data, Tensor position_map) {
             Check(tvmkv_dl_transpose_append_mla(T(pages), T(kv_data), T(position_map), StreamOf(pages)));
           })
      // slot 15 ragged prefill
      .def("tvmkv.batch_prefill_ragged_kv",
           [](Tensor q, Tensor qo_indptr, Tensor k, Tensor v, Tensor kv_indptr, Tensor q_rope_position,
              Tensor k_rope_pos_offset, Tensor out, Tensor lse, int64_t causal, int64_t rotary_mode, double rope_scale,
              double rope_theta, double sm_scale) {
             Check(tvmkv_dl_batch_prefill_ragged_kv(T(q), T(qo_indptr), T(k), T(v), T(kv_indptr), T(q_rope_position),
                                                    T(k_rope_pos_offset), T(out), T(lse), causal, rotary_mode, rope_scale,
                                                    rope_theta, sm_scale, StreamOf(q)));
           })
      // slot 16 paged prefill
      .def("tvmkv.batch_prefill_paged_kv",
           [](Tensor q, Tensor qo_indptr, Tensor pages, Tensor page_indptr, Tensor page_indices, Tensor length_info,
              Tensor k_rope_pos_offset, Tensor q_rope_position, Tensor out, Tensor lse, int64_t causal,
              int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale) {
             PagedPrefill(0, q, qo_indptr, pages, page_indptr, page_indices, length_info, k_rope_pos_offset,
                          q_rope_position, out, lse, causal, rotary_mode, rope_scale, rope_theta, sm_scale);
           })
      // slot 18 paged prefill of layers with their own window: tvmkv.make_...(cache_config[5]) -> kernel
      .def("tvmkv.make_batch_prefill_paged_kv_sliding_window", MakePagedPrefillSlidingWindow)
      // slots 17 and 19 paged decode (the (3, batch) length_info selects the sliding-window form)
      .def("tvmkv.batch_decode_paged_kv",
           [](Tensor q, Tensor pages, Tensor page_indptr, Tensor page_indices, Tensor length_info,
              Tensor k_rope_pos_offset, Tensor q_rope_position, Tensor out, Tensor lse, int64_t rotary_mode,
              double rope_scale, double rope_theta, double sm_scale) {
             Check(tvmkv_dl_batch_decode_paged_kv(T(q), T(pages), T(page_indptr), T(page_indices), T(length_info),
                                                  T(k_rope_pos_offset), T(q_rope_position), T(out), T(lse), rotary_mode,
                                                  rope_scale, rope_theta, sm_scale, StreamOf(q)));
           })
      // slot 20 paged prefill with a token-tree mask
      .def("tvmkv.tree_attn_paged_kv",
           [](Tensor q, Tensor qo_indptr, Tensor pages, Tensor page_indptr, Tensor page_indices, Tensor length_info,
              Tensor k_rope_pos_offset, Tensor q_rope_position, Tensor out, Tensor lse, int64_t rotary_mode,
              double rope_scale, double rope_theta, double sm_scale, Tensor tree_attn_mn_indptr, Tensor tree_attn_mask) {
             Check(tvmkv_dl_tree_attn_paged_kv(T(q), T(qo_indptr), T(pages), T(page_indptr), T(page_indices),
                                               T(length_info), T(k_rope_pos_offset), T(q_rope_position), T(out), T(lse),
                                               rotary_mode, rope_scale, rope_theta, sm_scale, T(tree_attn_mn_indptr),
                                               T(tree_attn_mask), StreamOf(q)));
           })
      // slot 21 ragged prefill with a token-tree mask
      .def("tvmkv.batch_tree_attn",
           [](Tensor q, Tensor qo_indptr, Tensor k, Tensor v, Tensor kv_indptr, Tensor q_rope_position,
              Tensor tree_attn_mn_indptr, Tensor tree_attn_mask, Tensor out, Tensor lse, int64_t rotary_mode,
              double rope_scale, double rope_theta, double sm_scale) {
             Check(tvmkv_dl_batch_tree_attn(T(q), T(qo_indptr), T(k), T(v), T(kv_indptr), T(q_rope_position),
                                            T(tree_attn_mn_indptr), T(tree_attn_mask), T(out), T(lse), rotary_mode,
                                            rope_scale, rope_theta, sm_scale, StreamOf(q)));
           })
      // slot 22 MLA paged prefill / decode
      .def("tvmkv.batch_prefill_paged_kv_mla",
           [](Tensor q, Tensor qo_indptr, Tensor pages, Tensor page_indptr, Tensor page_indices, Tensor length_info,
              Tensor out, Tensor lse, int64_t causal, double sm_scale) {
             Check(tvmkv_dl_batch_prefill_paged_kv_mla(T(q), T(qo_indptr), T(pages), T(page_indptr), T(page_indices),
                                                       T(length_info), T(out), T(lse), causal, sm_scale, StreamOf(q)));
           })
      // slot 23 f_merge_inplace (one function serves MHA and MLA: the head dim comes with the tensor)
      .def("tvmkv.merge_state_inplace",
           [](Tensor v, Tensor s, Tensor v_other, Tensor s_other) {
             Check(tvmkv_dl_merge_state_inplace(T(v), T(s), T(v_other), T(s_other), StreamOf(v)));
           })
      // slot 24 f_split_rotary: tvmkv.make_fused_rope(scale, theta, rope_type, ...) -> kernel
      .def("tvmkv.make_fused_rope", MakeFusedRope)
      // slots 15 / 16 / 17 / 21 of a model with inline RoPE and a frequency variant -> kernel
      .def("tvmkv.make_attention_with_rope_scaling", MakeAttentionWithRopeScaling)
      // slot 25 f_copy_single_page (MHA and MLA layers: the rank of `pages` tells)
      .def("tvmkv.copy_single_page",
           [](Tensor pages, int64_t src_page_id, int64_t tgt_page_id, int64_t copy_length) {
             Check(tvmkv_dl_copy_single_page(T(pages), src_page_id, tgt_page_id, copy_length, StreamOf(pages)));
           })
      // slot 26 f_debug_get_kv: (pages, position_map, k_data, v_data, layer_id), MLA (pages, position_map, kv_data, layer_id)
      .def_packed("tvmkv.debug_get_kv",
                  [](tvm::ffi::PackedArgs args, tvm::ffi::Any* rv) {
                    TVM_FFI_ICHECK(args.size() == 4 || args.size() == 5) << "tvmkv debug_get_kv takes 4 or 5 arguments";
                    Tensor pages = args[0].cast<Tensor>(), position_map = args[1].cast<Tensor>();
                    Tensor k_data = args[2].cast<Tensor>();
                    if (args.size() == 5) {
                      Tensor v_data = args[3].cast<Tensor>();
                      Check(tvmkv_dl_debug_get_kv(T(pages), T(position_map), T(k_data), T(v_data), args[4].cast<int64_t>(),
                                                  StreamOf(pages)));
                    } else {
                      Check(tvmkv_dl_debug_get_kv_mla(T(pages), T(position_map), T(k_data), args[3].cast<int64_t>(),
                                                      StreamOf(pages)));
                    }
                  })
      // slot 27 f_compact_copy
      .def("tvmkv.compact_kv_copy", [](Tensor pages, Tensor copy_length_indptr, Tensor copy_src_dst_pos, int64_t batch_size) {
        Check(tvmkv_dl_compact_kv_copy(T(pages), T(copy_length_indptr), T(copy_src_dst_pos), batch_size, StreamOf(pages)));
      });
}
#endif  // TVMKV_HAVE_TVM_FFI
