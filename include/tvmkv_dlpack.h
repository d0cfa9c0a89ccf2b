/*
 * libtvmkv at the level the reference calls its kernels: DLPack tensors in, in the argument order of
 * the reference's "tirx" kernel slots.
 *
 * `vm.builtin.paged_attention_kv_cache_create` receives its kernels as packed functions
 * (src/runtime/vm/paged_kv_cache.cc:2562-2585, src/runtime/vm/attn_backend.cc:28-132) and calls them
 * with tvm::runtime::Tensor arguments, i.e. DLTensor views: the int32 auxiliary arrays are views at a
 * non-zero `byte_offset` into one merged buffer (src/runtime/vm/attn_utils.h:1027-1035), shapes travel
 * in the tensors and scalars are int64 / double.  Each function below takes exactly the arguments of
 * one slot, in the slot's order, as `const DLTensor*` and C scalars, followed by what the reference
 * kernel has baked in at compile time (RoPE scale and theta for slot 24, the per-layer window for
 * slot 18) and the HIP stream.  A packed-function adapter is then one line per slot: unpack, pass on
 * (tvm_amd/csrc/tvm_ffi_adapter.cc registers all of them when tvm-ffi's headers are present).
 *
 * Every function validates what the pointer-level launchers of tvmkv.h must take on trust: device
 * type and id (all tensors on one ROCm device), dtype, ndim, compact strides, consistent shapes and
 * alignment of `data + byte_offset`; a mismatch returns TVMKV_EINVAL and tvmkv_last_error() names the
 * argument.  Return codes as in tvmkv.h.
 *
 * Storage type.  q / k / v / pages / out of the MHA slots (13, 15-21, 23-27) are float16 or float32, the
 * same in every tensor of a call (the reference builds each kernel for one storage dtype); lse and the
 * RoPE factor tensor are float32, index arrays int32.  float32 storage runs on the generic kernels
 * (tvmkv.h, "Shapes"), rotary_mode 1 (head dims that are a multiple of 8) and the (3, batch)
 * length_info included.  The MLA slots (14, 22) are float16.
 */
#ifndef TVMKV_DLPACK_H_
#define TVMKV_DLPACK_H_

#include <stdint.h>

#include "tvmkv.h"

/* The DLPack ABI (dlpack/dlpack.h, v0.8 / v1.x: the structs below have not changed).  If the real
 * header was included first, its definitions are used. */
#ifndef DLPACK_DLPACK_H_
#define TVMKV_OWN_DLPACK_STRUCTS 1
typedef enum {
  kDLCPU = 1,
  kDLCUDA = 2,
  kDLCUDAHost = 3,
  kDLROCM = 10,
  kDLROCMHost = 11
} DLDeviceType;
typedef struct {
  int32_t device_type; /* DLDeviceType */
  int32_t device_id;
} DLDevice;
typedef enum { kDLInt = 0U, kDLUInt = 1U, kDLFloat = 2U, kDLBfloat = 4U } DLDataTypeCode;
typedef struct {
  uint8_t code;
  uint8_t bits;
  uint16_t lanes;
} DLDataType;
typedef struct {
  void* data;
  DLDevice device;
  int32_t ndim;
  DLDataType dtype;
  int64_t* shape;
  int64_t* strides; /* NULL = compact row-major */
  uint64_t byte_offset;
} DLTensor;
#endif

#ifdef __cplusplus
extern "C" {
#endif

/* Slot 24 `f_split_rotary`, called at paged_kv_cache.cc:1360-1366 as
 * (qkv, q_rope_position_map, q, k, v, apply_rope) or, for models with per-dimension frequency factors
 * (position_embedding.py:164-188), (qkv, q_rope_position_map, q, k, v, apply_rope, rope_ext_factors).
 * rope_ext_factors: NULL, or the float32 tensor of head_dim factors of a longrope model (long factors,
 * then short ones); the reference's kernel of that form has no apply_rope argument and always rotates,
 * so apply_rope is ignored when the tensor is given.
 * scaling / rope_scale / rope_theta: what the reference kernel was compiled with (scaling NULL = none). */
int tvmkv_dl_fused_rope(const DLTensor* qkv, const DLTensor* q_rope_position_map, const DLTensor* q,
                        const DLTensor* k, const DLTensor* v, int64_t apply_rope,
                        const DLTensor* rope_ext_factors, const tvmkv_rope_scaling* scaling,
                        double rope_scale, double rope_theta, void* stream);

/* Slot 13 `f_transpose_append_mha`, paged_kv_cache.cc:1371-1372:
 * (pages, k_data, v_data, append_position_map). */
int tvmkv_dl_transpose_append(const DLTensor* pages, const DLTensor* k_data, const DLTensor* v_data,
                              const DLTensor* append_position_map, void* stream);

/* Slot 14 `f_transpose_append_mla`, paged_kv_cache.cc:1550: (pages, kv_data, append_position_map). */
int tvmkv_dl_transpose_append_mla(const DLTensor* pages, const DLTensor* kv_data,
                                  const DLTensor* append_position_map, void* stream);

/* Slot 15 ragged prefill, attn_backend.h:392-395. */
int tvmkv_dl_batch_prefill_ragged_kv(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* k,
                                     const DLTensor* v, const DLTensor* kv_indptr,
                                     const DLTensor* q_rope_position, const DLTensor* k_rope_pos_offset,
                                     const DLTensor* out, const DLTensor* lse, int64_t causal,
                                     int64_t rotary_mode, double rope_scale, double rope_theta,
                                     double sm_scale, void* stream);

/* Slots 16 / 18 paged prefill, attn_backend.h:239-242.  length_info (batch,) or (3, batch); the
 * second form selects the sliding-window kernel.  layer_sliding_window_size: the window a slot-18
 * kernel was compiled for (cache_config[5]), 0 for slot 16. */
int tvmkv_dl_batch_prefill_paged_kv(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* pages,
                                    const DLTensor* page_indptr, const DLTensor* page_indices,
                                    const DLTensor* length_info, const DLTensor* k_rope_pos_offset,
                                    const DLTensor* q_rope_position, const DLTensor* out,
                                    const DLTensor* lse, int64_t causal, int64_t rotary_mode,
                                    double rope_scale, double rope_theta, double sm_scale,
                                    int64_t layer_sliding_window_size, void* stream);

/* Slots 17 / 19 paged decode, attn_backend.h:511-514. */
int tvmkv_dl_batch_decode_paged_kv(const DLTensor* q, const DLTensor* pages, const DLTensor* page_indptr,
                                   const DLTensor* page_indices, const DLTensor* length_info,
                                   const DLTensor* k_rope_pos_offset, const DLTensor* q_rope_position,
                                   const DLTensor* out, const DLTensor* lse, int64_t rotary_mode,
                                   double rope_scale, double rope_theta, double sm_scale, void* stream);

/* Slot 20 paged prefill with a token-tree mask, attn_backend.h:623-626. */
int tvmkv_dl_tree_attn_paged_kv(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* pages,
                                const DLTensor* page_indptr, const DLTensor* page_indices,
                                const DLTensor* length_info, const DLTensor* k_rope_pos_offset,
                                const DLTensor* q_rope_position, const DLTensor* out, const DLTensor* lse,
                                int64_t rotary_mode, double rope_scale, double rope_theta,
                                double sm_scale, const DLTensor* tree_attn_mn_indptr,
                                const DLTensor* tree_attn_mask, void* stream);

/* Slot 21 ragged prefill with a token-tree mask, attn_backend.h:669-672. */
int tvmkv_dl_batch_tree_attn(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* k,
                             const DLTensor* v, const DLTensor* kv_indptr,
                             const DLTensor* q_rope_position, const DLTensor* tree_attn_mn_indptr,
                             const DLTensor* tree_attn_mask, const DLTensor* out, const DLTensor* lse,
                             int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                             void* stream);

/* The four launchers above that rotate inside the kernel (rotary_mode = 1), for a model whose RoPE has a
 * frequency variant: the reference compiles rope_scaling into these kernels (_decode_kernels.py:138,150,
 * _prefill_kernels.py:291-305, tree_attn.py:272-286), so a kernel function is made per model and passes
 * the model's rope_scaling here (NULL = the default frequencies, the entry points above). */
int tvmkv_dl_batch_prefill_ragged_kv_scaled(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* k,
                                            const DLTensor* v, const DLTensor* kv_indptr,
                                            const DLTensor* q_rope_position, const DLTensor* k_rope_pos_offset,
                                            const DLTensor* out, const DLTensor* lse, int64_t causal,
                                            int64_t rotary_mode, double rope_scale, double rope_theta,
                                            double sm_scale, const tvmkv_rope_scaling* rope_scaling, void* stream);
int tvmkv_dl_batch_prefill_paged_kv_scaled(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* pages,
                                           const DLTensor* page_indptr, const DLTensor* page_indices,
                                           const DLTensor* length_info, const DLTensor* k_rope_pos_offset,
                                           const DLTensor* q_rope_position, const DLTensor* out,
                                           const DLTensor* lse, int64_t causal, int64_t rotary_mode,
                                           double rope_scale, double rope_theta, double sm_scale,
                                           int64_t layer_sliding_window_size,
                                           const tvmkv_rope_scaling* rope_scaling, void* stream);
int tvmkv_dl_batch_decode_paged_kv_scaled(const DLTensor* q, const DLTensor* pages, const DLTensor* page_indptr,
                                          const DLTensor* page_indices, const DLTensor* length_info,
                                          const DLTensor* k_rope_pos_offset, const DLTensor* q_rope_position,
                                          const DLTensor* out, const DLTensor* lse, int64_t rotary_mode,
                                          double rope_scale, double rope_theta, double sm_scale,
                                          const tvmkv_rope_scaling* rope_scaling, void* stream);
int tvmkv_dl_batch_tree_attn_scaled(const DLTensor* q, const DLTensor* qo_indptr, const DLTensor* k,
                                    const DLTensor* v, const DLTensor* kv_indptr,
                                    const DLTensor* q_rope_position, const DLTensor* tree_attn_mn_indptr,
                                    const DLTensor* tree_attn_mask, const DLTensor* out, const DLTensor* lse,
                                    int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                    const tvmkv_rope_scaling* rope_scaling, void* stream);

/* Slot 22 MLA paged prefill (and decode), attn_backend.h:248-249. */
int tvmkv_dl_batch_prefill_paged_kv_mla(const DLTensor* q, const DLTensor* qo_indptr,
                                        const DLTensor* pages, const DLTensor* page_indptr,
                                        const DLTensor* page_indices, const DLTensor* length_info,
                                        const DLTensor* out, const DLTensor* lse, int64_t causal,
                                        double sm_scale, void* stream);

/* Slot 23 `f_merge_inplace`, paged_kv_cache.cc:2292, :2329, :1557: (v, s, v_other, s_other). */
int tvmkv_dl_merge_state_inplace(const DLTensor* v, const DLTensor* s, const DLTensor* v_other,
                                 const DLTensor* s_other, void* stream);

/* Slot 25 `f_copy_single_page`, paged_kv_cache.cc:728: (pages, src_page_id, tgt_page_id, copy_length).
 * Five-dimensional pages are an MHA layer's, three-dimensional ones an MLA layer's. */
int tvmkv_dl_copy_single_page(const DLTensor* pages, int64_t src_page_id, int64_t tgt_page_id,
                              int64_t copy_length, void* stream);

/* Slot 26 `f_debug_get_kv`, paged_kv_cache.cc:1718: (pages, position_map, k_data, v_data, layer_id),
 * and its MLA form, :1764: (pages, position_map, kv_data, layer_id). */
int tvmkv_dl_debug_get_kv(const DLTensor* pages, const DLTensor* position_map, const DLTensor* k_data,
                          const DLTensor* v_data, int64_t layer_id, void* stream);
int tvmkv_dl_debug_get_kv_mla(const DLTensor* pages, const DLTensor* position_map,
                              const DLTensor* kv_data, int64_t layer_id, void* stream);

/* Slot 27 `f_compact_copy`, paged_kv_cache.cc:759-760:
 * (pages, copy_length_indptr, copy_src_dst_pos, batch_size). */
int tvmkv_dl_compact_kv_copy(const DLTensor* pages, const DLTensor* copy_length_indptr,
                             const DLTensor* copy_src_dst_pos, int64_t batch_size, void* stream);

#ifdef __cplusplus
}
#endif

#endif /* TVMKV_DLPACK_H_ */
