// The MHA kernels behind one more argument: the storage type of q / k / v / pages / out.
//
// The reference builds every kernel for a storage dtype, a page size and a head dim
// (python/tvm/relax/frontend/nn/llm/kv_cache.py:559-736; its tests run float16 and float32 storage,
// tests/python/relax/test_runtime_builtin_paged_attention_kv_cache_cpu.py:269-276).  This library's tuned
// kernels are fp16 with pages of 16 / 32 / 64 / 128 tokens and head dims 64 / 80 / 96 / 112 / 128 / 256 (80 / 96 /
// 112 in their plain form only); everything else those factories accept -- float32 storage, any page size, any
// head dim that is a multiple of 4 (fp32) or 8 (fp16) up to 256 -- runs on the generic matrix-core kernels of
// kernels_generic.hip: float32 sums, K and V rows read straight from their pages with one page-table lookup per
// row, the sliding-window cache (length_info (3, batch)), the per-layer window mask and RoPE inside the kernel
// included.  Not built there: MLA.
//
// elem_bits is 16 or 32.  The functions return the library's error codes and leave the message in the
// thread's last-error slot, like the extern "C" launchers they stand beside; they are internal: the
// tensor-level boundary (the dtype travels in the DLTensor) and the cache object (dtype_bits) call them.
#ifndef TVMKV_CSRC_TYPED_KERNELS_H_
#define TVMKV_CSRC_TYPED_KERNELS_H_

#include <cstdint>

#include "../../include/tvmkv.h"

namespace tvmkv {

// What the tuned fp16 attention kernels are built for; anything else goes to the generic kernels.
inline bool tuned_page_size(int page_size) { return page_size == 16 || page_size == 32 || page_size == 64 || page_size == 128; }
inline bool tuned_head_dim(int d) { return d == 64 || d == 80 || d == 96 || d == 112 || d == 128 || d == 256; }

// One launcher for every MHA attention slot.  Sources: paged (pages != NULL: page_indptr, page_values,
// last_page_len (batch,), page_size) or ragged (k, v, kv_indptr).  q_indptr NULL: one query row per
// sequence (decode).  Masks: causal (query i of n sees the first kv_len - n + i + 1 keys,
// _kernel_common.py:130-135), or, with tree labels, the token-tree mask (tree_attn.py:48-65: the last
// tree_indptr[b+1] - tree_indptr[b] keys of sequence b are tree nodes, labels = (first, second) per node);
// neither: every key.
struct GenericAttention {
  int elem_bits = 16;
  const void* q = nullptr;
  const int32_t* q_indptr = nullptr;
  const void* k = nullptr;
  const void* v = nullptr;
  const int32_t* kv_indptr = nullptr;
  const void* pages = nullptr;
  const int32_t* page_indptr = nullptr;
  const int32_t* page_values = nullptr;
  const int32_t* last_page_len = nullptr;
  const int32_t* tree_indptr = nullptr;
  const int32_t* tree_labels = nullptr;
  void* out = nullptr;
  float* lse = nullptr;
  int64_t total_q = 0;
  int64_t nnz_pages = 0;
  int64_t num_pages = 0;
  int32_t batch = 0, h_q = 0, h_kv = 0, d = 0, page_size = 0;
  int32_t causal = 0;
  double sm_scale = 1.0;
  const char* what = "attention";
  // The extended form, as the tuned kernels have it.  sliding_window: last_page_len is the (3, batch) length_info of
  // a sliding-window cache (last page length, window offset, sink size; attn_utils.h:483-495), keys have logical
  // indices, the sink tokens first (_kernel_common.py:155-170); layer_window > 0 with causal on such a cache: the
  // per-layer window mask (:138-144).  rotary_mode 1: q and k are rotated inside the kernel, query token i at
  // q_rope_position[i], logical key t of sequence b at k_rope_pos_offset[b] + t (ragged with k_rope_pos_offset NULL:
  // at q_rope_position[kv_indptr[b] + t], the token-tree form, tree_attn.py:93-259), frequencies of rope_scaling
  // (NULL: the default ones).  Needs a head dim that is a multiple of 16 (fp16) or 8 (float32).
  int32_t sliding_window = 0;
  int32_t layer_window = 0;
  int64_t rotary_mode = 0;
  const int32_t* q_rope_position = nullptr;
  const int32_t* k_rope_pos_offset = nullptr;
  double rope_scale = 1.0, rope_theta = 1e4;
  const tvmkv_rope_scaling* rope_scaling = nullptr;
};
int generic_attention(const GenericAttention& args, void* stream);

// Slot 24 (and 24 + 13 with pages != NULL) for any even head dim up to 256 and either storage type; the
// arguments of tvmkv_fused_rope_append_scaled.
int typed_fused_rope(int elem_bits, const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                     int64_t apply_rope, const float* rope_ext_factors, const tvmkv_rope_scaling* scaling, void* pages,
                     const int32_t* append_position_map, int64_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                     int32_t head_dim, int64_t num_pages, int32_t page_size, double rope_scale, double rope_theta,
                     void* stream);
// Slot 23 for either storage type.
int typed_merge_state_inplace(int elem_bits, void* v, float* s, const void* v_other, const float* s_other, int64_t n,
                              int32_t h, int32_t d, void* stream);

// The copy kernels move rows of head_dim elements whatever they hold: float32 rows are fp16 rows of twice
// the length.
inline int32_t copy_dim(int elem_bits, int32_t head_dim) { return head_dim * (elem_bits / 16); }

}  // namespace tvmkv

#endif  // TVMKV_CSRC_TYPED_KERNELS_H_
