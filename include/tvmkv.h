/*
 * tvmkv -- MI355X (gfx950) paged KV-cache attention behind the interface of apache/tvm's
 * PagedAttentionKVCache.  C ABI: plain pointers and sizes, no C++ or framework types.
 *
 * Two layers, both exported from libtvmkv.so:
 *
 *  (1) KERNEL LAUNCHERS.  One per kernel slot that the reference's
 *      `vm.builtin.paged_attention_kv_cache_create` takes as an ffi::Function
 *      (src/runtime/vm/paged_kv_cache.cc:2562-2585).  Tensor arguments appear in the order
 *      of the reference's "tirx" calling convention (src/runtime/vm/attn_backend.h); what a
 *      DLTensor would carry implicitly (shapes, byte_offset-adjusted data pointers, the
 *      stream) is passed explicitly after them.  All data pointers are DEVICE pointers, fp16
 *      for K/V/Q/O data, int32 for index arrays, fp32 for log-sum-exp.  Index arrays that the
 *      reference passes as views with a non-zero byte_offset (src/runtime/vm/attn_utils.h:
 *      1027-1035) must already have that offset added.  `stream` is a hipStream_t (NULL = the
 *      null stream).  Launchers are asynchronous and never synchronise the device.
 *
 *      Shapes.  The tuned kernels are fp16 with pages of 16 / 32 / 64 / 128 tokens and head dims
 *      64 / 80 / 96 / 112 / 128 / 256 (the comment of each launcher says what it has of them).
 *      A call with another page size or head dim (80 / 96 / 112 as soon as it has rotary_mode 1
 *      or a three-row length_info) is handed to generic matrix-core kernels (float32 sums; any page
 *      size, head dims that are a multiple of 8 up to 256, of 16 with rotary_mode 1): the reference's kernel
 *      factories take both as free parameters (_decode_kernels.py:49,181;
 *      _prefill_kernels.py:54-60,217-225).  The same kernels serve float32 K/V storage, which the
 *      reference's tests also run (tests/python/relax/
 *      test_runtime_builtin_paged_attention_kv_cache_cpu.py:269-276): float32 tensors are taken
 *      by the tensor-level entry points of tvmkv_dlpack.h, where the dtype travels in the
 *      tensor, and by a cache object created with dtype_bits 32; the pointer-level launchers of
 *      this file are fp16.
 *
 *  (2) CACHE OBJECT.  `tvmkv_cache_*` / `tvmkv_kv_state_*` / `tvmkv_attention_kv_cache_*`:
 *      the host-side page pool, block tree and per-step auxiliary arrays, with the verbs and
 *      error behaviour of the reference's global functions `vm.builtin.kv_state_*` and
 *      `vm.builtin.attention_kv_cache_*` (src/runtime/vm/kv_state.cc:33-116), calling (1).
 *
 * Error convention: every function returning int returns 0 on success and a negative
 * TVMKV_E* code on failure; tvmkv_last_error() then returns a thread-local message (the
 * text of the reference's failed check where one exists).  Nothing throws across the ABI.
 *
 * Threading: a cache object is not thread-safe (neither is the reference's).  The split-KV
 * launchers (decode, MLA decode) keep their scratch memory per (device, stream): calls on one
 * stream are ordered and share it, calls on different streams never do, and the table of buffers
 * is guarded by a mutex.  A buffer grows with hipMalloc when a call needs more than any before it
 * on that stream (after synchronising that stream only).
 */
#ifndef TVMKV_H_
#define TVMKV_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TVMKV_OK 0
#define TVMKV_EINVAL (-1)      /* a check of the reference failed (bad argument / state)   */
#define TVMKV_EUNSUPPORTED (-2) /* valid in the reference, not built here (clear message)   */
#define TVMKV_EDEVICE (-3)     /* a HIP runtime call failed                                */
#define TVMKV_ENODEVICE (-4)   /* device work requested from a host-only cache             */

/* Thread-local message of the last failed call on this thread ("" if none). */
const char* tvmkv_last_error(void);
/* Library version string. */
const char* tvmkv_version(void);

/* ======================================================================================
 * (1) Kernel launchers
 * ====================================================================================== */

/* Slot 24 `f_split_rotary` -- replaces `fused_rope`
 * (python/tvm/relax/frontend/nn/llm/position_embedding.py:525-565), called at
 * src/runtime/vm/paged_kv_cache.cc:1360-1366 as (qkv, q_rope_position_map, q, k, v, apply_rope).
 * qkv (seq_len, num_q_heads + 2*num_kv_heads, head_dim) -> q (seq_len, num_q_heads, head_dim),
 * k, v (seq_len, num_kv_heads, head_dim); rotate-half RoPE on q and k in fp32 when apply_rope>0.
 * theta/scale are baked into the reference kernel at build time; here they are arguments. */
int tvmkv_fused_rope(const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                     int64_t apply_rope, int64_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                     int32_t head_dim, double rope_scale, double rope_theta, void* stream);

/* The frequency variants of slot 24 (`switch_rope_freq_func`, position_embedding.py:258-299), which the
 * reference bakes into the kernel it compiles for a model.  rope_type DEFAULT: angle = pos * scale /
 * theta^(2i/D).  LLAMA3 (:130-161): smoothed inverse frequencies from factor, low_freq_factor,
 * high_freq_factor, original_max_position_embeddings.  LONGROPE (:164-188): the default divisors times a
 * per-dimension factor tensor, cos and sin scaled by sqrt(1 + ln(max / original_max) / ln(original_max)).
 * YARN (:191-255): interpolated / extrapolated inverse frequencies blended over the dimensions between
 * the correction dims of beta_fast and beta_slow.  Rotation is over the first rotary_dim features of a head
 * (the whole head by default), with the rotate-half pairing or, for GPTJ, in interleaved pairs. */
enum {
  TVMKV_ROPE_FREQ_DEFAULT = 0,
  TVMKV_ROPE_FREQ_LLAMA3 = 1,
  TVMKV_ROPE_FREQ_LONGROPE = 2,
  TVMKV_ROPE_FREQ_YARN = 3,
  TVMKV_ROPE_FREQ_GPTJ = 4, /* :70-76, :509-514: pairs (2i, 2i+1) instead of (i, i + rotary_dim/2), default frequencies */
  TVMKV_ROPE_FREQ_LLAMA4 = 5 /* :79-127: the llama3 smoothing (or, with equal low and high factors, a hard threshold on
                                the wavelength) on the frequency of pair d / 2, rotate-half pairing; same fields as LLAMA3 */
};
typedef struct tvmkv_rope_scaling {
  int32_t rope_type;
  int32_t rotary_dim;     /* features 0 .. rotary_dim-1 of a head are rotated, in pairs (d, d + rotary_dim/2), with
                             frequencies over rotary_dim; the others pass through (position_embedding.py:507-520).
                             0 = head_dim.  Even, at most head_dim; any frequency variant. */
  double factor;          /* llama3, yarn */
  double low_freq_factor; /* llama3 */
  double high_freq_factor;
  double beta_fast; /* yarn */
  double beta_slow;
  int64_t max_position_embeddings; /* longrope */
  int64_t original_max_position_embeddings;
} tvmkv_rope_scaling;

/* tvmkv_fused_rope with a frequency variant.  scaling NULL = DEFAULT.  rope_ext_factors: device tensor of
 * head_dim float32, LONGROPE only: the long factors (head_dim / 2), then the short ones; as in the
 * reference's kernel (position_embedding.py:582-668) the long ones apply when the call has more rows
 * than original_max_position_embeddings.  The tables are computed on the host in float32 in the
 * reference's order of operations and travel as a kernel argument. */
int tvmkv_fused_rope_scaled(const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                            int64_t apply_rope, const float* rope_ext_factors,
                            const tvmkv_rope_scaling* scaling, int64_t seq_len, int32_t num_q_heads,
                            int32_t num_kv_heads, int32_t head_dim, double rope_scale, double rope_theta,
                            void* stream);

/* tvmkv_fused_rope_append (below) with a frequency variant. */
int tvmkv_fused_rope_append_scaled(const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                                   int64_t apply_rope, const float* rope_ext_factors,
                                   const tvmkv_rope_scaling* scaling, void* pages,
                                   const int32_t* append_position_map, int64_t seq_len, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_dim, int64_t num_pages,
                                   int32_t page_size, double rope_scale, double rope_theta, void* stream);

/* Slot 24 followed by slot 13 in one launch; no counterpart among the reference's kernels.
 * Besides the q / k / v outputs of tvmkv_fused_rope, the rotated k and the v rows are written into
 * their page slots append_position_map[token] (-1 = none), which is what
 * tvmkv_kv_cache_transpose_append would do from k and v afterwards (paged_kv_cache.cc:1360-1373).
 * The cache uses it when it appends before attention; k and v stay available to the ragged kernel. */
int tvmkv_fused_rope_append(const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                            int64_t apply_rope, void* pages, const int32_t* append_position_map,
                            int64_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                            int32_t head_dim, int64_t num_pages, int32_t page_size, double rope_scale,
                            double rope_theta, void* stream);

/* (q may be NULL in tvmkv_fused_rope_append: the q rows are then not written; the caller hands the
 * fused qkv tensor to tvmkv_batch_prefill_cached_and_new_kv_fused_q, which rotates them itself.) */

/* Slot 13 `f_transpose_append_mha` -- replaces `tir_kv_cache_transpose_append`
 * (python/tvm/relax/frontend/nn/llm/_page_kernels.py:40-74), called at paged_kv_cache.cc:1371
 * as (pages, k_data, v_data, position_map).  pages (num_pages, 2, num_kv_heads, page_size,
 * head_dim); row i goes to slot position_map[i] (= page*page_size + offset), -1 = skip. */
int tvmkv_kv_cache_transpose_append(void* pages, const void* k_data, const void* v_data,
                                    const int32_t* position_map, int64_t ntoken, int64_t num_pages,
                                    int32_t num_kv_heads, int32_t page_size, int32_t head_dim,
                                    void* stream);

/* Slot 14 `f_transpose_append_mla` -- replaces `tir_kv_cache_transpose_append_mla`
 * (_page_kernels.py:77-103), called at paged_kv_cache.cc:1550 as (pages, kv_data, position_map).
 * pages (num_pages, page_size, d_qk). */
int tvmkv_kv_cache_transpose_append_mla(void* pages, const void* kv_data, const int32_t* position_map,
                                        int64_t ntoken, int64_t num_pages, int32_t page_size,
                                        int32_t d_qk, void* stream);

/* Slot 15 ragged prefill -- replaces `batch_prefill_ragged_kv`
 * (python/tvm/relax/frontend/nn/llm/_prefill_kernels.py:795-923; llvm form :677-791), calling
 * convention src/runtime/vm/attn_backend.h:392-395:
 * (q, qo_indptr, k, v, kv_indptr, q_rope_position, k_rope_pos_offset, out, lse, causal,
 *  rotary_mode, rope_scale, rope_theta, sm_scale).
 * q (total_q, h_q, d_qk), k (total_kv, h_kv, d_qk), v (total_kv, h_kv, d_v),
 * out (total_q, h_q, d_v) fp16, lse (total_q, h_q) fp32 base-2.  rotary_mode 0: q and k are used
 * as they are; 1 (inline RoPE): q is rotated at q_rope_position[token], key t of sequence b at
 * k_rope_pos_offset[b] + t (built for head dims 64, 128 and 256). */
int tvmkv_batch_prefill_ragged_kv(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                  const int32_t* kv_indptr, const int32_t* q_rope_position,
                                  const int32_t* k_rope_pos_offset, void* output, float* lse,
                                  int64_t causal, int64_t rotary_mode, double rope_scale,
                                  double rope_theta, double sm_scale, int32_t batch_size,
                                  int64_t total_q, int32_t h_q, int32_t h_kv, int32_t d_qk,
                                  int32_t d_v, void* stream);

/* Slots 16/18 paged prefill -- replaces `batch_prefill_paged_kv`
 * (_prefill_kernels.py:217-391; llvm form :54-214), calling convention attn_backend.h:239-242:
 * (q, qo_indptr, pages, page_indptr, page_indices, length_info, k_rope_pos_offset,
 *  q_rope_position, out, lse, causal, rotary_mode, rope_scale, rope_theta, sm_scale).
 * length_info is (batch,) = last_page_len, or (3, batch) = [last_page_len; sliding_window_offset;
 * sink_size] when sliding_window != 0 (python/tvm/relax/frontend/nn/llm/_kernel_common.py:147-170).
 * kv_len = (npages-1)*page_size + last_page_len, 0 without pages; in the (3, batch) form the keys
 * are the first sink_size cached tokens followed by those from sliding_window_offset on, and with
 * causal != 0 and sliding_window_size > 0 query row r sees only the last sliding_window_size - r - 1
 * keys (_kernel_common.py:138-144).  rotary_mode as for the ragged kernel, key positions counted
 * over the keys as just defined. */
int tvmkv_batch_prefill_paged_kv(const void* q, const int32_t* q_indptr, const void* pages,
                                 const int32_t* page_indptr, const int32_t* page_values,
                                 const int32_t* length_info, const int32_t* k_rope_pos_offset,
                                 const int32_t* q_rope_position, void* output, float* lse,
                                 int64_t causal, int64_t rotary_mode, double rope_scale,
                                 double rope_theta, double sm_scale, int32_t batch_size,
                                 int64_t total_q, int64_t nnz_pages, int64_t num_pages, int32_t h_q,
                                 int32_t h_kv, int32_t d, int32_t page_size, int32_t sliding_window,
                                 int32_t sliding_window_size, void* stream);

/* Slot 16 followed by slot 23 in one launch; no counterpart among the reference's kernels.
 * `output` / `lse` already hold an attention state of the same query rows (what the ragged kernel
 * wrote for the new tokens, paged_kv_cache.cc:2169-2172); the attention over the pages is merged
 * into it in the kernel's epilogue with the arithmetic of `merge_state_inplace`
 * (_decode_kernels.py:441-450), so the temporary output and the separate merge pass of
 * paged_kv_cache.cc:2285-2292 are not needed.  Arguments as tvmkv_batch_prefill_paged_kv. */
int tvmkv_batch_prefill_paged_kv_merge(const void* q, const int32_t* q_indptr, const void* pages,
                                       const int32_t* page_indptr, const int32_t* page_values,
                                       const int32_t* length_info, const int32_t* k_rope_pos_offset,
                                       const int32_t* q_rope_position, void* output, float* lse,
                                       int64_t causal, int64_t rotary_mode, double rope_scale,
                                       double rope_theta, double sm_scale, int32_t batch_size,
                                       int64_t total_q, int64_t nnz_pages, int64_t num_pages,
                                       int32_t h_q, int32_t h_kv, int32_t d, int32_t page_size,
                                       int32_t sliding_window, int32_t sliding_window_size,
                                       void* stream);

/* Slots 15, 16 and 23 in one launch; no counterpart among the reference's kernels.  A chunked-
 * prefill step of a plain (no sliding window, no inline RoPE, no token tree) cache in one pass: every
 * query attends to the tokens its sequence has in the page pool (all visible) and to the new
 * tokens k, v of the call under the causal mask, which is what the reference computes as ragged
 * self-attention + paged cross-attention + merge_state_inplace (paged_kv_cache.cc:2161-2180,
 * :2285-2292), without the temporary output, the second read of q and the merge pass.
 * k, v (total_q, h_kv, d): the rows of the queries' own tokens, indexed by q_indptr. */
int tvmkv_batch_prefill_cached_and_new_kv(const void* q, const int32_t* q_indptr, const void* k,
                                          const void* v, const void* pages,
                                          const int32_t* page_indptr, const int32_t* page_values,
                                          const int32_t* last_page_len, void* output, float* lse,
                                          double sm_scale, int32_t batch_size, int64_t total_q,
                                          int64_t nnz_pages, int64_t num_pages, int32_t h_q,
                                          int32_t h_kv, int32_t d, int32_t page_size, void* stream);

/* The same pass with the queries taken from the fused qkv tensor of the step (rows of
 * (h_q + 2*h_kv) * d elements whose first h_q heads are q), rotated inside the kernel at
 * q_rope_position[token] when apply_rope != 0 (rotate-half RoPE in fp32, rounded once to fp16, as
 * slot 24 does it): together with tvmkv_fused_rope_append(q = NULL) a chunked-prefill step never
 * writes the rotated q rows to memory or reads them back.  k, v: the rotated k and the v rows of the
 * new tokens, as tvmkv_fused_rope_append leaves them. */
int tvmkv_batch_prefill_cached_and_new_kv_fused_q(const void* qkv, const int32_t* q_rope_position,
                                                  int64_t apply_rope, double rope_scale,
                                                  double rope_theta, const int32_t* q_indptr,
                                                  const void* k, const void* v, const void* pages,
                                                  const int32_t* page_indptr,
                                                  const int32_t* page_values,
                                                  const int32_t* last_page_len, void* output,
                                                  float* lse, double sm_scale, int32_t batch_size,
                                                  int64_t total_q, int64_t nnz_pages, int64_t num_pages,
                                                  int32_t h_q, int32_t h_kv, int32_t d,
                                                  int32_t page_size, void* stream);

/* Slots 17/19 paged decode -- replaces `batch_decode_paged_kv`
 * (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:181-411; llvm form :49-178), calling
 * convention attn_backend.h:511-514:
 * (q, pages, page_indptr, page_indices, length_info, k_rope_pos_offset, q_rope_position, out,
 *  lse, rotary_mode, rope_scale, rope_theta, sm_scale).
 * q/out (B, h_q, d) fp16, lse (B, h_q) fp32.  Split-KV across workgroups with a merge pass;
 * the partition count is derived from B and nnz_pages only (no host read of the page table).
 * Head dims 64, 128 and 256, any GQA group (groups above 16 are walked in blocks of 16 heads), with the
 * (3, batch) length_info and rotary_mode = 1 built in for all of them. */
int tvmkv_batch_decode_paged_kv(const void* q, const void* pages, const int32_t* page_indptr,
                                const int32_t* page_values, const int32_t* length_info,
                                const int32_t* k_rope_pos_offset, const int32_t* q_rope_position,
                                void* output, float* lse, int64_t rotary_mode, double rope_scale,
                                double rope_theta, double sm_scale, int32_t batch_size,
                                int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                                int32_t d, int32_t page_size, int32_t sliding_window, void* stream);

/* The attention launchers with a frequency variant for their in-kernel RoPE (rotary_mode != 0).  The
 * reference bakes the model's rope_scaling dictionary into every attention kernel when it builds them
 * (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:138,150,301,321; _prefill_kernels.py:159,171,336,357,
 * 752,758,877,894; kv_cache.py:494-497); here the description travels with the call.  rope_scaling NULL =
 * the default frequencies, i.e. the launchers without the suffix.  As in the reference's `_rope`
 * (_kernel_common.py:115-127) the attention kernels rotate the whole head with the rotate-half pairing,
 * whatever rotary_dim or pairing the split-rotary kernel of the variant uses, and take no factor tensor
 * (LONGROPE inside the attention kernels is the default frequencies times its magnitude).  The other
 * arguments are those of the launcher without the suffix; tvmkv_batch_prefill_paged_kv_scaled takes
 * merge_into != 0 for tvmkv_batch_prefill_paged_kv_merge. */
int tvmkv_batch_decode_paged_kv_scaled(const void* q, const void* pages, const int32_t* page_indptr,
                                       const int32_t* page_values, const int32_t* length_info,
                                       const int32_t* k_rope_pos_offset, const int32_t* q_rope_position,
                                       void* output, float* lse, int64_t rotary_mode, double rope_scale,
                                       double rope_theta, double sm_scale, int32_t batch_size,
                                       int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                                       int32_t d, int32_t page_size, int32_t sliding_window,
                                       const tvmkv_rope_scaling* rope_scaling, void* stream);
int tvmkv_batch_prefill_ragged_kv_scaled(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                         const int32_t* kv_indptr, const int32_t* q_rope_position,
                                         const int32_t* k_rope_pos_offset, void* output, float* lse,
                                         int64_t causal, int64_t rotary_mode, double rope_scale,
                                         double rope_theta, double sm_scale, int32_t batch_size, int64_t total_q,
                                         int32_t h_q, int32_t h_kv, int32_t d_qk, int32_t d_v,
                                         const tvmkv_rope_scaling* rope_scaling, void* stream);
int tvmkv_batch_prefill_paged_kv_scaled(const void* q, const int32_t* q_indptr, const void* pages,
                                        const int32_t* page_indptr, const int32_t* page_values,
                                        const int32_t* length_info, const int32_t* k_rope_pos_offset,
                                        const int32_t* q_rope_position, void* output, float* lse, int64_t causal,
                                        int64_t rotary_mode, double rope_scale, double rope_theta,
                                        double sm_scale, int32_t batch_size, int64_t total_q, int64_t nnz_pages,
                                        int64_t num_pages, int32_t h_q, int32_t h_kv, int32_t d,
                                        int32_t page_size, int32_t sliding_window, int32_t sliding_window_size,
                                        int32_t merge_into, const tvmkv_rope_scaling* rope_scaling, void* stream);
int tvmkv_batch_tree_attn_scaled(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                 const int32_t* kv_indptr, const int32_t* q_rope_position,
                                 const int32_t* mn_indptr, const int32_t* mask, void* output, float* lse,
                                 int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                 int32_t batch_size, int64_t total_q, int32_t h_q, int32_t h_kv, int32_t d,
                                 const tvmkv_rope_scaling* rope_scaling, void* stream);

/* Slots 24 + 13 + 17 in one launch (no counterpart among the reference's kernels; what
 * AttentionWithFusedQKV does for a decode step, src/runtime/vm/paged_kv_cache.cc:1360-1373 and
 * :2236-2260, as three kernels): the decode step of one layer over a plain cache.  qkv is the fused
 * (batch, h_q + 2 h_kv, d) tensor of the step, one new token per sequence.  The kernel reads q from it
 * and rotates it at q_rope_position[b] (apply_rope != 0: rotate-half RoPE with the default frequencies
 * theta^(-2i/d); 0: no rotation); the work items of every sequence's last chunk rotate the new k row the
 * same way and write it and the v row to slot append_position_map[b] (page * page_size + offset, -1 =
 * none) of `pages`, wait for those stores and then attend to the slot like to any cached token.  The
 * page table must already cover the new token, i.e. the step appends before it attends
 * (paged_kv_cache.cc:990-997).  Results as tvmkv_batch_decode_paged_kv; the same head dims and page
 * sizes; a group of more than 16 query heads per kv head is served by work items of 32 heads. */
int tvmkv_fused_decode_step(const void* qkv, void* pages, const int32_t* page_indptr, const int32_t* page_values,
                            const int32_t* last_page_len, const int32_t* q_rope_position,
                            const int32_t* append_position_map, void* output, float* lse, int64_t apply_rope,
                            double rope_scale, double rope_theta, double sm_scale, int32_t batch_size,
                            int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv, int32_t d,
                            int32_t page_size, void* stream);

/* tvmkv_batch_decode_paged_kv for callers that cannot allocate.  It has no counterpart in the
 * reference; it is for code under HIP graph capture, tight serving loops and harnesses that
 * forbid hipMalloc.  Arguments and results as tvmkv_batch_decode_paged_kv.  Its scratch memory
 * (arrival counters and split-KV partial states) is an array of 24 MiB built into the library, one
 * per device, held until the process ends; the call makes no hipMalloc / hipFree and returns
 * TVMKV_EINVAL with a message when the shapes need more: 256 KiB + (nnz_pages / chunk_pages +
 * batch_size) * h_q * (head_dim + 2) * 4 bytes, chunk_pages as tvmkv_decode_split_plan reports
 * (configs of 64 x 8k-token and 8 x 128k-token sequences need 8 and 12 MiB).  All calls on a device
 * share the array: calls that overlap on one device (different streams) race, stream-ordered
 * calls do not.  A call captured into a graph may be replayed: the workgroup that merges the chunks
 * of a sequence puts the arrival counter back to zero.  (tvmkv_batch_decode_paged_kv under capture
 * works on a stream it has been called on before with shapes at least as large; when it would have
 * to allocate it returns TVMKV_EINVAL and leaves the capture intact.) */
int tvmkv_batch_decode_paged_kv_noalloc(const void* q, const void* pages, const int32_t* page_indptr,
                                        const int32_t* page_values, const int32_t* length_info,
                                        const int32_t* k_rope_pos_offset,
                                        const int32_t* q_rope_position, void* output, float* lse,
                                        int64_t rotary_mode, double rope_scale, double rope_theta,
                                        double sm_scale, int32_t batch_size, int64_t nnz_pages,
                                        int64_t num_pages, int32_t h_q, int32_t h_kv, int32_t d,
                                        int32_t page_size, int32_t sliding_window, void* stream);

/* Slot 21 ragged prefill with a token-tree mask -- replaces `batch_tree_attn`
 * (python/tvm/relax/frontend/nn/llm/tree_attn.py:264-603; llvm form :68-259), calling convention
 * attn_backend.h:669-672:
 * (q, qo_indptr, k, v, kv_indptr, q_rope_position, mn_indptr, mask, out, lse, rotary_mode,
 *  rope_scale, rope_theta, sm_scale).
 * mn_indptr (batch+1) gives the first tree node of each sequence, mask (nodes, 2) holds per node
 * its pre-order number and the end of the range its subtree covers; the last
 * mn_indptr[b+1]-mn_indptr[b] keys of sequence b are its tree nodes, and a query node sees the keys
 * before the tree plus the nodes n with mask[n][0] <= mask[self][0] < mask[n][1]
 * (tree_attn.py:48-65).  Under rotary_mode 1 key t is rotated at q_rope_position[kv_indptr[b]+t]. */
int tvmkv_batch_tree_attn(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                          const int32_t* kv_indptr, const int32_t* q_rope_position,
                          const int32_t* mn_indptr, const int32_t* mask, void* output, float* lse,
                          int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                          int32_t batch_size, int64_t total_q, int32_t h_q, int32_t h_kv, int32_t d,
                          void* stream);

/* Slot 20 paged prefill with a token-tree mask -- replaces `tree_attn_paged_kv`
 * (tree_attn.py:798-1259; llvm form :606-797), calling convention attn_backend.h:623-626:
 * (q, qo_indptr, pages, page_indptr, page_indices, length_info, k_rope_pos_offset,
 *  q_rope_position, out, lse, rotary_mode, rope_scale, rope_theta, sm_scale, tree_order_indptr,
 *  tree_order).  Like the reference kernel (tree_attn.py:700-702) it rejects rotary_mode != 0. */
int tvmkv_tree_attn_paged_kv(const void* q, const int32_t* q_indptr, const void* pages,
                             const int32_t* page_indptr, const int32_t* page_values,
                             const int32_t* length_info, const int32_t* k_rope_pos_offset,
                             const int32_t* q_rope_position, void* output, float* lse,
                             int64_t rotary_mode, double rope_scale, double rope_theta,
                             double sm_scale, const int32_t* tree_order_indptr,
                             const int32_t* tree_order, int32_t batch_size, int64_t total_q,
                             int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                             int32_t d, int32_t page_size, int32_t sliding_window, void* stream);

/* Slot 22 MLA paged prefill (also used for MLA decode, paged_kv_cache.cc:954-956) -- replaces
 * `batch_prefill_paged_kv_mla` (_prefill_kernels.py:927-1071), calling convention
 * attn_backend.h:248-249: (q, qo_indptr, pages, page_indptr, page_indices, length_info, out, lse,
 * causal, sm_scale).  q (total_q, h_q, d_latent + d_rope), pages (num_pages, page_size,
 * d_latent + d_rope), out (total_q, h_q, d_latent). */
int tvmkv_batch_prefill_paged_kv_mla(const void* q, const int32_t* q_indptr, const void* pages,
                                     const int32_t* page_indptr, const int32_t* page_values,
                                     const int32_t* length_info, void* output, float* lse,
                                     int64_t causal, double sm_scale, int32_t batch_size,
                                     int64_t total_q, int64_t nnz_pages, int64_t num_pages,
                                     int32_t h_q, int32_t d_latent, int32_t d_rope,
                                     int32_t page_size, void* stream);

/* Slot 23 `f_merge_inplace` -- replaces `merge_state_inplace` (_decode_kernels.py:455-526),
 * called at paged_kv_cache.cc:2292, :2329, :1557 as (v, s, v_other, s_other).
 * v (N, H, D) fp16 and s (N, H) fp32 are updated in place. */
int tvmkv_merge_state_inplace(void* v, float* s, const void* v_other, const float* s_other,
                              int64_t n, int32_t h, int32_t d, void* stream);

/* Slot 25 `f_copy_single_page` -- replaces `copy_single_page` / `copy_single_page_mla`
 * (_page_kernels.py:169-210), called at paged_kv_cache.cc:728 as
 * (pages, src_page_id, tgt_page_id, copy_length). */
int tvmkv_copy_single_page(void* pages, int64_t src_page_id, int64_t tgt_page_id, int64_t copy_length,
                           int64_t num_pages, int32_t num_kv_heads, int32_t page_size,
                           int32_t head_dim, void* stream);
int tvmkv_copy_single_page_mla(void* pages, int64_t src_page_id, int64_t tgt_page_id,
                               int64_t copy_length, int64_t num_pages, int32_t page_size,
                               int32_t d_qk, void* stream);

/* Slot 26 `f_debug_get_kv` -- replaces `tir_kv_cache_debug_get_kv(_mla)`
 * (_page_kernels.py:106-166), called at paged_kv_cache.cc:1718 / :1764 as
 * (pages, position_map, k_data, v_data, layer_id) / (pages, position_map, kv_data, layer_id).
 * k_data/v_data (num_layers, seqlen, num_kv_heads, head_dim); writes layer `layer_id`. */
int tvmkv_kv_cache_debug_get_kv(const void* pages, const int32_t* position_map, void* k_data,
                                void* v_data, int64_t layer_id, int64_t seqlen, int64_t num_pages,
                                int32_t num_kv_heads, int32_t page_size, int32_t head_dim,
                                void* stream);
int tvmkv_kv_cache_debug_get_kv_mla(const void* pages, const int32_t* position_map, void* kv_data,
                                    int64_t layer_id, int64_t seqlen, int64_t num_pages,
                                    int32_t page_size, int32_t d_qk, void* stream);

/* Slot 27 `f_compact_copy` -- replaces `compact_kv_copy` (_page_kernels.py:235-263), called at
 * paged_kv_cache.cc:759-760 as (pages, copy_length_indptr, copy_src_dst_pos, batch_size).
 * copy_src_dst_pos is (2, total_copy_length): row 0 = source slots, row 1 = destination slots. */
int tvmkv_compact_kv_copy(void* pages, const int32_t* copy_length_indptr,
                          const int32_t* copy_src_dst_pos, int32_t batch_size,
                          int32_t total_copy_length, int64_t num_pages, int32_t num_kv_heads,
                          int32_t page_size, int32_t head_dim, void* stream);

/* Tuning options (no counterpart in the reference).  Each starts from an environment variable read
 * once when the library is loaded (TVMKV_ + the upper-case name) and defaults to 0:
 *   decode_chunk_pages     pages per split-KV chunk of the decode kernel (a multiple of 8); 0 = from shapes
 *   decode_separate_merge  != 0: merge the decode chunks in a second launch instead of inside the kernel
 *   decode_wgs_per_cu      > 0: cap the decode grid at this many workgroups per compute unit
 *   mla_chunk_tokens       lower bound of the tokens per split-KV chunk of MLA decode; 0 = 128
 *   mla_separate_merge     accepted and ignored: the MLA decode chunks are always merged in a second launch
 *   prefill_kv_splits      > 0: the paged prefill, one-pass chunked prefill and paged tree-attention launches
 *                          split the keys of every row tile over this many workgroups (at most 64) and merge
 *                          the states in a second launch; 0 = derived from the shapes (launches with few row
 *                          tiles and long cached sequences are split, all others are not)
 *   no_fused_decode_step   != 0: the cache object runs a plain decode step as two launches (split + RoPE +
 *                          append, then decode attention) instead of tvmkv_fused_decode_step */
int tvmkv_set_option(const char* name, int64_t value);
int tvmkv_get_option(const char* name, int64_t* value);

/* Host view of the decode split (no counterpart in the reference; the tests check the arithmetic the
 * kernel repeats on the device).  page_indptr_host is a HOST array (batch_size + 1).  Writes the
 * chunk size in pages and the number of chunk slots of the launch; when slot_seq and slot_chunk are
 * not NULL (room for slot_capacity entries each) also the sequence and chunk index every slot
 * resolves to, -1 for a spare slot.  The figures are those of a cache with 16-token pages; with pages
 * of 16 << s tokens (s = 1, 2, 3) the launch uses chunks of max(1, chunk_pages(nnz_pages << s) >> s) pages. */
int tvmkv_decode_split_plan(const int32_t* page_indptr_host, int32_t batch_size, int64_t nnz_pages,
                            int32_t h_kv, int32_t* chunk_pages, int64_t* num_slots, int32_t* slot_seq,
                            int32_t* slot_chunk, int64_t slot_capacity);

/* Frees the split-KV scratch buffers that the launchers keep for (current device, stream), after
 * synchronising the stream (no counterpart in the reference).  The launchers keep one buffer per device,
 * stream and kernel family, grown on demand and otherwise never freed: a caller that creates and destroys
 * streams calls this before it destroys one.  A buffer whose address a graph under capture has recorded is
 * not freed but kept until the process ends (the graph may be replayed at any time); for the same reason a
 * larger eager call on a stream that was captured from leaves the old buffer in place and allocates the
 * new one beside it.  Refused while the stream is being captured. */
int tvmkv_release_scratch(void* stream);
/* Test aid (no counterpart in the reference): sets the launch count of every pooled scratch buffer and of
 * the built-in buffers of tvmkv_batch_decode_paged_kv_noalloc.  The arrival counters of a split-KV launch
 * are tagged with the low 32 bits of that count; the tests set it just below 2^32 and run launches across
 * the wrap. */
int tvmkv_debug_set_scratch_launches(uint64_t launches);
/* The same arithmetic on the host alone: advances *launches and returns the epoch of that launch (never
 * 0); *wrapped = 1 when the epochs started over, which is when the launchers clear the counters. */
uint32_t tvmkv_debug_next_scratch_epoch(uint64_t* launches, int32_t* wrapped);

/* ======================================================================================
 * (2) Cache object
 * ====================================================================================== */

typedef struct tvmkv_cache tvmkv_cache;

/* attn_kinds values (src/runtime/vm/attn_utils.h:66-71) and rope modes (:341-345). */
#define TVMKV_ATTN_MHA 0
#define TVMKV_ATTN_MLA 1
#define TVMKV_ATTN_MHA_SLIDING 3
#define TVMKV_ROPE_NONE 0
#define TVMKV_ROPE_NORMAL 1
#define TVMKV_ROPE_INLINE 2

/* `vm.builtin.paged_attention_kv_cache_create` (paged_kv_cache.cc:2532-2640) without the
 * kernel-function arguments (the kernels are this library's own).
 *   cache_config  [reserved_num_seqs, total_token_capacity, prefill_chunk_size, page_size,
 *                  support_sliding_window(, layer_sliding_window_size)]   (n_config 5 or 6)
 *   layer_indptr  [begin, end] layer range owned by this cache (one group: {0, num_layers})
 *   attn_kinds    one TVMKV_ATTN_* per global layer id
 *   dtype_bits    16 (fp16 storage) or 32 (float32 storage: every q / k / v / output tensor handed to the
 *                 verbs is float32 then).  float32 storage, page sizes other than 16 / 32 / 64 / 128 and
 *                 head dims other than 64 / 80 / 96 / 112 / 128 / 256 (multiples of 8, of 4 for float32, up
 *                 to 256) run on the generic kernels, as do head dims 80 / 96 / 112 in a cache with sliding
 *                 windows or RoPE inside the attention kernels; that rotation needs a head dim that is a
 *                 multiple of 16 (of 8 for float32), and none of this is built for caches with MLA layers
 *                 (TVMKV_EUNSUPPORTED)
 *   device_id     HIP device ordinal, or -1 for a HOST-ONLY cache: page-pool bookkeeping and
 *                 auxiliary arrays work, anything that touches device memory returns
 *                 TVMKV_ENODEVICE. */
int tvmkv_cache_create(const int64_t* cache_config, int32_t n_config, const int64_t* layer_indptr,
                       int32_t n_layer_indptr, int64_t num_qo_heads, int64_t num_kv_heads,
                       int64_t qk_head_dim, int64_t v_head_dim, const int64_t* attn_kinds,
                       int32_t n_attn_kinds, int32_t enable_kv_transfer, int32_t rope_mode,
                       double rope_scale, double rope_theta, int32_t dtype_bits, int32_t device_id,
                       tvmkv_cache** out);
void tvmkv_cache_destroy(tvmkv_cache* cache);
/* The RoPE frequency variant of the model (what the reference bakes into the f_split_rotary kernel it is
 * created with, paged_kv_cache.cc:2583) and, for longrope, the factor tensor the reference's create call
 * takes as `rope_ext_factors` (device memory, head_dim float32, kept by reference: it must outlive the
 * cache).  scaling NULL or rope_type DEFAULT: back to plain frequencies.  Caches that rotate inside the
 * attention kernels (RoPE mode inline, i.e. sliding-window caches) hand the variant to those kernels (the
 * *_scaled launchers); they take no factor tensor. */
int tvmkv_cache_set_rope_scaling(tvmkv_cache* cache, const tvmkv_rope_scaling* scaling,
                                 const float* rope_ext_factors);
/* Stream on which the cache enqueues kernels (the reference uses the device's current stream,
 * paged_kv_cache.cc:524).  Default: the null stream. */
int tvmkv_cache_set_stream(tvmkv_cache* cache, void* stream);

/* vm.builtin.kv_state_* (src/runtime/vm/kv_state.cc:33-55). */
int tvmkv_kv_state_clear(tvmkv_cache* cache);
int tvmkv_kv_state_add_sequence(tvmkv_cache* cache, int64_t seq_id);
int tvmkv_kv_state_remove_sequence(tvmkv_cache* cache, int64_t seq_id);
int tvmkv_kv_state_fork_sequence(tvmkv_cache* cache, int64_t parent_seq_id, int64_t child_seq_id,
                                 int64_t fork_pos);
int tvmkv_kv_state_popn(tvmkv_cache* cache, int64_t seq_id, int32_t n);
/* token_tree_parent_ptr may be NULL (n_tree ignored).  Unknown ids and lengths of 0 are found before anything
 * changes.  A step that fails later (the pool runs out, a sliding window meets a shared prefix) has already
 * bumped sequence lengths, as in the reference (paged_kv_cache.cc:919), where such a failure aborts the
 * program: here the cache then refuses every verb except tvmkv_kv_state_clear with a message that says so. */
int tvmkv_kv_state_begin_forward(tvmkv_cache* cache, const int64_t* seq_ids,
                                 const int64_t* append_lengths, int32_t batch_size,
                                 const int64_t* token_tree_parent_ptr, int32_t n_tree);
int tvmkv_kv_state_end_forward(tvmkv_cache* cache);

/* vm.builtin.attention_kv_cache_* (src/runtime/vm/kv_state.cc:58-116).  Tensors are device
 * pointers to contiguous arrays; the row counts are shape[0] of the reference's tensors. */
int tvmkv_attention_kv_cache_enable_sliding_window_for_seq(tvmkv_cache* cache, int64_t seq_id,
                                                           int32_t sliding_window_size,
                                                           int32_t attn_sink_size);
int tvmkv_attention_kv_cache_commit_accepted_token_tree_nodes(tvmkv_cache* cache,
                                                              const int64_t* seq_ids,
                                                              const int64_t* leaf_indices,
                                                              int32_t n);
int tvmkv_attention_kv_cache_empty(tvmkv_cache* cache, int32_t* out);
int tvmkv_attention_kv_cache_get_num_available_pages(tvmkv_cache* cache, int32_t* out);
int tvmkv_attention_kv_cache_get_total_sequence_length(tvmkv_cache* cache, int32_t* out);
/* Returns a device pointer to q_rope_position_map (int32) and its length. */
int tvmkv_attention_kv_cache_get_query_positions(tvmkv_cache* cache, const int32_t** device_ptr,
                                                 int64_t* length);
/* (cache, layer_id, sm_scale, qkv, out): qkv (qkv_rows, Hq+2Hkv, D), out (out_rows, Hq, D). */
int tvmkv_attention_kv_cache_attention_with_fused_qkv(tvmkv_cache* cache, int64_t layer_id,
                                                      double sm_scale, const void* qkv,
                                                      int64_t qkv_rows, void* out, int64_t out_rows);
/* (cache, layer_id, sm_scale, q, k, v, o, lse): rows must equal the batch's total append length. */
int tvmkv_attention_kv_cache_self_attention(tvmkv_cache* cache, int64_t layer_id, double sm_scale,
                                            const void* q, const void* k, const void* v, void* o,
                                            float* lse, int64_t rows, int32_t k_heads,
                                            int32_t qk_dim, int32_t v_dim);
/* (cache, layer_id, sm_scale, q, o, lse). */
int tvmkv_attention_kv_cache_cross_attention(tvmkv_cache* cache, int64_t layer_id, double sm_scale,
                                             const void* q, void* o, float* lse, int64_t rows);
/* `vm.builtin.attention_kv_cache_attention_with_shared_kv` (src/runtime/vm/kv_state.cc:97-105,
 * paged_kv_cache.cc:1487-1525): (cache, source_layer_id, sm_scale, q, current_k, current_v, o).
 * The step's queries attend to the K/V that layer `source_layer_id` holds in its pages plus the
 * rows current_k / current_v (rows, Hkv, D) of the step's own tokens; nothing is appended and q is
 * used as it is handed in.  rows must equal the batch's total append length. */
int tvmkv_attention_kv_cache_attention_with_shared_kv(tvmkv_cache* cache, int64_t source_layer_id,
                                                      double sm_scale, const void* q,
                                                      const void* current_k, const void* current_v,
                                                      void* o, int64_t rows);
/* (cache, layer_id, kv): kv (rows, qk_head_dim). */
int tvmkv_attention_kv_cache_append_mla_kv(tvmkv_cache* cache, int64_t layer_id, const void* kv,
                                           int64_t rows);
/* (cache, o_self, lse_self, o_cross, lse_cross): merges into o_self / lse_self. */
int tvmkv_attention_kv_cache_merge_attn_output_inplace(tvmkv_cache* cache, void* o_self,
                                                       float* lse_self, const void* o_cross,
                                                       const float* lse_cross, int64_t rows,
                                                       int32_t heads, int32_t dim);
/* (cache, seq_id, start_pos, end_pos, k_data, v_data): (num_layers, end-start, Hkv, D) each.
 * Synchronises the stream before returning (debug path). */
int tvmkv_attention_kv_cache_debug_get_kv(tvmkv_cache* cache, int64_t seq_id, int64_t start_pos,
                                          int64_t end_pos, void* k_data, void* v_data);
int tvmkv_attention_kv_cache_debug_get_kv_mla(tvmkv_cache* cache, int64_t seq_id, int64_t start_pos,
                                              int64_t end_pos, void* kv_data);

/* ---- introspection (no counterpart in the reference's public functions; used by the parity
 * tests to compare page tables, append indices and pool state bit for bit) --------------- */

/* Host copy of one auxiliary array built by begin_forward.  `name` is the reference's member
 * name without the `_on_depths_host_` / `_host_` suffix: "qo_indptr", "page_indptr",
 * "page_indices", "last_page_len", "sliding_window_offset", "sink_size", "k_rope_pos_offset",
 * "page_indptr_sliding_window", "page_indices_sliding_window",
 * "k_rope_pos_offset_sliding_window", "tree_attn_mask", "tree_attn_mn_indptr" (per depth) and
 * "q_rope_position_map", "append_position_map", "cur_append_lengths_indptr",
 * "k_ragged_rope_pos_offset", "commit_copy_length_indptr", "commit_copy_src_pos",
 * "commit_copy_dst_pos" (depth ignored).  The pointer stays valid until the next call on the cache. */
int tvmkv_cache_get_aux(tvmkv_cache* cache, const char* name, int32_t depth, const int32_t** data,
                        int64_t* size);
/* flags[0]=num_depths, [1]=append_before_attn, [2]=is_decode_request,
 * [3..4]=use_decode_kernel per depth, [5..6]=is_chain per depth, [7]=num_total_pages,
 * [8]=rope_mode in effect. */
int tvmkv_cache_get_flags(tvmkv_cache* cache, int64_t* flags, int32_t n_flags);
/* Serialises the pool into `buf` (int64): [n_free_pages, pages..., n_free_blocks, blocks...,
 * n_blocks, {n_pages, pages..., seq_length, start_pos, sink_length, sliding_window_offset,
 * parent_idx, external_ref_cnt}..., n_seqs, {seq_id, last_block_idx, seq_length,
 * sliding_window_size, last_block_attn_sink_size}... (ascending seq_id)].  *needed receives the
 * element count; returns TVMKV_EINVAL if cap is too small (call again with a bigger buffer). */
int tvmkv_cache_dump_state(tvmkv_cache* cache, int64_t* buf, int64_t cap, int64_t* needed);
/* Log of the page copies issued by fork (src, tgt, length) triples since the last clear. */
int tvmkv_cache_get_copy_log(tvmkv_cache* cache, const int64_t** triples, int64_t* n_triples);
/* Device pointer of one layer's page pool (local layer index). */
int tvmkv_cache_get_pages(tvmkv_cache* cache, int64_t local_layer, void** device_ptr,
                          int64_t* num_bytes);

#ifdef __cplusplus
}
#endif
#endif /* TVMKV_H_ */
