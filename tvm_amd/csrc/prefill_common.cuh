// Declarations of the prefill kernels (kernels_prefill.hip): launch parameters, the row-tile slot arithmetic and the LDS swizzles of the K / V tiles.
#ifndef TVMKV_CSRC_PREFILL_COMMON_CUH_
#define TVMKV_CSRC_PREFILL_COMMON_CUH_

#include "kernels_common.cuh"

namespace tvmkv {

constexpr int NW = 4;        // wavefronts per workgroup, 32 rows each
constexpr int BM = NW * 32;  // rows per workgroup
constexpr int RPW = 64 / NW; // token rows of a tile copied by each wave
constexpr int BN = 64;   // kv tokens per tile

struct PrefillParams {
  const half_t* q;
  const int32_t* q_indptr;
  const half_t* k;  // ragged
  const half_t* v;
  const int32_t* kv_indptr;
  const half_t* pages;  // paged
  const int32_t* page_indptr;
  const int32_t* page_values;
  const int32_t* last_page_len;
  half_t* output;
  float* lse;
  int batch_size;
  int h_q;
  int h_kv;
  int group;
  int causal;
  float scale_log2;
  // extended form (prefill_kernel<..., EXT = true>): sliding-window cache, per-layer sliding-window
  // mask, inline RoPE
  const int32_t* window_offset;      // paged, (B): physical index of the first token of the window, or NULL
  const int32_t* sink_size;          // paged, (B): attention-sink tokens kept at the front, or NULL
  int layer_window;                  // > 0 with causal: row r sees only the last layer_window - r - 1 keys
  const int32_t* q_rope_position;    // (total_q) position of each query token (inline RoPE)
  const int32_t* k_rope_pos_offset;  // (B) position of logical key 0 (inline RoPE)
  int rotary;
  float rope_scale;
  // token-tree mask (python/tvm/relax/frontend/nn/llm/tree_attn.py:48-65), or NULL
  const int32_t* tree_indptr;  // (B + 1) first tree node of each sequence
  const int32_t* tree_order;   // (nodes, 2): pre-order number of the node, end of its subtree's range
  int k_pos_from_q;            // ragged tree attention under inline RoPE: key t sits at q_rope_position[t]
  // != 0: output / lse already hold an attention state of the same rows, and this kernel's state is
  // merged into it (the arithmetic of merge_state_inplace) instead of overwriting it
  int merge_into;
  // q rows are read from the fused qkv tensor of the step: q points at it, consecutive tokens are
  // q_token_stride elements apart (0 = a dense q tensor, h_q * d_qk); q_inline_rope != 0: the kernel
  // rotates them at q_rope_position[token] itself (with rope_scale and the divisors of the launch)
  int64_t q_token_stride;
  int q_inline_rope;
  // > 1: gridDim.z workgroups share a row tile, each taking an equal share of its key tiles and writing
  // its own attention state: output / lse then point at kv_splits arrays of split_rows rows each
  int kv_splits;
  int64_t split_rows;
  int page_shift;   // pages hold 16 << page_shift tokens; the kernel walks them as runs of 16-token pages
  int stream_kv;    // != 0: every K/V row is read by one row tile only: copy it with the streaming hint
  int d_mem;        // padded head dims (prefill_kernel<..., PAD = true>): elements per row in memory
  // how the entries of the RoPE table are used (InlineRopeTable): position * entry instead of position /
  // entry; separate entries for the two halves of a head; a factor on cos and sin
  int rope_inverse;
  int rope_halves_differ;
  float rope_magnitude;
};

// One entry per element of the head for in-kernel RoPE (the default: theta^(2i/D) for elements i and
// i + D/2), computed on the host with the libm call the CPU kernels use
struct PrefillRopeDivisors {
  float v[256];
};

__device__ __forceinline__ int tile_slot_begin(const int32_t* q_indptr, int b, int group) {
  return static_cast<int>((static_cast<int64_t>(q_indptr[b]) * group) / BM) + b;
}

// LDS image of a tile of BN token rows x W features (W = 64 or 128), pieces of 8 features.
// Piece c of row r is kept at piece position c ^ swz(r).
//  * K is read as MFMA A-fragments with ds_read_b128, 16 lanes = 16 consecutive rows at the same
//    piece: swz spreads 16 consecutive rows over the 16 piece positions of a 256-byte bank line.
//  * V is read with ds_read_b64_tr_b16, 32 lanes = 4 consecutive rows x 64 bytes: swz moves the 4
//    rows to the 4 different 64-byte quarters of the bank line.
template <int W>
__device__ __forceinline__ int k_swizzle(int row) {
  return W == 128 ? (row & 15) : ((row >> 1) & 7);
}
template <int W>
__device__ __forceinline__ int v_swizzle(int row) {
  return W == 128 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2);
}

// SRC of a prefill kernel: where the keys come from.  kRagged: k / v rows of the call; kPaged: the page
// pool; kBoth: the cached tokens of the page pool, all visible, followed by the k / v rows of the call
// under the causal mask.
constexpr int kRagged = 0, kPaged = 1, kBoth = 2;

}  // namespace tvmkv

#endif  // TVMKV_CSRC_PREFILL_COMMON_CUH_
