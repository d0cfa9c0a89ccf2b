// Generic MHA attention for gfx950: what the reference's kernel factories accept for a plain cache and the
// tuned fp16 kernels are not built for -- float32 storage, pages of any size, head dims that are a multiple
// of 4 (fp32) or 8 (fp16) up to 256.  One kernel serves ragged prefill (_prefill_kernels.py:677-923), paged
// prefill (:54-391), paged decode (_decode_kernels.py:49-411) and both token-tree forms (tree_attn.py:93-259,
// :634-797): base-2 online softmax (m = -5e4 to start with), K and V rows read straight from memory into matrix
// operands with one page-table lookup per row.  float32 storage multiplies on v_mfma_f32_16x16x4_f32; fp16 storage
// on the fp16 instructions of the same shape (v_mfma_f32_16x16x32_f16 for the scores, v_mfma_f32_16x16x16_f16 for
// the output, the probabilities rounded to fp16 as in the tuned kernels), float32 sums in both.
//
// Tile: ROWS = 16 * NB query rows of one (sequence, kv head) -- a row is a (token, head of the GQA group)
// pair -- against 16 keys per step and wave.  The four waves of a workgroup take every fourth 16-key block
// and fold their states at the end through LDS; launches with few row tiles also split the keys over
// workgroups (partial states in scratch memory, merged by a second kernel).
//
// Matrix operand layout (v_mfma_f32_16x16x4_f32): lane = 16 * k + i holds A[i][k] and B[k][i]; the result
// register r of lane 16 * g + j is C[4 g + r][j].  Every load of a K / V / q row is one 16-byte piece (4 floats,
// 8 halfs), which the freedom in numbering the contraction index and the output features allows:
//  * S^T = K Q^T: the contraction runs over the features in the order that suits the loads -- lane (i, g) loads
//    piece 4 s + g of key i (of query row i for the B operand) and feeds its elements to consecutive
//    instructions, so A and B agree by construction;
//  * O^T += V^T P: the four keys 4 g + m of lane group g are the contraction slots, which is the order in which
//    lane (j, g) already holds the probabilities of row j; output "block" fb, row i of the product is feature
//    i * KS + fb, so lane (i, g) reads KS consecutive features of a key (the 16 lanes of a group read a whole
//    row) and lane (j, g) ends up with runs of KS consecutive output features.
// The fp16 instructions keep both choices: a lane's 8 halfs of a piece are 8 consecutive contraction slots of
// v_mfma_f32_16x16x32_f16 (lane (i, g) holds A[i][8 g .. 8 g + 7] and B[8 g .. 8 g + 7][i]), and the four keys 4 g + m
// are the four slots A[i][4 g + m] / B[4 g + m][i] that lane group g holds for v_mfma_f32_16x16x16_f16, so the
// V^T operand of feature block fb is one half of each of the lane's four key rows.
#include <algorithm>

#include "kernels_common.cuh"
#include "runtime_support.h"
#include "typed_kernels.h"

namespace tvmkv {
namespace {

struct GAttn {
  const void* q;
  const void* k;
  const void* v;
  const void* pages;
  const int32_t* q_indptr;
  const int32_t* kv_indptr;
  const int32_t* page_indptr;
  const int32_t* page_values;
  const int32_t* last_page_len;
  const int32_t* tree_indptr;
  const int32_t* tree_labels;
  void* out;
  float* lse;
  float* part_o;  // (splits, total_q, h_q, d) normalised partial outputs
  float* part_s;  // (splits, total_q, h_q) their base-2 log-sum-exp, kNoKeys for an empty share
  int64_t total_q;
  int batch, h_q, h_kv, d, page_size, causal, splits;
  float scale_log2;
  // extended form (generic_attn_kernel<..., EXT = true>)
  const int32_t* window_offset;      // paged, (batch): physical index of the first token of the window, or NULL
  const int32_t* sink_size;          // paged, (batch): attention-sink tokens kept at the front, or NULL
  int layer_window;                  // > 0 with causal and a sliding-window cache: the per-layer window mask
  int rotary;                        // q and k are rotated inside the kernel
  const int32_t* q_rope_position;    // (total_q) position of each query token
  const int32_t* k_rope_pos_offset;  // (batch) position of logical key 0; NULL (ragged): key t of sequence b sits at
                                     // q_rope_position[kv_indptr[b] + t]
  float rope_scale;
};

constexpr float kMasked = -1.0e30f;  // a masked score; exp2 of it is 0 against any running maximum
constexpr float kNoKeys = -1.0e30f;  // the log-sum-exp of a share that saw no key

// N consecutive elements (N * sizeof(T) = 8 or 16 bytes, aligned) as floats
template <typename T, int N>
__device__ __forceinline__ void load_run(const T* p, float* out);
template <>
__device__ __forceinline__ void load_run<float, 4>(const float* p, float* out) {
  const float4_t v = *reinterpret_cast<const float4_t*>(p);
#pragma unroll
  for (int e = 0; e < 4; ++e) out[e] = v[e];
}
template <typename T, int N>
__device__ __forceinline__ void store_run(T* p, const float* in);
template <>
__device__ __forceinline__ void store_run<float, 4>(float* p, const float* in) {
  float4_t v;
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = in[e];
  *reinterpret_cast<float4_t*>(p) = v;
}
template <>
__device__ __forceinline__ void store_run<half_t, 4>(half_t* p, const float* in) {
  half4_t v;
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = static_cast<half_t>(in[e]);
  *reinterpret_cast<half4_t*>(p) = v;
}
template <>
__device__ __forceinline__ void store_run<half_t, 8>(half_t* p, const float* in) {
  half8_t v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = static_cast<half_t>(in[e]);
  *reinterpret_cast<half8_t*>(p) = v;
}
__device__ __forceinline__ void store4(float* p, float4_t v) { *reinterpret_cast<float4_t*>(p) = v; }

// In-kernel RoPE (rotate-half over the whole head, python/tvm/relax/frontend/nn/llm/_kernel_common.py:115-127) of
// two 16-byte pieces of a q / k row that lie half a head apart: lo[e] is feature f + e, hi[e] its partner
// f + d/2 + e.  float32 arithmetic, one rounding to the storage type; tbl: the table of InlineRopeTable in LDS (an
// element and its partner share the angle unless the variant's halves differ).
template <int N>
__device__ __forceinline__ void rotate_pair(float* lo, float* hi, int f, int d, float pos_scaled, const float* tbl, int inverse,
                                            int halves_differ, float magnitude) {
#pragma unroll
  for (int e = 0; e < N; ++e) {
    float sn, cs;
    sincos_reduced(inverse ? pos_scaled * tbl[f + e] : pos_scaled / tbl[f + e], sn, cs);
    float sn_hi = sn, cs_hi = cs;
    if (halves_differ) sincos_reduced(inverse ? pos_scaled * tbl[f + d / 2 + e] : pos_scaled / tbl[f + d / 2 + e], sn_hi, cs_hi);
    const float xl = lo[e], xh = hi[e];
    lo[e] = magnitude * (cs * xl - sn * xh);
    hi[e] = magnitude * (cs_hi * xh + sn_hi * xl);
  }
}
__device__ __forceinline__ void rotate_pair(half8_t& lo, half8_t& hi, int f, int d, float pos_scaled, const float* tbl, int inverse,
                                            int halves_differ, float magnitude) {
  float x[8], y[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    x[e] = static_cast<float>(lo[e]);
    y[e] = static_cast<float>(hi[e]);
  }
  rotate_pair<8>(x, y, f, d, pos_scaled, tbl, inverse, halves_differ, magnitude);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    lo[e] = static_cast<half_t>(x[e]);
    hi[e] = static_cast<half_t>(y[e]);
  }
}

// workgroups per CU: the fp16 form holds its operands in half the registers
constexpr int generic_workgroups(int elem_bytes, int dmax, int nb) {
  return elem_bytes == 2 ? (dmax > 128 ? 2 : (nb == 1 ? 4 : 3)) : (dmax > 128 ? 1 : (nb == 1 ? 3 : 2));
}
// 16-row blocks per row tile: one for decode-shaped calls and for head dims above 128 (registers), two when a
// (sequence, kv head) has more than 16 rows on average.  Three and four blocks (fp16 storage, one workgroup fewer
// per CU) measured slower: causal self-attention of 4 x 2048 tokens at head dim 72 173 against 195 TFLOP/s, at
// head dim 48 144 against 197; only calls that rotate inside the kernel gained (head dim 96: 99 against 90).
inline int generic_row_blocks(int d, int rows_hint) { return d > 128 || rows_hint <= 16 ? 1 : 2; }
// Also measured and not kept: a form for prefill-shaped calls whose four waves take rows of their own and share
// stages of 32 keys through LDS (a K / V row fetched and rotated once per 128 query rows).  Plain calls ran slower
// (head dim 72: 156 against 196 TFLOP/s, with the next stage's loads held in registers during the matrix work 109:
// twelve independent waves per CU hide the loads better than three workgroups in step); calls that rotate inside
// the kernel gained (head dim 96: 135 against 103).

// EXT adds what the extended tuned kernels add: the sliding-window cache (the page table covers `sink` tokens at the
// front, evicted tokens up to `window_offset`, then the window; keys have logical indices, sink tokens first, that
// the masks and RoPE use, _kernel_common.py:155-170), the per-layer sliding-window mask (:138-144) and RoPE inside
// the kernel with any frequency variant (the table, one entry per element; the halves of a variant whose halves
// differ are rotated by their own entries).
template <typename T, int DMAX, int NB, bool EXT>
__global__ __launch_bounds__(256, generic_workgroups(sizeof(T), DMAX, NB)) void generic_attn_kernel(GAttn p, InlineRopeTable rope) {
  constexpr bool HALF = sizeof(T) == 2;
  constexpr int ROWS = 16 * NB;
  constexpr int KS = DMAX / 16;  // output feature "blocks": lane (i, g) of the V^T operand owns features i * KS .. + KS - 1
  constexpr int PIECE = 16 / static_cast<int>(sizeof(T));  // elements of a 16-byte load
  constexpr int QS = DMAX / (4 * PIECE);                   // load steps of the score product (4 pieces each)
  constexpr int VP = KS < PIECE ? KS : PIECE;              // elements per load of the V^T operand (8 or 16 bytes)
  static_assert(KS % VP == 0 && DMAX % (4 * PIECE) == 0, "head dim vs load width");
  __shared__ __attribute__((aligned(16))) float o_lds[2 * ROWS * DMAX];
  __shared__ float ml_lds[2 * ROWS * 2];
  __shared__ float rope_lds[EXT ? kMaxHeadDim : 1];

  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  const int j = lane & 15;  // query row of a 16-row block (matrix column) / key of a block / feature of a block
  const int g = lane >> 4;
  const int group = p.h_q / p.h_kv;
  const int kvh = blockIdx.y;
  const int split = blockIdx.z;
  const int d = p.d;

  // the sequence of this row-tile slot: sequence b owns the slots from (q_start(b) * group) / ROWS + b on
  auto q_begin = [&](int b) { return p.q_indptr != nullptr ? p.q_indptr[b] : b; };
  auto slot_begin = [&](int b) { return static_cast<int>(static_cast<int64_t>(q_begin(b)) * group / ROWS) + b; };
  const int slot = blockIdx.x;
  int lo = 0, hi = p.batch - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (slot_begin(mid) <= slot) {
      lo = mid;
    } else {
      hi = mid - 1;
    }
  }
  const int b = lo;
  const int q_start = q_begin(b);
  const int qo_len = q_begin(b + 1) - q_start;
  const int rows = qo_len * group;
  const int r0 = (slot - slot_begin(b)) * ROWS;
  if (r0 >= rows) return;  // the whole workgroup: a slot beyond the sequence's last row tile
  const bool rotary = EXT && p.rotary != 0;
  if (EXT && rotary) {
    if (tid < d) rope_lds[tid] = rope.v[tid];
    __syncthreads();
  }

  const bool paged = p.pages != nullptr;
  int kv_len, kv_start = 0, pbeg = 0;
  int sink = 0, window_first = 0;  // logical key t lies at physical index t (t < sink) or t - sink + window_first
  if (paged) {
    pbeg = p.page_indptr[b];
    const int npages = p.page_indptr[b + 1] - pbeg;
    kv_len = npages > 0 ? (npages - 1) * p.page_size + p.last_page_len[b] : 0;  // _kernel_common.py:155-159
    if (EXT && p.window_offset != nullptr && npages > 0) {
      sink = p.sink_size[b];
      window_first = p.window_offset[b];
      kv_len = kv_len - window_first + sink;
    }
  } else {
    kv_start = p.kv_indptr[b];
    kv_len = p.kv_indptr[b + 1] - kv_start;
  }
  const bool tree = p.tree_labels != nullptr;
  int tree_len = 0, tree_start = 0, tree_base = 0;
  if (tree) {
    tree_base = p.tree_indptr[b];
    tree_len = p.tree_indptr[b + 1] - tree_base;
    tree_start = kv_len - tree_len;
  }
  const bool causal = p.causal != 0 && !tree;
  // the per-layer window mask replaces the causal one: query i of the chunk sees the last max(window - i - 1, 0)
  // cached keys (_kernel_common.py:138-144; sliding-window caches only, as the reference passes it)
  const bool windowed = EXT && causal && p.layer_window > 0 && p.window_offset != nullptr;

  // this lane's query rows (one per 16-row block): key limits, tree label, q fragments
  int limit[NB];
  int lower[NB];
  int child_first[NB];
  float qf[NB][QS][PIECE];  // float32 storage
  half8_t qh[NB][QS];       // fp16 storage: the pieces as they are in memory
  const T* qbase = static_cast<const T*>(p.q);
  // Which 16-byte piece of a q / k row lane group g feeds to load step s of the score product: any assignment
  // serves, as long as q and k agree.  Plain: piece 4 s + g.  With rotation inside the kernel: the first half of
  // the steps takes the pieces of the lower half of the head, the second half their partners half a head away,
  // so that a lane holds both elements of every rotated pair.
  static_assert(QS % 2 == 0, "load steps come in pairs");
  auto piece_feature = [&](int s) {
    if (!(EXT && rotary)) return (4 * s + g) * PIECE;
    const int lower = (4 * (s % (QS / 2)) + g) * PIECE;
    return s < QS / 2 ? lower : lower + d / 2;
  };
  auto piece_inside = [&](int s) {
    if (!(EXT && rotary)) return (4 * s + g) * PIECE < d;
    return (4 * (s % (QS / 2)) + g) * PIECE < d / 2;
  };
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int row = r0 + nb * 16 + j;
    const bool valid = row < rows;
    const int qi = valid ? row / group : 0;
    const int head = kvh * group + (valid ? row % group : 0);
    limit[nb] = !valid ? 0 : (causal && !windowed ? max(0, min(kv_len, kv_len - qo_len + qi + 1)) : kv_len);
    lower[nb] = windowed ? max(kv_len - max(p.layer_window - qi - 1, 0), 0) : 0;
    child_first[nb] = 0;
    if (tree && valid && tree_len > 0) {  // the queries are the last qo_len nodes of the tree
      const int node = min(max(qi + tree_len - qo_len, 0), tree_len - 1);
      child_first[nb] = p.tree_labels[2 * static_cast<int64_t>(tree_base + node)];
    }
    const T* qrow = qbase + (static_cast<int64_t>(q_start + qi) * p.h_q + head) * d;
#pragma unroll
    for (int s = 0; s < QS; ++s) {
      const int f = piece_feature(s);
      const bool inside = valid && piece_inside(s);
      if constexpr (HALF) {
        half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
        qh[nb][s] = inside ? *reinterpret_cast<const half8_t*>(qrow + f) : z;
      } else if (inside) {
        load_run<T, PIECE>(qrow + f, qf[nb][s]);
      } else {
#pragma unroll
        for (int e = 0; e < PIECE; ++e) qf[nb][s][e] = 0.f;
      }
    }
    if (EXT && rotary && valid) {
      const float pos = static_cast<float>(p.q_rope_position[q_start + qi]) * p.rope_scale;
#pragma unroll
      for (int s = 0; s < QS / 2; ++s) {
        if (!piece_inside(s)) continue;
        if constexpr (HALF) {
          rotate_pair(qh[nb][s], qh[nb][s + QS / 2], piece_feature(s), d, pos, rope_lds, rope.inverse, rope.halves_differ, rope.magnitude);
        } else {
          rotate_pair<PIECE>(qf[nb][s], qf[nb][s + QS / 2], piece_feature(s), d, pos, rope_lds, rope.inverse, rope.halves_differ,
                             rope.magnitude);
        }
      }
    }
  }
  // keys of this row tile, and this workgroup's share of their 16-key blocks
  const int last_row = min(rows, r0 + ROWS) - 1;
  const int tile_limit = causal && !windowed ? max(0, min(kv_len, kv_len - qo_len + last_row / group + 1)) : kv_len;
  // the first row of the tile sees the most keys of the window
  const int tile_lower = windowed ? max(kv_len - max(p.layer_window - r0 / group - 1, 0), 0) : 0;
  const int kb_first = tile_lower / 16;
  const int nkb = max((tile_limit + 15) / 16 - kb_first, 0);
  const int kb_lo = kb_first + static_cast<int>(static_cast<int64_t>(split) * nkb / p.splits);
  const int kb_hi = kb_first + static_cast<int>(static_cast<int64_t>(split + 1) * nkb / p.splits);

  float m[NB], lsum[NB];
  float4_t o[NB][KS];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    m[nb] = kNegInit;
    lsum[nb] = 0.f;
#pragma unroll
    for (int fb = 0; fb < KS; ++fb) {
      float4_t z = {0.f, 0.f, 0.f, 0.f};
      o[nb][fb] = z;
    }
  }

  const T* kbase = paged ? static_cast<const T*>(p.pages) : static_cast<const T*>(p.k);
  const T* vbase = paged ? static_cast<const T*>(p.pages) : static_cast<const T*>(p.v);
  const int ps = p.page_size;
  for (int kb = kb_lo + wave; kb < kb_hi; kb += 4) {
    // row of key kb * 16 + j in its tensor (rows of d elements); keys past the end repeat the last one (masked)
    const int t = min(kb * 16 + j, kv_len - 1);
    int krow, vrow;
    if (paged) {
      const int at = EXT && t >= sink ? t - sink + window_first : t;  // _kernel_common.py:162-170
      const int pg = at / ps;
      const int page = p.page_values[pbeg + pg];
      krow = ((page * 2) * p.h_kv + kvh) * ps + (at - pg * ps);  // pages (num_pages, 2, h_kv, page_size, d)
      vrow = krow + p.h_kv * ps;
    } else {
      krow = vrow = (kv_start + t) * p.h_kv + kvh;
    }
    float kf[QS][PIECE];
    half8_t kh[QS];
    const T* krow_ptr = kbase + static_cast<int64_t>(krow) * d;
#pragma unroll
    for (int s = 0; s < QS; ++s) {
      const int f = piece_feature(s);
      if constexpr (HALF) {
        half8_t z = {0, 0, 0, 0, 0, 0, 0, 0};
        kh[s] = piece_inside(s) ? *reinterpret_cast<const half8_t*>(krow_ptr + f) : z;
      } else if (piece_inside(s)) {
        load_run<T, PIECE>(krow_ptr + f, kf[s]);
      } else {
#pragma unroll
        for (int e = 0; e < PIECE; ++e) kf[s][e] = 0.f;
      }
    }
    if (EXT && rotary) {
      const int key_pos = p.k_rope_pos_offset != nullptr ? p.k_rope_pos_offset[b] + t : p.q_rope_position[kv_start + t];
      const float pos = static_cast<float>(key_pos) * p.rope_scale;
#pragma unroll
      for (int s = 0; s < QS / 2; ++s) {
        if (!piece_inside(s)) continue;
        if constexpr (HALF) {
          rotate_pair(kh[s], kh[s + QS / 2], piece_feature(s), d, pos, rope_lds, rope.inverse, rope.halves_differ, rope.magnitude);
        } else {
          rotate_pair<PIECE>(kf[s], kf[s + QS / 2], piece_feature(s), d, pos, rope_lds, rope.inverse, rope.halves_differ,
                             rope.magnitude);
        }
      }
    }
    // V^T operands: features j * KS .. + KS - 1 of the four keys 4 g + m
    float vf[4][KS];
    half_t vh[4][KS];
#pragma unroll
    for (int mm = 0; mm < 4; ++mm) {
      const int vr = __shfl(vrow, 4 * g + mm);
      const T* vrow_ptr = vbase + static_cast<int64_t>(vr) * d + j * KS;
#pragma unroll
      for (int c = 0; c < KS / VP; ++c) {
        const bool inside = j * KS + c * VP < d;
        if constexpr (HALF) {
          typedef half_t run_t __attribute__((ext_vector_type(VP)));
          run_t run;
#pragma unroll
          for (int e = 0; e < VP; ++e) run[e] = 0;
          if (inside) run = *reinterpret_cast<const run_t*>(vrow_ptr + c * VP);
#pragma unroll
          for (int e = 0; e < VP; ++e) vh[mm][c * VP + e] = run[e];
        } else if (inside) {
          load_run<T, VP>(vrow_ptr + c * VP, vf[mm] + c * VP);
        } else {
#pragma unroll
          for (int e = 0; e < VP; ++e) vf[mm][c * VP + e] = 0.f;
        }
      }
    }
    half4_t va[KS];  // fp16 storage: feature block fb of the four keys
    if constexpr (HALF) {
#pragma unroll
      for (int fb = 0; fb < KS; ++fb) {
        half4_t a = {vh[0][fb], vh[1][fb], vh[2][fb], vh[3][fb]};
        va[fb] = a;
      }
    }
    const bool in_tree = tree && kb * 16 + 15 >= tree_start;  // wave-uniform
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < QS; ++s) {
        if constexpr (HALF) {
          acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(kh[s], qh[nb][s], acc, 0, 0, 0);
        } else {
#pragma unroll
          for (int c = 0; c < PIECE; ++c) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[s][c], qf[nb][s][c], acc, 0, 0, 0);
        }
      }
      // acc[r]: key kb * 16 + 4 g + r, query row nb * 16 + j
      float sc[4];
      float mx = kMasked;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int key = kb * 16 + 4 * g + r;
        bool visible = key < limit[nb] && key >= lower[nb];
        if (in_tree && key >= tree_start && key < kv_len) {  // tree_attn.py:48-65
          const int32_t* parent = p.tree_labels + 2 * static_cast<int64_t>(tree_base + key - tree_start);
          visible = visible && child_first[nb] >= parent[0] && child_first[nb] < parent[1];
        }
        sc[r] = visible ? acc[r] * p.scale_log2 : kMasked;
        mx = fmaxf(mx, sc[r]);
      }
      mx = max_xor32(max_xor16(mx));  // over the four lane groups that hold the row's other keys
      const float m_new = fmaxf(m[nb], mx);
      const float alpha = fast_exp2(m[nb] - m_new);
      m[nb] = m_new;
      float pr[4];
      float sum = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        pr[r] = fast_exp2(sc[r] - m_new);
        sum += pr[r];
      }
      lsum[nb] = lsum[nb] * alpha + sum;
#pragma unroll
      for (int fb = 0; fb < KS; ++fb) {
        o[nb][fb] *= alpha;
        if constexpr (HALF) {
          const half4_t ph = {static_cast<half_t>(pr[0]), static_cast<half_t>(pr[1]), static_cast<half_t>(pr[2]),
                              static_cast<half_t>(pr[3])};
          o[nb][fb] = __builtin_amdgcn_mfma_f32_16x16x16f16(va[fb], ph, o[nb][fb], 0, 0, 0);
        } else {
#pragma unroll
          for (int mm = 0; mm < 4; ++mm) o[nb][fb] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[mm][fb], pr[mm], o[nb][fb], 0, 0, 0);
        }
      }
    }
  }
  // the row sums of the four lane groups
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) lsum[nb] = sum_xor32(sum_xor16(lsum[nb]));

  // ---- the four waves' states into wave 0: waves 2, 3 -> 0, 1, then 1 -> 0 --------------------------------
  // o[nb][fb][r] of lane (j, g) is feature (4 g + r) * KS + fb of row nb * 16 + j; the slots in LDS are the lane's own
  auto put = [&](int buf) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
#pragma unroll
      for (int fb = 0; fb < KS; ++fb) store4(o_lds + (buf * ROWS + nb * 16 + j) * DMAX + fb * 16 + 4 * g, o[nb][fb]);
      if (g == 0) {
        ml_lds[(buf * ROWS + nb * 16 + j) * 2 + 0] = m[nb];
        ml_lds[(buf * ROWS + nb * 16 + j) * 2 + 1] = lsum[nb];
      }
    }
  };
  auto take = [&](int buf) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const float m_other = ml_lds[(buf * ROWS + nb * 16 + j) * 2 + 0];
      const float l_other = ml_lds[(buf * ROWS + nb * 16 + j) * 2 + 1];
      const float m_new = fmaxf(m[nb], m_other);
      const float mine = fast_exp2(m[nb] - m_new), theirs = fast_exp2(m_other - m_new);
      m[nb] = m_new;
      lsum[nb] = lsum[nb] * mine + l_other * theirs;
#pragma unroll
      for (int fb = 0; fb < KS; ++fb) {
        const float4_t other = *reinterpret_cast<const float4_t*>(o_lds + (buf * ROWS + nb * 16 + j) * DMAX + fb * 16 + 4 * g);
        o[nb][fb] = o[nb][fb] * mine + other * theirs;
      }
    }
  };
  if (wave >= 2) put(wave - 2);
  __syncthreads();
  if (wave < 2) take(wave);
  __syncthreads();
  if (wave == 1) put(0);
  __syncthreads();
  if (wave != 0) return;
  take(0);

  // ---- wave 0 writes the rows: the result, or this share's partial state -----------------------------------
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int row = r0 + nb * 16 + j;
    if (row >= rows) continue;
    const int64_t out_row = static_cast<int64_t>(q_start + row / group) * p.h_q + kvh * group + row % group;
    const bool any = lsum[nb] > 0.f;
    const float inv = any ? 1.0f / lsum[nb] : 0.f;
    const float s_row = any ? m[nb] + fast_log2(lsum[nb]) : kNoKeys;
    // runs of KS consecutive features: (4 g + r) * KS + fb, fb = 0 .. KS - 1
    if (p.splits == 1) {
      T* dst = static_cast<T*>(p.out) + out_row * d;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int c = 0; c < KS / VP; ++c) {
          const int f = (4 * g + r) * KS + c * VP;
          float run[VP];
#pragma unroll
          for (int e = 0; e < VP; ++e) run[e] = o[nb][c * VP + e][r] * inv;
          if (f < d) store_run<T, VP>(dst + f, run);
        }
      }
      // a row without keys: out = 0 and the state the reference's kernels start from, m = -5e4, d = 1
      if (g == 0) p.lse[out_row] = any ? s_row : kNegInit;
    } else {
      float* dst = p.part_o + (static_cast<int64_t>(split) * p.total_q * p.h_q + out_row) * d;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
#pragma unroll
        for (int c = 0; c < KS / 4; ++c) {
          const int f = (4 * g + r) * KS + c * 4;
          float run[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) run[e] = o[nb][c * 4 + e][r] * inv;
          if (f < d) store_run<float, 4>(dst + f, run);
        }
      }
      if (g == 0) p.part_s[static_cast<int64_t>(split) * p.total_q * p.h_q + out_row] = s_row;
    }
  }
}

// The shares of a split launch: one workgroup of 64 lanes per (query, head) row.
template <typename T>
__global__ __launch_bounds__(64) void generic_merge_kernel(const float* part_o, const float* part_s, T* out, float* lse,
                                                          int64_t rows, int d, int splits) {
  const int64_t row = blockIdx.x;
  float s_max = kNoKeys;
  for (int z = 0; z < splits; ++z) s_max = fmaxf(s_max, part_s[z * rows + row]);
  const bool any = s_max > 0.5f * kNoKeys;
  float total = 0.f;
  for (int z = 0; z < splits; ++z) total += any ? fast_exp2(part_s[z * rows + row] - s_max) : 0.f;
  for (int f = threadIdx.x; f < d; f += 64) {
    float acc = 0.f;
    for (int z = 0; z < splits; ++z) {
      const float w = any ? fast_exp2(part_s[z * rows + row] - s_max) : 0.f;
      acc += w * part_o[(z * rows + row) * d + f];
    }
    out[row * d + f] = static_cast<T>(any ? acc / total : 0.f);
  }
  if (threadIdx.x == 0) lse[row] = any ? s_max + fast_log2(total) : kNegInit;
}

template <typename T, bool EXT>
void launch_attention(const GAttn& p, const InlineRopeTable& rope, int rows_hint, hipStream_t stream) {
  const int group = p.h_q / p.h_kv;
  auto run = [&](auto kernel, int rows_per_tile) {
    const int64_t slots = p.total_q * group / rows_per_tile + p.batch;
    KV_CHECK(slots < (int64_t{1} << 31)) << "too many row tiles for one launch";
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(slots), p.h_kv, p.splits), dim3(256), 0, stream, p, rope);
  };
  const int nb = generic_row_blocks(p.d, rows_hint);
  if (p.d <= 64) {
    if (nb == 2) run(generic_attn_kernel<T, 64, 2, EXT>, 32); else run(generic_attn_kernel<T, 64, 1, EXT>, 16);
  } else if (p.d <= 128) {
    if (nb == 2) run(generic_attn_kernel<T, 128, 2, EXT>, 32); else run(generic_attn_kernel<T, 128, 1, EXT>, 16);
  } else {
    run(generic_attn_kernel<T, 256, 1, EXT>, 16);
  }
  KV_LAUNCH_CHECK();
}

}  // namespace

int generic_attention(const GenericAttention& a, void* stream_) {
  KV_API_BEGIN();
  hipStream_t stream = as_stream(stream_);
  const bool f32 = a.elem_bits == 32;
  KV_CHECK(a.elem_bits == 16 || a.elem_bits == 32) << a.what << ": elem_bits must be 16 or 32";
  KV_CHECK(a.batch >= 0 && a.total_q >= 0 && a.h_q > 0 && a.h_kv > 0 && a.h_q % a.h_kv == 0) << a.what << ": bad shape";
  KV_UNSUPPORTED(a.d <= 0 || a.d > 256 || a.d % (f32 ? 4 : 8) != 0)
      << a.what << ": head_dim " << a.d << " is not built (the generic kernels take multiples of " << (f32 ? 4 : 8)
      << " up to 256)";
  const bool rotary = a.rotary_mode != 0;
  KV_UNSUPPORTED(rotary && a.d % (f32 ? 8 : 16) != 0)
      << a.what << ": RoPE inside the generic kernels needs a head dim that is a multiple of " << (f32 ? 8 : 16) << ", got "
      << a.d << " (an element and its partner half a head away are loaded as whole 16-byte pieces)";
  if (a.batch == 0 || a.total_q == 0) return TVMKV_OK;
  const bool paged = a.pages != nullptr;
  KV_CHECK(a.q && a.out && a.lse) << a.what << ": NULL tensor";
  const bool sliding = paged && a.sliding_window != 0;
  KV_CHECK(a.sliding_window == 0 || paged) << a.what << ": a sliding-window cache is a paged one";
  if (rotary) {
    KV_UNSUPPORTED(paged && a.tree_labels != nullptr)
        << a.what << ": RoPE inside the kernel is not built for token trees over the page pool (the reference's kernel "
        << "asserts the same, tree_attn.py:700-702)";
    KV_CHECK(a.q_rope_position != nullptr) << a.what << ": NULL q_rope_position";
    KV_CHECK(!paged || a.k_rope_pos_offset != nullptr) << a.what << ": NULL k_rope_pos_offset";
  }
  if (paged) {
    KV_CHECK(a.page_indptr && a.page_values && a.last_page_len && a.page_size > 0) << a.what << ": NULL page table or bad page size";
    KV_CHECK(a.num_pages * 2 * a.h_kv * a.page_size < (int64_t{1} << 31)) << a.what << ": the page pool has too many rows for 32-bit row ids";
  } else {
    KV_CHECK(a.k && a.v && a.kv_indptr) << a.what << ": NULL tensor";
  }
  KV_CHECK((a.tree_indptr == nullptr) == (a.tree_labels == nullptr)) << a.what << ": tree_indptr and the labels come together";
  KV_CHECK(a.total_q * a.h_q < (int64_t{1} << 31)) << a.what << ": too many rows for one launch";

  GAttn p{};
  p.q = a.q;
  p.k = a.k;
  p.v = a.v;
  p.pages = a.pages;
  p.q_indptr = a.q_indptr;
  p.kv_indptr = a.kv_indptr;
  p.page_indptr = a.page_indptr;
  p.page_values = a.page_values;
  p.last_page_len = a.last_page_len;
  p.tree_indptr = a.tree_indptr;
  p.tree_labels = a.tree_labels;
  p.out = a.out;
  p.lse = a.lse;
  p.total_q = a.total_q;
  p.batch = a.batch;
  p.h_q = a.h_q;
  p.h_kv = a.h_kv;
  p.d = a.d;
  p.page_size = a.page_size;
  p.causal = a.causal;
  p.scale_log2 = static_cast<float>(a.sm_scale) * kLog2e;
  // length_info of a sliding-window cache: (3, batch) = last page length, window offset, sink size (attn_utils.h:483-495)
  p.window_offset = sliding ? a.last_page_len + a.batch : nullptr;
  p.sink_size = sliding ? a.last_page_len + 2 * static_cast<int64_t>(a.batch) : nullptr;
  p.layer_window = sliding ? a.layer_window : 0;
  p.rotary = rotary ? 1 : 0;
  p.q_rope_position = a.q_rope_position;
  p.k_rope_pos_offset = a.k_rope_pos_offset;
  p.rope_scale = static_cast<float>(a.rope_scale);
  InlineRopeTable rope{};
  if (rotary) {
    const InlineRopeHost table = inline_rope_table(a.rope_scaling, a.d, a.rope_theta);
    for (int i = 0; i < a.d; ++i) rope.v[i] = table.v[i];
    rope.inverse = table.inverse;
    rope.halves_differ = table.halves_differ;
    rope.magnitude = table.magnitude;
  }
  const bool ext = sliding || rotary;
  const int group = a.h_q / a.h_kv;
  const int rows_hint = static_cast<int>(std::min<int64_t>(a.total_q * group / a.batch, 1 << 20));
  // Few row tiles against long page lists: split the keys over workgroups until the chip has ~8 workgroups
  // per compute unit, at least 128 keys (8 blocks) per share on average.  Shapes only: no device read.
  p.splits = 1;
  ScratchLease lease{};
  if (paged) {
    const int rows_per_tile = 16 * generic_row_blocks(a.d, rows_hint);
    const int64_t tiles = (a.total_q * group / rows_per_tile + a.batch) * a.h_kv;
    const int64_t keys_per_seq = a.nnz_pages * a.page_size / a.batch;
    const int64_t want = (f32 ? 8 : 16) * static_cast<int64_t>(compute_units()) / std::max<int64_t>(tiles, 1);
    p.splits = static_cast<int>(std::max<int64_t>(1, std::min<int64_t>({want, keys_per_seq / 128, 64})));
  }
  if (p.splits > 1) {
    const size_t o_bytes = static_cast<size_t>(p.splits) * a.total_q * a.h_q * a.d * sizeof(float);
    const size_t s_bytes = static_cast<size_t>(p.splits) * a.total_q * a.h_q * sizeof(float);
    lease = lease_scratch(kScratchGeneric, stream, o_bytes + s_bytes, 0);  // held until the merge is enqueued
    p.part_o = reinterpret_cast<float*>(lease.ptr);
    p.part_s = reinterpret_cast<float*>(lease.ptr + o_bytes);
  }
  if (f32) {
    if (ext) launch_attention<float, true>(p, rope, rows_hint, stream); else launch_attention<float, false>(p, rope, rows_hint, stream);
  } else {
    if (ext) launch_attention<half_t, true>(p, rope, rows_hint, stream); else launch_attention<half_t, false>(p, rope, rows_hint, stream);
  }
  if (p.splits > 1) {
    const int64_t rows = a.total_q * a.h_q;
    if (f32) {
      hipLaunchKernelGGL(generic_merge_kernel<float>, dim3(static_cast<unsigned>(rows)), dim3(64), 0, stream, p.part_o, p.part_s,
                         static_cast<float*>(a.out), a.lse, rows, a.d, p.splits);
    } else {
      hipLaunchKernelGGL(generic_merge_kernel<half_t>, dim3(static_cast<unsigned>(rows)), dim3(64), 0, stream, p.part_o, p.part_s,
                         static_cast<half_t*>(a.out), a.lse, rows, a.d, p.splits);
    }
    KV_LAUNCH_CHECK();
  }
  KV_API_END();
}

}  // namespace tvmkv
