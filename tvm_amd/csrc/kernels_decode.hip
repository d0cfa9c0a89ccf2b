// Batched paged decode attention for gfx950, written as an HBM-bound streaming kernel.
//
// Replaces batch_decode_paged_kv (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:181-411),
// which walks the whole KV of one (sequence, kv head) in a single block.  Here the KV of a
// sequence is cut into chunks of `chunk_pages` pages; every (chunk, kv head) is one workgroup,
// so a handful of very long sequences still fill 256 CUs, and a second kernel merges the
// per-chunk partial states.  Arithmetic follows the reference: scores scaled by
// sm_scale*log2(e), base-2 online softmax with m = -5e4, d = 1 as the initial state, fp32
// accumulation, output O/d rounded once to fp16, lse = m + log2(d).
//
// One workgroup (4 wavefronts) takes one chunk of one kv head and up to 16 of the query heads that
// share it (a larger GQA group is walked in blocks of 16 heads by neighbouring workgroups, which read
// the same pages); decode_mfma_kernel below describes the data path.  The chunk result goes either
// straight to the output (single-chunk sequence) or to the fp32 partial buffer, and the workgroup
// that delivers the last partial state of a (sequence, kv head, head block) merges them.
//
// Chunk slots without a prologue kernel: sequence b owns slots
//   [floor(page_indptr[b]/CP) + b, floor(page_indptr[b+1]/CP) + b + 1)
// which always holds ceil(npages_b/CP) chunks; a workgroup finds its sequence by binary search
// on page_indptr, so the grid size depends on shapes only (floor(nnz_pages/CP) + B slots).
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "kernels_common.cuh"
#include "runtime_support.h"
#include "typed_kernels.h"
#include "split_plan.h"

namespace tvmkv {

struct DecodeParams {
  const half_t* q;
  const half_t* pages;
  const int32_t* page_indptr;
  const int32_t* page_values;
  const int32_t* last_page_len;
  half_t* output;
  float* lse;
  float* part_o;   // (slots, h_q, D) fp32, unnormalised, relative to part_ml[..][0]
  float* part_ml;  // (slots, h_q, 2) fp32: running max m, running sum l
  // extended form (decode_mfma_kernel<true>): sliding-window cache and inline RoPE
  const int32_t* window_offset;   // (B) physical index of the first token of the window, or NULL
  const int32_t* sink_size;       // (B) attention-sink tokens kept at the front, or NULL
  const int32_t* k_rope_pos_offset;  // (B) position of logical token 0 (inline RoPE)
  const int32_t* q_rope_position;    // (B) position of the query token (inline RoPE)
  int rotary;                     // 1: rotate q and k inside the kernel
  float rope_scale;
  // (batch, h_kv) arrival counters of the fused chunk merge of decode_mfma_kernel, or NULL.  A counter
  // is epoch << 32 | workgroups that have delivered their partial state in the launch with that epoch;
  // a word with an older epoch is what an earlier launch left behind and counts as zero, so nothing
  // has to be reset between launches, not even after one that failed half way.
  unsigned long long* arrivals;
  uint32_t epoch;
  int batch_size;
  int h_q;
  int h_kv;
  int chunk_pages;
  int page_shift;  // pages hold 16 << page_shift tokens; the kernel walks them as runs of 16-token pages
  float scale_log2;  // sm_scale * log2(e)
  // fused step (decode_mfma_kernel<..., FUSED = true>): the launch does the split + RoPE + append of the
  // step's new token itself.  q is read from the fused (B, h_q + 2 h_kv, D) tensor and rotated at
  // q_rope_position[b]; the work items of a sequence's last chunk rotate its new k row, write it and the
  // v row to slot append_slot[b] of the page pool, and then attend to them like to any cached token.
  const half_t* qkv;
  half_t* pages_rw;             // == pages
  const int32_t* append_slot;   // (B) page * page_size + offset, -1 = none
  int apply_rope;               // 0: q and k are used as they come
  // padded head dims (80, 96, 112 on the head dim 128 kernel): elements per row of q, the pages and the
  // output in memory; 0 = the kernel's head dim
  int d_mem;
  // how the entries of the RoPE table are used (InlineRopeTable): position * entry instead of position /
  // entry; separate entries for the two halves of a head; a factor on cos and sin
  int rope_inverse;
  int rope_halves_differ;
  float rope_magnitude;
};

// Same answer as find_sequence, computed by one wavefront as a 64-ary search: the lanes probe
// slot_begin at 64 evenly spaced sequences of the range that is left, and because slot_begin is
// increasing the number of lanes that qualify tells which sixty-fourth holds the answer.  One round
// trip to memory per factor of 64 in the batch size (a linear scan in blocks of 64 sequences cost a
// launch of 2048 sequences up to 32 dependent round trips per work item).
__device__ __forceinline__ int find_sequence_wave(const int32_t* page_indptr, int batch, int cp, int slot,
                                                  int lane) {
  int lo = 0, n = batch;  // the answer lies in [lo, lo + n), and slot_begin(lo) <= slot
  while (n > 64) {
    const int stride = (n + 63) >> 6;
    const int idx = lo + lane * stride;
    const bool le = idx < lo + n && slot_begin(page_indptr, idx, cp) <= slot;
    const int first = lo + (__popcll(__ballot(le)) - 1) * stride;  // lane 0 always qualifies
    n = min(stride, lo + n - first);
    lo = first;
  }
  const bool le = lane < n && slot_begin(page_indptr, lo + lane, cp) <= slot;
  return lo + max(__popcll(__ballot(le)), 1) - 1;
}

// Merge of the per-chunk partial states of one (sequence, query head) row by one wavefront.
// Lane c first fetches (m, l) of chunk c, a wave reduction gives the common maximum and the total
// sum, and every lane keeps the rescale factor of "its" chunk; the second pass streams the partial
// outputs (each lane owns D/64 features) with the factor broadcast by shuffle, loads of several
// chunks in flight at once.
//
// COHERENT: the partial states were written by other workgroups of the SAME kernel, possibly on
// another XCD (each XCD has its own L2): they are written with device-scope stores (write-through)
// and must be read with device-scope loads, which do not hit lines another XCD may have changed.
__device__ __forceinline__ float load_partial(const float* ptr, bool coherent) {
  return coherent ? __hip_atomic_load(ptr, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : *ptr;
}
__device__ __forceinline__ void store_partial(float* ptr, float v) {
  __hip_atomic_store(ptr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// EPL consecutive floats of a partial output, with the widest loads that come as device-scope loads
template <int EPL, bool COHERENT>
__device__ __forceinline__ void load_partial_row(const float* src, float (&dst)[EPL]) {
  if constexpr (!COHERENT) {
#pragma unroll
    for (int e = 0; e < EPL; ++e) dst[e] = src[e];
  } else if constexpr (EPL % 2 == 0) {
#pragma unroll
    for (int e = 0; e < EPL; e += 2) {
      const unsigned long long two = __hip_atomic_load(reinterpret_cast<const unsigned long long*>(src + e), __ATOMIC_RELAXED,
                                                       __HIP_MEMORY_SCOPE_AGENT);
      dst[e] = __uint_as_float(static_cast<unsigned>(two));
      dst[e + 1] = __uint_as_float(static_cast<unsigned>(two >> 32));
    }
  } else {
#pragma unroll
    for (int e = 0; e < EPL; ++e) dst[e] = load_partial(src + e, true);
  }
}

template <int D, bool COHERENT>
__device__ __forceinline__ void merge_row(const DecodeParams& p, int b, int hq, int nchunks, int lane) {
  constexpr int EPL = D / 64;  // features per lane
  const int64_t row = static_cast<int64_t>(b) * p.h_q + hq;
  const int dm = p.d_mem > 0 ? p.d_mem : D;
  half_t* out = p.output + row * dm + lane * EPL;
  const int s0 = slot_begin(p.page_indptr, b, p.chunk_pages);
  float mx = kNegInit, lsum = 0.f;
  float acc[EPL];
#pragma unroll
  for (int e = 0; e < EPL; ++e) acc[e] = 0.f;
  for (int c0 = 0; c0 < nchunks; c0 += 64) {
    const int c = c0 + lane;
    float m_c = kNegInit, l_c = 0.f;
    if (c < nchunks) {
      const float* ml = p.part_ml + (static_cast<int64_t>(s0 + c) * p.h_q + hq) * 2;
      m_c = load_partial(ml, COHERENT);
      l_c = load_partial(ml + 1, COHERENT);
    }
    float mx_new = m_c;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) mx_new = fmaxf(mx_new, __shfl_xor(mx_new, off, 64));
    mx_new = fmaxf(mx_new, mx);
    const float rescale_old = fast_exp2(mx - mx_new);
    const float sc = fast_exp2(m_c - mx_new);
    float lpart = l_c * sc;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) lpart += __shfl_xor(lpart, off, 64);
    lsum = lsum * rescale_old + lpart;
#pragma unroll
    for (int e = 0; e < EPL; ++e) acc[e] *= rescale_old;
    mx = mx_new;
    const int n_here = min(64, nchunks - c0);
    const float* po = p.part_o + (static_cast<int64_t>(s0 + c0) * p.h_q + hq) * D + lane * EPL;
    const int64_t stride = static_cast<int64_t>(p.h_q) * D;
    // The loads of a batch are all issued before the first is used: the merge is a chain of round trips
    // to memory (device-scope loads do not hit in this XCD's L2), and what it costs is their number.
    constexpr int BATCH = 16;  // (32 costs the main loop registers: 166 instead of 136, and 1.2 % of the decode rate)
    for (int k0 = 0; k0 < n_here; k0 += BATCH) {
      float part[BATCH][EPL];
#pragma unroll
      for (int k = 0; k < BATCH; ++k) {
        const float* src = po + min(k0 + k, n_here - 1) * stride;
        load_partial_row<EPL, COHERENT>(src, part[k]);
      }
#pragma unroll
      for (int k = 0; k < BATCH; ++k) {
        const float w = k0 + k < n_here ? __shfl(sc, min(k0 + k, 63), 64) : 0.f;
#pragma unroll
        for (int e = 0; e < EPL; ++e) acc[e] = fmaf(part[k][e], w, acc[e]);
      }
    }
  }
  const float denom = lsum + fast_exp2(kNegInit - mx);
  const float inv = 1.0f / denom;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    if (lane * EPL + e < dm) out[e] = static_cast<half_t>(acc[e] * inv);
  }
  if (lane == 0) p.lse[row] = mx + fast_log2(denom);
}

// The empty-KV answer out = 0, lse = -5e4 (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:129-130,173-176).
template <int D>
__device__ __forceinline__ void empty_row(const DecodeParams& p, int b, int hq, int lane) {
  constexpr int EPL = D / 64;
  const int64_t row = static_cast<int64_t>(b) * p.h_q + hq;
  const int dm = p.d_mem > 0 ? p.d_mem : D;
#pragma unroll
  for (int e = 0; e < EPL; ++e) {
    if (lane * EPL + e < dm) p.output[row * dm + lane * EPL + e] = static_cast<half_t>(0.f);
  }
  if (lane == 0) p.lse[row] = kNegInit;
}

// Stand-alone merge for the kernels that do not merge themselves: one wavefront per (sequence,
// query head), four per block.  Sequences with one chunk were finished by the main kernel.
template <int D>
__global__ __launch_bounds__(256) void decode_merge_kernel(DecodeParams p, int total_rows) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);  // (b, hq) flattened
  if (row >= total_rows) return;
  const int b = row / p.h_q;
  const int hq = row % p.h_q;
  const int npages = p.page_indptr[b + 1] - p.page_indptr[b];
  const int nchunks = (npages + p.chunk_pages - 1) / p.chunk_pages;
  if (nchunks == 1) return;
  if (nchunks == 0) {
    empty_row<D>(p, b, hq, lane);
    return;
  }
  merge_row<D, false>(p, b, hq, nchunks, lane);
}

// ------------------------------------------------------------------------------------------
// The decode kernel, for head dims 64, 128 and 256 and any GQA group.
//
// A vector-ALU formulation spends ~90 instructions per query head and 8 KiB page, which for groups of
// 4-8 query heads is about as much issue time as the page's HBM time.  Here the two contractions
// run on v_mfma_f32_16x16x32_f16 with (a block of 16 of) the query heads of the group on the N axis:
//   S^T[token, head] = K Q^T   -- K fragments come straight from global memory in the MFMA
//                                 A-layout (lane = token row, 16 bytes of features), no staging;
//   O^T[d, head]     = V^T P^T -- the V rows go from global memory straight into a wave-private
//                                 LDS tile (global_load_lds_dwordx4, no registers) and come out
//                                 of it transposed (ds_read_b64_tr_b16), tokens along the
//                                 contraction axis; P stays in registers (the S^T accumulator
//                                 layout is the B-operand layout).
// A wave consumes two pages (32 tokens) per step: 16 KiB of K/V, 16 MFMAs, a handful of vector
// instructions for the softmax.  Per-head state (m, l) is lane-local; the running maximum is
// shared across the four lane groups with two shuffles per step.
// ------------------------------------------------------------------------------------------
constexpr int DM_PS = 16;

// Piece (16 bytes) c of V row r sits at piece position c ^ dm_swizzle(r): the transposing read of
// 32 lanes touches 8 consecutive rows x 32 bytes, which this spreads over the 8 32-byte parts of a
// 256-byte bank line (head dim 128: one row per line) or over the 4 parts of each half of two lines
// (head dim 64: two rows per line, the rows of equal parity share a half).
template <int D>
__device__ __forceinline__ int dm_swizzle(int row) {
  return D >= 128 ? (row & 7) << 1 : ((row >> 1) & 3) << 1;
}

// One entry per element of the head for in-kernel RoPE (the default: theta^(2i/D) for elements i and
// i + D/2), computed on the host with the libm call the CPU kernels use; DecodeParams says how they are used
struct DecodeRopeDivisors {
  float v[256];
};

// EXT = false: plain cache, q and k already rotated (or no RoPE).  EXT = true adds the sliding-window
// cache (length_info (3, B): the page table covers `sink` tokens at the front, evicted tokens up to
// `window_offset`, then the window, python/tvm/relax/frontend/nn/llm/_kernel_common.py:155-170) and
// inline RoPE (q at q_rope_position[b], the key with logical index t at k_rope_pos_offset[b] + t,
// _decode_kernels.py:141-156).  Attention does not depend on the order of the keys, so the pages are
// still walked in physical order; evicted tokens are masked and logical indices only feed RoPE.
// REREAD: the group has several blocks of 16 heads, whose work items read the same K/V rows one after
// the other: those rows are loaded without the streaming hint, so that the L2 keeps them for the next
// head block (64 sequences, 32 query heads on one kv head: 0.077 against 0.083 ms).  Chosen at run
// time inside one kernel, the load flavour cost the single-block case 4 %.
// HB: blocks of 16 query heads per work item (1 or 2).  A group of up to 32 heads is one work item whose K
// fragments and V tile feed the matrix instructions of both blocks, so the K/V rows are fetched once
// (one kv head with 32 query heads: two items that each streamed the rows before); larger groups take
// several such items.
// FUSED (plain cache only): the launch also does the step's split + RoPE + append, see DecodeParams.
// PAD: rows of q, the pages and the output hold p.d_mem (80, 96, 112) elements, fewer than the kernel's
// head dim: the missing q features are zero, K fragments and V pieces beyond the row repeat its last 16
// bytes (finite values that meet zeros, or feed output features that are not stored).
// VARIANT (with EXT): the in-kernel RoPE takes a frequency variant (rope_pair_ex: a table entry per element,
// inverse frequencies, a magnitude).  A kernel of its own: the second set of table entries and the general
// rotation made every extended launch spill (46-143 registers) while they sat in the same kernel.
template <bool EXT, int D, bool REREAD, int HB = 1, bool FUSED = false, bool PAD = false, bool VARIANT = false>
__global__ __launch_bounds__(256, D > 128 ? 1 : ((EXT || HB > 1) ? 2 : 3)) void decode_mfma_kernel(DecodeParams p, int group, int num_items,
                                                             DecodeRopeDivisors div) {
  static_assert(HB == 1 || HB == 2, "head blocks per work item");
  static_assert(!(FUSED && EXT), "the fused step exists for the plain cache");
  static_assert(!PAD || (!EXT && !FUSED), "padded head dims: plain cache, no in-kernel RoPE");
  const int dm = PAD ? p.d_mem : D;  // elements per row in memory
  constexpr int PS = DM_PS;
  constexpr int KS = D / 32;                // k-steps of the score product
  constexpr int DB = D / 16;                // 16-wide output feature blocks
  constexpr int PPR = D / 8;                // 16-byte pieces per row
  constexpr int RPI = 64 / PPR;             // rows one copy instruction covers
  constexpr int DM_VTILE = 2 * PS * D;      // halfs of a wave's V tile: two pages, row-major
  // K fragments by whole 128-byte lines (see the main loop); the head dim 64 kernel with inline RoPE
  // keeps the half-line form, where a feature and its rotation partner lie in one lane
  constexpr bool KLINE = !(EXT && D == 64);
  constexpr int TI = KS / 2;                // K load instructions per 8-token tile (KLINE)
  constexpr int NPAIR = KLINE ? KS / 4 : KS / 2;  // fragment pairs (f, f + D/2) of a K token in one lane
  static_assert(D == 64 || D == 128 || D == 256, "head dim");
  static_assert(DM_VTILE * sizeof(half_t) >= 16 * D * sizeof(float), "the merge buffer aliases the V tile");
  __shared__ __attribute__((aligned(16))) half_t Vt_all[4][DM_VTILE];
  __shared__ float sm_m[4][16];
  __shared__ float sm_l[4][16];
  __shared__ int sm_last;

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int c16 = lane & 15;   // MFMA column (query head in group) / A-row (token) / V feature piece
  const int g4 = lane >> 4;    // lane group 0..3
  const int cp = p.chunk_pages;
  half_t* Vt = Vt_all[wave];
  const int psh = p.page_shift;  // a page of the table is 1 << psh of the 16-token pages the steps consume
  const int64_t head_stride = static_cast<int64_t>(PS << psh) * dm;

  // Persistent workgroups: item = (chunk slot, kv head, block of 16 heads of the group), strided over
  // the grid.  Neighbouring workgroups take the head blocks and kv heads of one slot, i.e. the same pages.
  constexpr int HPI = 16 * HB;  // query heads per work item
  const int head_blocks = (group + HPI - 1) / HPI;
  for (int item = blockIdx.x; item < num_items; item += gridDim.x) {
  const int slot = item / (p.h_kv * head_blocks);
  const int rest = item - slot * (p.h_kv * head_blocks);
  const int kvh = rest / head_blocks;
  const int hb = rest - kvh * head_blocks;
  const int hq0 = kvh * group + hb * HPI;      // first query head of this item
  const int heads = min(HPI, group - hb * HPI);  // and how many
  const int b = find_sequence_wave(p.page_indptr, p.batch_size, cp, slot, lane);
  const int pbeg = p.page_indptr[b];
  const int npages = p.page_indptr[b + 1] - pbeg;
  const int chunk = slot - slot_begin(p.page_indptr, b, cp);
  const int nchunks = (npages + cp - 1) / cp;
  if (chunk >= nchunks) {  // spare slot (uniform over the workgroup)
    if (p.arrivals != nullptr && npages == 0 && chunk == 0) {  // a sequence without pages: nobody else answers for it
      for (int g = wave; g < heads; g += 4) empty_row<D>(p, b, hq0 + g, lane);
    }
    continue;
  }
  const int kv_len = (npages - 1) * (PS << psh) + p.last_page_len[b];  // physical end of the cached tokens
  // the chunk's 16-token pages (chunks are counted in pages of the table; the last one may be partly filled)
  const int page_lo = (chunk * cp) << psh;
  const int page_hi = min(min(chunk * cp + cp, npages) << psh, (kv_len + PS - 1) / PS);
  // physical token t is attended to iff t < sink or win_lo <= t < kv_len
  const int sink = EXT && p.sink_size != nullptr ? p.sink_size[b] : 0;
  const int win_lo = EXT && p.window_offset != nullptr ? p.window_offset[b] : 0;
  // RoPE divisors of the first halves of this lane's K fragment pairs: features i*32 + g4*8 + e, or
  // with KLINE i*64 + (c16&1)*32 + g4*8 + e
  // (and of the second halves, features + D/2, which differ from the first in some frequency variants)
  float divr[8 * (NPAIR > 0 ? NPAIR : 1)], divh[VARIANT ? 8 * (NPAIR > 0 ? NPAIR : 1) : 1];
  float k_pos0 = 0.f;
  if (EXT && p.rotary) {
#pragma unroll
    for (int i = 0; i < 8 * NPAIR; ++i) {
      const int f = KLINE ? (i >> 3) * 64 + (c16 & 1) * 32 + g4 * 8 + (i & 7) : (i >> 3) * 32 + g4 * 8 + (i & 7);
      divr[i] = div.v[f];
      if constexpr (VARIANT) divh[i] = div.v[f + D / 2];
    }
    k_pos0 = static_cast<float>(p.k_rope_pos_offset[b]);
  }

  // The fused step's append: every work item of the sequence's last chunk writes the new token's k row
  // (rotated with the precise sinf / cosf, the arithmetic of fused_rope_kernel) and v row of its kv head
  // to the page slot, waits until the stores have completed and meets the other waves at a barrier.  All
  // K/V loads of this workgroup come after that, through the same vector cache and L2 as the stores; the
  // items of other head blocks of the same kv head write the same bytes.  The loads of the append are
  // issued here, its arithmetic and stores follow the q fragments below, whose loads are in flight beside them.
  const bool appends = FUSED && chunk == nchunks - 1;
  int32_t aslot = -1;
  float app_xl = 0.f, app_xh = 0.f;
  Vec16 app_v = zero16();
  if (appends) {
    aslot = p.append_slot[b];
    const half_t* krow = p.qkv + (static_cast<int64_t>(b) * (p.h_q + 2 * p.h_kv) + p.h_q + kvh) * D;
    if (tid < D / 2) {
      app_xl = static_cast<float>(krow[tid]);
      app_xh = static_cast<float>(krow[tid + D / 2]);
    } else if (tid >= 128 && tid < 128 + D / 8) {
      app_v = ld16(krow + static_cast<int64_t>(p.h_kv) * D + (tid - 128) * 8);
    }
  }

  // The fused step rotates q itself.  A lane needs the angles of its 8 * KS/2 feature pairs, the same
  // for every head and so for the 16 lanes of its group: each lane computes ONE of them (pair
  // (i / 8) * 32 + g4 * 8 + i % 8 for i = c16, and i = 16 + c16 at head dim 256; spare lanes repeat one) and
  // the group shares them through lane shuffles -- a twentieth of the sin / cos work of every lane
  // computing all of its own.
  constexpr int NA = 4 * KS;               // angles a lane needs
  constexpr int PER_LANE = (NA + 15) / 16;  // angles a lane computes (head dim 256: two)
  float rope_sn[PER_LANE], rope_cs[PER_LANE];
  if (FUSED && p.apply_rope) {
    const float q_pos = static_cast<float>(p.q_rope_position[b]) * p.rope_scale;
#pragma unroll
    for (int r = 0; r < PER_LANE; ++r) {
      const int mine = min(r * 16 + c16, NA - 1);
      sincos_reduced(q_pos / div.v[(mine >> 3) * 32 + g4 * 8 + (mine & 7)], rope_sn[r], rope_cs[r]);
    }
  }

  // Q^T fragments (B operand): column = head c16 of block j of the item, contraction slots = 8 features.
  half8_t qf[HB][KS];
#pragma unroll
  for (int j = 0; j < HB; ++j) {
    const bool head_valid = j * 16 + c16 < heads;
    const half_t* qrow = FUSED ? p.qkv + (static_cast<int64_t>(b) * (p.h_q + 2 * p.h_kv) + hq0 + j * 16 + c16) * D + g4 * 8
                               : p.q + (static_cast<int64_t>(b) * p.h_q + hq0 + j * 16 + c16) * dm + g4 * 8;
    Vec16 qv[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qv[ks] = (head_valid && (!PAD || ks * 32 + g4 * 8 < dm)) ? ld16(qrow + ks * 32) : zero16();
    if (FUSED && p.apply_rope) {
      // the arithmetic of rope_pair with the shared angles: fp32, one rounding to fp16
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int i = ks * 8 + e;  // angle i sits in lane i % 16 of this lane's group
          const float cs = __shfl(rope_cs[i / 16], (lane & 48) + (i & 15), 64);
          const float sn = __shfl(rope_sn[i / 16], (lane & 48) + (i & 15), 64);
          const float xl = static_cast<float>(qv[ks].h8[e]);
          const float xh = static_cast<float>(qv[ks + KS / 2].h8[e]);
          qv[ks].h8[e] = static_cast<half_t>(cs * xl + sn * (-xh));
          qv[ks + KS / 2].h8[e] = static_cast<half_t>(cs * xh + sn * xl);
        }
      }
    }
    if (EXT && p.rotary) {
      // feature f < D/2 rotates with f + D/2: k-step ks with ks + KS/2
      const float q_pos = static_cast<float>(p.q_rope_position[b]) * p.rope_scale;
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {
        float qdiv[8], qdivh[VARIANT ? 8 : 1];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          qdiv[e] = div.v[ks * 32 + g4 * 8 + e];
          if constexpr (VARIANT) qdivh[e] = div.v[D / 2 + ks * 32 + g4 * 8 + e];
        }
        if constexpr (VARIANT) {
          rope_pair_ex(qv[ks].h8, qv[ks + KS / 2].h8, q_pos, qdiv, qdivh, p.rope_inverse, p.rope_halves_differ, p.rope_magnitude);
        } else {
          rope_pair(qv[ks].h8, qv[ks + KS / 2].h8, q_pos, qdiv);
        }
      }
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[j][ks] = qv[ks].h8;
  }
  if (appends) {
    if (aslot >= 0) {
      const int page_tokens = PS << psh;
      half_t* kdst = p.pages_rw + (static_cast<int64_t>(aslot / page_tokens) * 2 * p.h_kv + kvh) * head_stride +
                     (aslot % page_tokens) * D;
      half_t* vdst = kdst + static_cast<int64_t>(p.h_kv) * head_stride;
      if (tid < D / 2) {
        if (p.apply_rope) {
          const float freq = static_cast<float>(p.q_rope_position[b]) * p.rope_scale / div.v[tid];
          const float cs = cosf(freq), sn = sinf(freq);
          kdst[tid] = static_cast<half_t>(cs * app_xl + sn * (-app_xh));
          kdst[tid + D / 2] = static_cast<half_t>(cs * app_xh + sn * app_xl);
        } else {
          kdst[tid] = static_cast<half_t>(app_xl);
          kdst[tid + D / 2] = static_cast<half_t>(app_xh);
        }
      } else if (tid >= 128 && tid < 128 + D / 8) {
        st16(vdst + (tid - 128) * 8, app_v);
      }
    }
    wait_vmcnt<0>();
    __syncthreads();
  }
  float4_t o[HB][DB];
#pragma unroll
  for (int j = 0; j < HB; ++j) {
#pragma unroll
    for (int db = 0; db < DB; ++db) o[j][db] = float4_t{0.f, 0.f, 0.f, 0.f};
  }
  float m[HB], lsum[HB];
#pragma unroll
  for (int j = 0; j < HB; ++j) {
    m[j] = kNegInit;
    lsum[j] = 0.f;
  }

  // V^T fragment via the transposing read: lane li of a 16-lane group points at 4 features of token
  // (li >> 2) of the group's 4 tokens and receives feature li of the group's 16 for the 4 tokens
  const uint32_t vt_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)Vt));
  // the 8 contraction slots of lane group g4 are 4 tokens of each page: 4*g4 .. 4*g4+3, or with KLINE
  // 2*g4, 2*g4+1, 8+2*g4, 8+2*g4+1 (the order in which the score product leaves them in a lane)
  const int v_row = KLINE ? ((c16 >> 3) & 1) * 8 + 2 * g4 + ((c16 >> 2) & 1)
                          : 4 * g4 + (c16 >> 2);     // + PS for the second page: same swizzle
  const int v_swz = dm_swizzle<D>(v_row);
  const int v_lane_off = v_row * D + (c16 & 1) * 4;
  const int v_piece = (c16 & 3) >> 1;                // + 2 * feature block

  // One step = pages (pi, pi+1).  K comes straight from global memory in the MFMA A layout, where lane
  // (c16, g4) holds 16 bytes of A-row c16.  Were A-row c16 simply token c16, one load instruction would
  // touch a quarter of 16 rows of 256 bytes, half a 128-byte line each, and partial lines with the
  // streaming hint measured 10-15 % less bandwidth than without it.  KLINE: an instruction covers 8
  // tokens x one whole line.  A-rows 2t and 2t+1 are token t's features [0,32) and [32,64) of that
  // line, so one fragment goes through two MFMAs, one against the q features of the even rows and one
  // against those of the odd rows (the matrix cores are busy 5 % of the time), and token t's score is row 2t of the
  // first plus row 2t+1 of the second, both in one lane.  Whole lines take the streaming hint: 0.1965
  // -> 0.1915 ms on 64 sequences of 1024-8192 tokens; 4 tokens x a whole 256-byte row per instruction
  // (four MFMAs per fragment) measured the same as this.  K through LDS with whole-row copies like V
  // measured slower (two workgroups per CU instead of three).
  // V: copy instructions of 1 KiB each (4 rows of head dim 128, 8 of head dim 64) fill the wave's LDS tile; rows at or past
  // kv_len repeat the last cached row of their page and a missing second page repeats the first
  // (their P is 0, and 0 times cached data is 0, whereas unwritten memory could hold NaN patterns).
  struct Regs {
    Vec16 k[2][KS];
  };
  auto issue = [&](int pi, Regs& r) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int pg = min(pi + h, page_hi - 1);
      const int page = __builtin_amdgcn_readfirstlane(p.page_values[pbeg + (pg >> psh)]);
      const half_t* kbase = p.pages + (static_cast<int64_t>(page) * 2 * p.h_kv + kvh) * head_stride +
                            __builtin_amdgcn_readfirstlane(pg & ((1 << psh) - 1)) * (PS * dm);
      const half_t* vbase = kbase + static_cast<int64_t>(p.h_kv) * head_stride;
      const int last_row = min(PS, kv_len - pg * PS) - 1;  // >= 0: every page of the table holds a token
#pragma unroll
      for (int i = 0; i < PS / RPI; ++i) {
        const int row = i * RPI + lane / PPR;
        int piece = (lane % PPR) ^ dm_swizzle<D>(h * PS + row);
        if (PAD) piece = min(piece, dm / 8 - 1);
        const uint32_t src_off = static_cast<uint32_t>(min(row, last_row) * (dm * 2) + piece * 16);
        const uint32_t dst = vt_lds + (h * PS + i * RPI) * (D * 2);
        if (REREAD) copy16_to_lds(vbase, src_off, dst); else copy16_to_lds_nt(vbase, src_off, dst);
      }
      if (pi + h < page_hi) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          if (KLINE) {  // fragment ks: tile ks / TI (8 tokens), line ks % TI of the row
            const int feature = (ks % TI) * 64 + (c16 & 1) * 32 + g4 * 8;
            const half_t* src = kbase + ((ks / TI) * 8 + (c16 >> 1)) * dm + (PAD ? min(feature, dm - 8) : feature);
            r.k[h][ks] = REREAD ? ld16(src) : ld16_nt(src);
          } else {
            r.k[h][ks] = ld16(kbase + c16 * D + ks * 32 + g4 * 8);
          }
        }
      } else {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) r.k[h][ks] = zero16();
      }
    }
  };

  auto consume = [&](int pi, Regs& r) {
    // wave-uniform: some token of the two pages is not attended to (end of the sequence, evicted)
    const bool partial = EXT ? !((pi * PS >= win_lo && (pi + 2) * PS <= kv_len) || (pi + 2) * PS <= sink)
                             : (pi + 2) * PS > kv_len;
    auto attended = [&](int t) { return EXT ? (t < sink || (t >= win_lo && t < kv_len)) : t < kv_len; };
    if (EXT && p.rotary) {
      // the key of this lane in page h is physical token (pi+h)*PS + c16 (KLINE: + 8*tile + c16/2);
      // logical index = position
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int tile = 0; tile < (KLINE ? 2 : 1); ++tile) {
          const int t = (pi + h) * PS + (KLINE ? tile * 8 + (c16 >> 1) : c16);
          const int logical = t < sink ? t : t - win_lo + sink;
          const float pos = (k_pos0 + static_cast<float>(logical)) * p.rope_scale;
          Vec16* frag = r.k[h] + (KLINE ? tile * TI : 0);
#pragma unroll
          for (int i = 0; i < NPAIR; ++i) {
            if constexpr (VARIANT) {
              rope_pair_ex(frag[i].h8, frag[i + NPAIR].h8, pos, divr + 8 * i, divh + 8 * i, p.rope_inverse, p.rope_halves_differ,
                           p.rope_magnitude);
            } else {
              rope_pair(frag[i].h8, frag[i + NPAIR].h8, pos, divr + 8 * i);
            }
          }
        }
      }
    }
    // ---- S^T = K Q^T for both pages, every head block against the same K fragments --------------
    // s[j][h][e]: head block j, token (pi+h)*PS + token_of(e), head j*16 + c16
    auto token_of = [&](int e) { return KLINE ? 8 * (e >> 1) + 2 * g4 + (e & 1) : 4 * g4 + e; };
    float4_t s[HB][2];
#pragma unroll
    for (int j = 0; j < HB; ++j) {
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        if (KLINE) {
#pragma unroll
          for (int tile = 0; tile < 2; ++tile) {
            float4_t even = float4_t{0.f, 0.f, 0.f, 0.f}, odd = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int i = 0; i < TI; ++i) {
              even = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.k[h][tile * TI + i].h8, qf[j][2 * i], even, 0, 0, 0);
              odd = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.k[h][tile * TI + i].h8, qf[j][2 * i + 1], odd, 0, 0, 0);
            }
            s[j][h][tile * 2 + 0] = even[0] + odd[1];
            s[j][h][tile * 2 + 1] = even[2] + odd[3];
          }
        } else {
          s[j][h] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) s[j][h] = __builtin_amdgcn_mfma_f32_16x16x32_f16(r.k[h][ks].h8, qf[j][ks], s[j][h], 0, 0, 0);
        }
      }
    }
    half8_t pf[HB];
#pragma unroll
    for (int j = 0; j < HB; ++j) {
      float mx = kNegInit;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = s[j][h][e] * p.scale_log2;
          if (partial) v = attended((pi + h) * PS + token_of(e)) ? v : kNegInit;
          s[j][h][e] = v;
          mx = fmaxf(mx, v);
        }
      }
      mx = max_xor32(max_xor16(mx));
      // the reference point moves only when the maximum exceeds it by more than 2^8 (p stays <= 256):
      // after the first steps almost no step rescales O
      const float m_new = mx > m[j] + 8.0f ? mx : m[j];
      const float alpha = fast_exp2(m[j] - m_new);
      m[j] = m_new;
      lsum[j] *= alpha;
      if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.0f))) {
#pragma unroll
        for (int db = 0; db < DB; ++db) o[j][db] *= alpha;
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float pj = fast_exp2(s[j][h][e] - m_new);
          if (partial) pj = attended((pi + h) * PS + token_of(e)) ? pj : 0.f;
          lsum[j] += pj;
          pf[j][h * 4 + e] = static_cast<half_t>(pj);
        }
      }
    }
    // ---- O^T += V^T P^T: contraction slot g4*8 + i <-> page i/4, token token_of(i%4) ----------
    // The tile is written (by the copies) and read by this wave only: the copies are done when
    // vmcnt reaches 0, and the reads below are done before the MFMAs that use them are issued,
    // which is before the next step's copies in program order.
    wait_vmcnt<0>();
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const half_t* vb = Vt + v_lane_off + (((db * 2 + v_piece) ^ v_swz) * 8);
      const half4_t lo = lds_read_tr16(vb);
      const half4_t hi = lds_read_tr16(vb + PS * D);
      half8_t a;
      a[0] = lo[0]; a[1] = lo[1]; a[2] = lo[2]; a[3] = lo[3];
      a[4] = hi[0]; a[5] = hi[1]; a[6] = hi[2]; a[7] = hi[3];
#pragma unroll
      for (int j = 0; j < HB; ++j) o[j][db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pf[j], o[j][db], 0, 0, 0);
    }
  };

  // No software pipelining: three waves per SIMD (twelve per CU, each with 16 KiB of loads in
  // flight while it waits) hide the load latency; four per SIMD measured 4 % slower (more page
  // streams at once than the memory system likes), two about the same.
  Regs ra;
  for (int pi = page_lo + 2 * wave; pi < page_hi; pi += 8) {
    issue(pi, ra);
    consume(pi, ra);
  }

  // ---- merge the 4 waves through LDS, one head block at a time: o[j][db][e] is feature db*16 + 4*g4 + e
  // of head j*16 + c16 (the wave's V tile is dead now and becomes its [16][D] fp32 output buffer) -----
  const bool single_chunk = nchunks == 1;
#pragma unroll
  for (int j = 0; j < HB; ++j) {
    if (j > 0) __syncthreads();  // the previous block's sums have been read
    // the row sums are per lane group: add them up; m is already common
    const float lrow = sum_xor32(sum_xor16(lsum[j]));
    float* sm_o_w = reinterpret_cast<float*>(Vt_all[wave]);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int e = 0; e < 4; ++e) sm_o_w[c16 * D + db * 16 + 4 * g4 + e] = o[j][db][e];
    }
    if (g4 == 0) {
      sm_m[wave][c16] = m[j];
      sm_l[wave][c16] = lrow;
    }
    __syncthreads();
    const int heads_here = min(16, heads - j * 16);
    for (int idx = tid; idx < heads_here * D; idx += 256) {
      const int g = idx / D;
      const int d = idx % D;
      float mx = sm_m[0][g];
#pragma unroll
      for (int w = 1; w < 4; ++w) mx = fmaxf(mx, sm_m[w][g]);
      float lt = 0.f, acc = 0.f;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const float sc = fast_exp2(sm_m[w][g] - mx);
        lt += sm_l[w][g] * sc;
        acc += reinterpret_cast<const float*>(Vt_all[w])[g * D + d] * sc;
      }
      const int hq = hq0 + j * 16 + g;
      if (single_chunk) {
        const float denom = lt + fast_exp2(kNegInit - mx);
        if (!PAD || d < dm) p.output[(static_cast<int64_t>(b) * p.h_q + hq) * dm + d] = static_cast<half_t>(acc / denom);
        if (d == 0) p.lse[static_cast<int64_t>(b) * p.h_q + hq] = mx + fast_log2(denom);
      } else {
        store_partial(p.part_o + (static_cast<int64_t>(slot) * p.h_q + hq) * D + d, acc);
        if (d == 0) {
          store_partial(p.part_ml + (static_cast<int64_t>(slot) * p.h_q + hq) * 2 + 0, mx);
          store_partial(p.part_ml + (static_cast<int64_t>(slot) * p.h_q + hq) * 2 + 1, lt);
        }
      }
    }
  }
  // Fused chunk merge: the workgroup that delivers the last partial state of a (sequence, kv head)
  // merges them all.  No device-scope fences (on this chip they write back and invalidate a whole
  // L2 and made the kernel 2-4 x slower): the partial states are written with device-scope stores,
  // every wave waits until its own have completed, the barrier collects the waves, one thread
  // counts the workgroup in with a device-scope atomic, and the workgroup that completes the count
  // reads the states with device-scope loads.  The counter carries the launch's epoch in its upper
  // half: the maximum brings a word of an older launch (one that was abandoned half way, too) to
  // (epoch, 0) and leaves this launch's alone.
  if (p.arrivals != nullptr && !single_chunk) {
    wait_vmcnt<0>();
    __syncthreads();
    if (tid == 0) {
      unsigned long long* counter = p.arrivals + (static_cast<int64_t>(b) * p.h_kv + kvh) * head_blocks + hb;
      __hip_atomic_fetch_max(counter, static_cast<unsigned long long>(p.epoch) << 32, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      const unsigned long long before =
          __hip_atomic_fetch_add(counter, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      sm_last = static_cast<uint32_t>(before) == static_cast<uint32_t>(nchunks - 1);
      // everyone has arrived: nobody of this launch touches the counter again.  Back to (epoch, 0), so
      // that a launch with the same arguments (a captured graph that is replayed) counts from zero.
      if (sm_last) {
        __hip_atomic_store(counter, static_cast<unsigned long long>(p.epoch) << 32, __ATOMIC_RELAXED,
                           __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    __syncthreads();
    if (sm_last) {
      for (int g = wave; g < heads; g += 4) merge_row<D, true>(p, b, hq0 + g, nchunks, lane);
    }
  }
  __syncthreads();  // the merge buffers are the next item's V tiles
  }  // items
}

constexpr size_t kArrivalBytes = 256 * 1024;  // the first bytes of the scratch buffer: arrival counters

}  // namespace tvmkv

using namespace tvmkv;

// ---- scratch memory of the entry point that allocates nothing --------------------------------
// One array per device that loads this library, held until the process ends: arrival counters, then
// the partial states.  The name below is a host-side handle of the symbol, not a device address:
// host code only ever uses the address hipGetSymbolAddress returns for the current device.
constexpr size_t kStaticScratchBytes = 24u << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

struct StaticScratch {
  char* ptr = nullptr;    // device address of `scratch` on this device
  uint64_t launches = 0;  // the epoch of a launch is the low half
};
static StaticScratch g_static_scratch[64];
static std::mutex g_static_scratch_mutex;

static ScratchLease lease_static_scratch(size_t bytes, hipStream_t stream) {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  KV_CHECK(dev >= 0 && dev < 64) << "device ordinal " << dev << " out of range";
  KV_CHECK(bytes <= kStaticScratchBytes)
      << "batch_decode_paged_kv_noalloc: the call needs " << bytes << " bytes of scratch memory, the built-in "
      << "buffer has " << kStaticScratchBytes << "; use tvmkv_batch_decode_paged_kv for this shape";
  std::unique_lock<std::mutex> lock(g_static_scratch_mutex);
  StaticScratch& s = g_static_scratch[dev];
  if (s.ptr == nullptr) {
    void* ptr = nullptr;
    HIP_CHECK(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    s.ptr = static_cast<char*>(ptr);  // device memory of a loaded code object starts out zeroed
  }
  bool wrapped = false;
  const uint32_t epoch = next_scratch_epoch(&s.launches, &wrapped);
  // 2^32 calls on this device: the epochs start over at 1 from counters cleared by a kernel in stream
  // order (no allocation, no memset node)
  if (wrapped) zero_scratch_counters(s.ptr, kArrivalBytes, stream);
  return ScratchLease{s.ptr, epoch, std::move(lock)};
}

extern "C" int tvmkv_debug_set_scratch_launches(uint64_t launches) {
  KV_API_BEGIN();
  debug_set_scratch_launches(launches);
  std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
  for (auto& s : g_static_scratch) s.launches = launches;
  KV_API_END();
}

// The fused step's extra arguments (qkv == nullptr: a plain decode call)
struct FusedStep {
  const void* qkv = nullptr;
  const int32_t* append_position_map = nullptr;
  int apply_rope = 0;
  const tvmkv_rope_scaling* rope_scaling = nullptr;  // frequency variant of the in-kernel RoPE of a plain call
};

// Body of the decode entry point.  lease(bytes) hands out the scratch memory of the call: arrival
// counters in the first kArrivalBytes, partial states behind them.
template <class Lease>
static void decode_entry(Lease&& lease, const FusedStep& fused_step, const void* q, const void* pages, const int32_t* page_indptr, const int32_t* page_values,
                         const int32_t* length_info, const int32_t* k_rope_pos_offset,
                         const int32_t* q_rope_position, void* output, float* lse, int64_t rotary_mode,
                         double rope_scale, double rope_theta, double sm_scale, int32_t batch_size,
                         int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv, int32_t d,
                         int32_t page_size, int32_t sliding_window, void* stream) {
  KV_CHECK(batch_size >= 0 && nnz_pages >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0)
      << "batch_decode_paged_kv: bad shape";
  const bool ext = rotary_mode != 0 || sliding_window != 0;
  KV_UNSUPPORTED(page_size < 16 || page_size > 128 || (page_size & (page_size - 1)) != 0)
      << "batch_decode_paged_kv: page_size " << page_size << " is not built (16, 32, 64, 128)";
  const bool padded = d == 80 || d == 96 || d == 112;  // run on the head dim 128 kernel, rows of d elements
  KV_UNSUPPORTED(d != 64 && d != 128 && d != 256 && !padded)
      << "batch_decode_paged_kv: head_dim " << d << " is not built (64, 80, 96, 112, 128, 256)";
  KV_UNSUPPORTED(padded && (ext || fused_step.qkv != nullptr))
      << "batch_decode_paged_kv: head_dim " << d << " is built for the plain cache only (no sliding window or inline RoPE)";
  const int dk = padded ? 128 : d;  // the kernel's head dim
  if (batch_size == 0) return;
  const bool fused_launch = fused_step.qkv != nullptr;
  KV_CHECK((q || fused_launch) && pages && page_indptr && length_info && output && lse) << "batch_decode_paged_kv: NULL tensor";
  KV_CHECK(!fused_launch || (!ext && fused_step.append_position_map && q_rope_position))
      << "fused decode step: plain cache only, and it needs the append slots and the positions";
  KV_CHECK(nnz_pages == 0 || page_values) << "batch_decode_paged_kv: NULL page table";
  hipStream_t s = as_stream(stream);

  DecodeParams p;
  p.q = static_cast<const half_t*>(q);
  p.pages = static_cast<const half_t*>(pages);
  p.page_indptr = page_indptr;
  p.page_values = page_values;
  p.last_page_len = length_info;  // row 0 of the (3, B) form
  p.window_offset = sliding_window != 0 ? length_info + batch_size : nullptr;
  p.sink_size = sliding_window != 0 ? length_info + 2 * static_cast<int64_t>(batch_size) : nullptr;
  p.k_rope_pos_offset = k_rope_pos_offset;
  p.q_rope_position = q_rope_position;
  p.rotary = rotary_mode != 0;
  p.rope_scale = static_cast<float>(rope_scale);
  p.output = static_cast<half_t*>(output);
  p.lse = lse;
  p.batch_size = batch_size;
  p.h_q = h_q;
  p.h_kv = h_kv;
  // the kernel walks a page of 16 << page_shift tokens as 1 << page_shift pages of 16: chunks are
  // sized in those and counted in pages of the table
  p.page_shift = 0;
  while ((16 << p.page_shift) < page_size) ++p.page_shift;
  const int group = h_q / h_kv;
  // groups of more than 16 heads: work items of 32 heads (two blocks against the same K/V fragments;
  // head dim 256 keeps items of 16: two blocks of its accumulators do not fit the register file)
  const int heads_per_item = (group > 16 && dk <= 128) ? 32 : 16;
  const int head_blocks = (group + heads_per_item - 1) / heads_per_item;
  const int chunk16 = heads_per_item == 32 ? decode_pick_chunk_pages_wide(nnz_pages << p.page_shift, h_kv, batch_size, head_blocks, 2 * compute_units())
                                           : decode_pick_chunk_pages(nnz_pages << p.page_shift, h_kv, batch_size, d);
  p.chunk_pages = std::max(1, chunk16 >> p.page_shift);
  p.scale_log2 = static_cast<float>(sm_scale) * kLog2e;
  p.qkv = static_cast<const half_t*>(fused_step.qkv);
  p.pages_rw = const_cast<half_t*>(p.pages);
  p.append_slot = fused_step.append_position_map;
  p.apply_rope = fused_step.apply_rope;
  const int64_t slots = nnz_pages / p.chunk_pages + batch_size;
  KV_CHECK(slots < (int64_t{1} << 31)) << "batch_decode_paged_kv: too many chunks";
  const size_t part_o_bytes = static_cast<size_t>(slots) * h_q * dk * sizeof(float);
  p.d_mem = padded ? d : 0;
  p.rope_inverse = p.rope_halves_differ = 0;
  p.rope_magnitude = 1.0f;
  const size_t part_ml_bytes = static_cast<size_t>(slots) * h_q * 2 * sizeof(float);
  const ScratchLease ws = lease(kArrivalBytes + part_o_bytes + part_ml_bytes);
  p.part_o = reinterpret_cast<float*>(ws.ptr + kArrivalBytes);
  p.part_ml = reinterpret_cast<float*>(ws.ptr + kArrivalBytes + part_o_bytes);
  p.arrivals = nullptr;
  p.epoch = ws.epoch;

  const int64_t num_items = slots * h_kv * head_blocks;
  KV_CHECK(num_items < (int64_t{1} << 31)) << "batch_decode_paged_kv: too many work items";
  // One item per workgroup by default (measured a little faster than a resident-size grid
  // striding over the items); the option decode_wgs_per_cu = n caps the grid at n workgroups per CU.
  const int64_t wgs_per_cu = option(kOptDecodeWgsPerCu);
  int64_t grid_x = num_items;
  if (wgs_per_cu > 0) grid_x = std::min<int64_t>(num_items, static_cast<int64_t>(compute_units()) * wgs_per_cu);
  // the chunk merge is done by the last workgroup of each (sequence, kv head, head block) when the
  // arrival counters fit their region; the option decode_separate_merge keeps the second kernel
  // (items of 32 heads leave the merge to the second kernel: the workgroup that arrives last would merge
  // 32 rows, eight per wave one after the other, every load a round trip to memory, while the second
  // kernel gives every row a wave of its own: 32 q / 1 kv heads 0.065 -> 0.053 ms, 64 / 1 0.096 -> 0.074)
  const bool fused = static_cast<size_t>(batch_size) * h_kv * head_blocks * sizeof(unsigned long long) <= kArrivalBytes &&
                     option(kOptDecodeSeparateMerge) == 0 && heads_per_item == 16;
  if (fused) p.arrivals = reinterpret_cast<unsigned long long*>(ws.ptr);
  DecodeRopeDivisors div{};
  if (p.rotary || (fused_launch && p.apply_rope)) {
    KV_CHECK(k_rope_pos_offset || fused_launch) << "batch_decode_paged_kv: inline RoPE needs the position arrays";
    KV_CHECK(q_rope_position) << "batch_decode_paged_kv: inline RoPE needs the position arrays";
    const InlineRopeHost table = inline_rope_table(fused_launch ? nullptr : fused_step.rope_scaling, d, rope_theta);
    for (int i = 0; i < d; ++i) div.v[i] = table.v[i];
    p.rope_inverse = table.inverse;
    p.rope_halves_differ = table.halves_differ;
    p.rope_magnitude = table.magnitude;
  }
  if (padded) {
    auto launch_padded = [&](auto kernel) {
      hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid_x)), dim3(256), 0, s, p, group, static_cast<int>(num_items), div);
    };
    if (head_blocks > 1) {
      launch_padded(decode_mfma_kernel<false, 128, true, 2, false, true>);
    } else if (heads_per_item == 32) {
      launch_padded(decode_mfma_kernel<false, 128, false, 2, false, true>);
    } else {
      launch_padded(decode_mfma_kernel<false, 128, false, 1, false, true>);
    }
  }
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(grid_x)), dim3(256), 0, s, p, group, static_cast<int>(num_items), div);
  };
  // the default frequencies (one divisor per pair, position / divisor) have the kernel without the general rotation
  const bool variant = p.rotary && (p.rope_inverse != 0 || p.rope_halves_differ != 0 || p.rope_magnitude != 1.0f);
  auto launch_d = [&](auto dim) {
    constexpr int kD = decltype(dim)::value;
    constexpr int kWide = kD <= 128 ? 2 : 1;  // head blocks per item for groups of more than 16 heads
    const bool wide = heads_per_item == 32;
    const bool reread = head_blocks > 1;       // several items read the same K/V rows
    if (fused_launch) {
      if (reread) {
        launch(decode_mfma_kernel<false, kD, true, kWide, true>);
      } else if (wide) {
        launch(decode_mfma_kernel<false, kD, false, kWide, true>);
      } else {
        launch(decode_mfma_kernel<false, kD, false, 1, true>);
      }
    } else if (ext && variant) {
      if (reread) {
        launch(decode_mfma_kernel<true, kD, true, kWide, false, false, true>);
      } else if (wide) {
        launch(decode_mfma_kernel<true, kD, false, kWide, false, false, true>);
      } else {
        launch(decode_mfma_kernel<true, kD, false, 1, false, false, true>);
      }
    } else if (reread) {
      if (ext) launch(decode_mfma_kernel<true, kD, true, kWide>); else launch(decode_mfma_kernel<false, kD, true, kWide>);
    } else if (wide) {
      if (ext) launch(decode_mfma_kernel<true, kD, false, kWide>); else launch(decode_mfma_kernel<false, kD, false, kWide>);
    } else {
      if (ext) launch(decode_mfma_kernel<true, kD, false>); else launch(decode_mfma_kernel<false, kD, false>);
    }
  };
  if (padded) {
    // launched above
  } else if (d == 128) {
    launch_d(std::integral_constant<int, 128>{});
  } else if (d == 256) {
    launch_d(std::integral_constant<int, 256>{});
  } else {
    launch_d(std::integral_constant<int, 64>{});
  }
  if (!fused) {
    KV_LAUNCH_CHECK();
    if (dk == 128) {
      hipLaunchKernelGGL(decode_merge_kernel<128>, dim3((batch_size * h_q + 3) / 4), dim3(256), 0, s, p, batch_size * h_q);
    } else if (d == 256) {
      hipLaunchKernelGGL(decode_merge_kernel<256>, dim3((batch_size * h_q + 3) / 4), dim3(256), 0, s, p, batch_size * h_q);
    } else {
      hipLaunchKernelGGL(decode_merge_kernel<64>, dim3((batch_size * h_q + 3) / 4), dim3(256), 0, s, p, batch_size * h_q);
    }
  }
  KV_LAUNCH_CHECK();
}

// Shapes the tuned kernel is not built for (pages other than 16 / 32 / 64 / 128 tokens, other head dims) run on
// the generic matrix-core kernel (sliding-window caches and RoPE inside the kernel included).  Head dims 80 / 96 /
// 112 run on the tuned kernel in its plain form only.
static bool decode_goes_generic(int64_t rotary_mode, int32_t sliding_window, int32_t d, int32_t page_size) {
  const bool plain = rotary_mode == 0 && sliding_window == 0;
  const bool tuned_dim = plain ? tuned_head_dim(d) : (d == 64 || d == 128 || d == 256);
  return !tuned_page_size(page_size) || !tuned_dim;
}
static int decode_generic(const void* q, const void* pages, const int32_t* page_indptr, const int32_t* page_values,
                          const int32_t* length_info, const int32_t* k_rope_pos_offset, const int32_t* q_rope_position,
                          void* output, float* lse, int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                          int32_t batch_size, int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv, int32_t d,
                          int32_t page_size, int32_t sliding_window, const tvmkv_rope_scaling* rope_scaling, void* stream) {
  GenericAttention a;
  a.what = "batch_decode_paged_kv";
  a.sliding_window = sliding_window;
  a.rotary_mode = rotary_mode;
  a.q_rope_position = q_rope_position;
  a.k_rope_pos_offset = k_rope_pos_offset;
  a.rope_scale = rope_scale;
  a.rope_theta = rope_theta;
  a.rope_scaling = rope_scaling;
  a.q = q;
  a.pages = pages;
  a.page_indptr = page_indptr;
  a.page_values = page_values;
  a.last_page_len = length_info;
  a.out = output;
  a.lse = lse;
  a.total_q = batch_size;
  a.nnz_pages = nnz_pages;
  a.num_pages = num_pages;
  a.batch = batch_size;
  a.h_q = h_q;
  a.h_kv = h_kv;
  a.d = d;
  a.page_size = page_size;
  a.sm_scale = sm_scale;
  return generic_attention(a, stream);
}

extern "C" int tvmkv_batch_decode_paged_kv(const void* q, const void* pages, const int32_t* page_indptr,
                                           const int32_t* page_values, const int32_t* length_info,
                                           const int32_t* k_rope_pos_offset, const int32_t* q_rope_position,
                                           void* output, float* lse, int64_t rotary_mode, double rope_scale,
                                           double rope_theta, double sm_scale, int32_t batch_size,
                                           int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                                           int32_t d, int32_t page_size, int32_t sliding_window, void* stream) {
  if (decode_goes_generic(rotary_mode, sliding_window, d, page_size)) {
    return decode_generic(q, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position, output, lse,
                          rotary_mode, rope_scale, rope_theta, sm_scale, batch_size, nnz_pages, num_pages, h_q, h_kv, d,
                          page_size, sliding_window, nullptr, stream);
  }
  KV_API_BEGIN();
  hipStream_t s = as_stream(stream);
  decode_entry([&](size_t bytes) { return lease_scratch(kScratchDecode, s, bytes, kArrivalBytes); }, FusedStep{}, q, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position, output, lse, rotary_mode,
               rope_scale, rope_theta, sm_scale, batch_size, nnz_pages, num_pages, h_q, h_kv, d, page_size,
               sliding_window, stream);
  KV_API_END();
}

// tvmkv_batch_decode_paged_kv with a frequency variant for the in-kernel RoPE (rotary_mode != 0)
extern "C" int tvmkv_batch_decode_paged_kv_scaled(const void* q, const void* pages, const int32_t* page_indptr,
                                                  const int32_t* page_values, const int32_t* length_info,
                                                  const int32_t* k_rope_pos_offset, const int32_t* q_rope_position,
                                                  void* output, float* lse, int64_t rotary_mode, double rope_scale,
                                                  double rope_theta, double sm_scale, int32_t batch_size,
                                                  int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                                                  int32_t d, int32_t page_size, int32_t sliding_window,
                                                  const tvmkv_rope_scaling* rope_scaling, void* stream) {
  if (decode_goes_generic(rotary_mode, sliding_window, d, page_size)) {
    return decode_generic(q, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position, output, lse,
                          rotary_mode, rope_scale, rope_theta, sm_scale, batch_size, nnz_pages, num_pages, h_q, h_kv, d,
                          page_size, sliding_window, rope_scaling, stream);
  }
  KV_API_BEGIN();
  hipStream_t s = as_stream(stream);
  FusedStep plain;
  plain.rope_scaling = rope_scaling;
  decode_entry([&](size_t bytes) { return lease_scratch(kScratchDecode, s, bytes, kArrivalBytes); }, plain, q, pages,
               page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position, output, lse, rotary_mode,
               rope_scale, rope_theta, sm_scale, batch_size, nnz_pages, num_pages, h_q, h_kv, d, page_size,
               sliding_window, stream);
  KV_API_END();
}

// A decode step of one layer in one launch: split of the fused qkv tensor, RoPE of q and of the new k
// row (apply_rope != 0, default frequencies), append of the new k / v rows to slot
// append_position_map[b] and decode attention over the page table, which must already cover the new
// token (the cache reserves before it attends when it appends before attention).
extern "C" int tvmkv_fused_decode_step(const void* qkv, void* pages, const int32_t* page_indptr,
                                       const int32_t* page_values, const int32_t* last_page_len,
                                       const int32_t* q_rope_position, const int32_t* append_position_map,
                                       void* output, float* lse, int64_t apply_rope, double rope_scale,
                                       double rope_theta, double sm_scale, int32_t batch_size, int64_t nnz_pages,
                                       int64_t num_pages, int32_t h_q, int32_t h_kv, int32_t d, int32_t page_size,
                                       void* stream) {
  KV_API_BEGIN();
  hipStream_t s = as_stream(stream);
  KV_CHECK(batch_size == 0 || (qkv && append_position_map && q_rope_position)) << "fused_decode_step: NULL tensor";
  FusedStep step;
  step.qkv = qkv;
  step.append_position_map = append_position_map;
  step.apply_rope = apply_rope != 0;
  decode_entry([&](size_t bytes) { return lease_scratch(kScratchDecode, s, bytes, kArrivalBytes); }, step, nullptr, pages,
               page_indptr, page_values, last_page_len, nullptr, q_rope_position, output, lse, 0, rope_scale, rope_theta,
               sm_scale, batch_size, nnz_pages, num_pages, h_q, h_kv, d, page_size, 0, stream);
  KV_API_END();
}

// The same entry point for callers that must not allocate (code under HIP graph capture, serving
// loops and harnesses that forbid hipMalloc): scratch memory is the built-in per-device array, and a
// call that needs more than it holds is refused.  Every call on a device shares that array, so calls
// that overlap on one device (two streams) race; stream-ordered calls do not.
extern "C" int tvmkv_batch_decode_paged_kv_noalloc(const void* q, const void* pages, const int32_t* page_indptr,
                                                   const int32_t* page_values, const int32_t* length_info,
                                                   const int32_t* k_rope_pos_offset, const int32_t* q_rope_position,
                                                   void* output, float* lse, int64_t rotary_mode, double rope_scale,
                                                   double rope_theta, double sm_scale, int32_t batch_size,
                                                   int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                                                   int32_t d, int32_t page_size, int32_t sliding_window,
                                                   void* stream) {
  KV_API_BEGIN();
  decode_entry([&](size_t bytes) { return lease_static_scratch(bytes, as_stream(stream)); }, FusedStep{}, q, pages, page_indptr, page_values,
               length_info, k_rope_pos_offset, q_rope_position, output, lse, rotary_mode, rope_scale, rope_theta,
               sm_scale, batch_size, nnz_pages, num_pages, h_q, h_kv, d, page_size, sliding_window, stream);
  KV_API_END();
}

// Host view of the split: which chunk size a launch of these shapes uses, how many chunk slots its
// grid has, and which (sequence, chunk) every slot resolves to (-1, -1 for a spare slot).
extern "C" int tvmkv_decode_split_plan(const int32_t* page_indptr_host, int32_t batch_size, int64_t nnz_pages,
                                       int32_t h_kv, int32_t* chunk_pages, int64_t* num_slots, int32_t* slot_seq,
                                       int32_t* slot_chunk, int64_t slot_capacity) {
  KV_API_BEGIN();
  KV_CHECK(page_indptr_host && chunk_pages && num_slots && batch_size > 0 && h_kv > 0 && nnz_pages >= 0)
      << "decode_split_plan: bad argument";
  const int cp = decode_pick_chunk_pages(nnz_pages, h_kv, batch_size);
  const int64_t slots = nnz_pages / cp + batch_size;
  *chunk_pages = cp;
  *num_slots = slots;
  if (slot_seq == nullptr || slot_chunk == nullptr) return TVMKV_OK;
  KV_CHECK(slots <= slot_capacity) << "decode_split_plan: " << slots << " slots, room for " << slot_capacity;
  for (int64_t slot = 0; slot < slots; ++slot) {
    const int b = find_sequence(page_indptr_host, batch_size, cp, static_cast<int>(slot));
    const int npages = page_indptr_host[b + 1] - page_indptr_host[b];
    const int chunk = static_cast<int>(slot) - slot_begin(page_indptr_host, b, cp);
    const int nchunks = (npages + cp - 1) / cp;
    const bool in_use = chunk < nchunks;
    slot_seq[slot] = in_use ? b : -1;
    slot_chunk[slot] = in_use ? chunk : -1;
  }
  KV_API_END();
}
