// Multi-head latent attention over the paged latent cache, on fp16 MFMA tiles for gfx950.
//
// Replaces batch_prefill_paged_kv_mla
// (python/tvm/relax/frontend/nn/llm/_prefill_kernels.py:927-1071): q is the absorbed query
// (d_latent + d_rope features), a cached row holds [latent | k_pe]; the score contracts all
// d_latent + d_rope features, the value is the latent part of the SAME row (:1046-1057), and all
// h_q heads share the single latent "kv head" (group_size = h_q, :929).  The reference runs the
// same kernel for MLA decode (src/runtime/vm/paged_kv_cache.cc:954-956), and so does this one.
// Numerics as in kernels_prefill.hip (base-2 online softmax, m = -5e4, d = 1 initial state).
//
// Tiling: 128 rows (position, head) per workgroup of 4 wavefronts, 32 rows per wave with the query
// on the N axis of v_mfma_f32_32x32x16_f16: O^T of one wave is 512 x 32 fp32 = 256 accumulator
// registers and Q is 144 registers of B-fragments, so a wave has a SIMD's whole register file (one
// workgroup per compute unit) and overlaps its own matrix and vector work.  32-token tiles of cached
// rows are copied from global memory straight into LDS (global_load_lds_dwordx4), four stages; the
// same LDS bytes serve as A-operand of S^T = KV Q^T (ds_read_b128) and of O^T = V^T P^T
// (ds_read_b64_tr_b16, which transposes on the way out of LDS).  Per matrix instruction the LDS
// delivers half as many bytes as with 16-row waves, which were bound by it.
//
// KV split: decode-shaped calls (one token per sequence) have too few row tiles to fill 256 CUs, so
// the KV tiles of the sequences are cut into chunks, one workgroup each, of a common maximum length:
// the smallest one with which the chunks fit the grid.  Every workgroup derives that length and its
// own (sequence, chunk) from the page table alone, with the sequences spread over the lanes (one
// round of loads; mla_split_plan).  A chunk's state leaves the kernel normalised, in fp16, with its
// log-sum-exp in fp32, as whole rows put together in LDS; workgroup ids are mapped to chunk slots so
// that the chunks of a sequence run on one XCD (they share the sequence's q rows in its L2); a second
// kernel merges the states.  (Merging inside the kernel -- the workgroups of a sequence counting
// themselves in and sharing the merge -- was built and measured: the states then have to cross between
// workgroups with device-scope stores and loads, which move 33 + 33 MB at under 4 TB/s while every
// workgroup waits for them, and the step took 102 us against 83 us with the second kernel.)
#include <algorithm>
#include <cstdlib>
#include <type_traits>
#include <utility>

#include "kernels_common.cuh"
#include "runtime_support.h"
#include "split_plan.h"

namespace tvmkv {

constexpr int MLA_BM = 128;
constexpr int MLA_BN = 32;
constexpr int MLA_MIN_CHUNK = 128;  // tokens

struct MlaParams {
  const half_t* q;
  const int32_t* q_indptr;
  const half_t* pages;
  const int32_t* page_indptr;
  const int32_t* page_values;
  const int32_t* last_page_len;
  half_t* output;
  float* lse;
  half_t* part_o;    // (chunk slots, h_q, DV): a chunk's attention output (normalised)
  float* part_lse;   // (chunk slots, h_q): its log-sum-exp, base 2
  int4* slot_plan;   // (chunk slots): {token row of the sequence, chunk, chunks of the sequence, its first slot}, for the merge
  int batch_size;
  int h_q;
  int page_size;
  int page_shift;    // log2(page_size) when it is a power of two, else -1
  int causal;
  int split;         // 1: decode-shaped call, the KV of the sequences is cut into chunks (see mla_split_plan)
  // split launch of a call with several tokens per sequence (a draft to verify, a short chunk): every
  // token is planned as a sequence of its own with one token, batch_size counts the tokens and tokens_of
  // is the number of real sequences behind q_indptr / page_indptr / last_page_len; 0 otherwise
  int tokens_of;
  int token_base;    // with tokens_of > 0: the launch plans tokens token_base .. token_base + batch_size - 1 of the call
  int min_chunk_tiles;  // split: lower bound of the chunk length
  int row_tiles;     // split: row tiles of a one-token sequence, ceil(h_q / MLA_BM)
  float scale_log2;
};

// First row-tile slot of sequence b.  A sequence starts a new tile; when h_q is not a multiple of
// the tile height the rows before it may end inside a tile, and one spare slot per sequence covers
// that.  (With h_q a multiple of the tile height there are no spare slots: in decode-shaped calls
// they would alternate with the real ones and leave half of the XCDs idle.)
__device__ __forceinline__ int mla_tile_slot_begin(const int32_t* q_indptr, int b, int h_q) {
  return static_cast<int>((static_cast<int64_t>(q_indptr[b]) * h_q) / MLA_BM) + (h_q % MLA_BM != 0 ? b : 0);
}

constexpr int MLA_WAVES = 4;    // wavefronts per workgroup, 32 rows each, one per SIMD
constexpr int MLA_STAGES = 4;   // 4 x 36 KiB of LDS: the tile whose V is in use, the one whose K is, two in flight

// LDS image of a tile: DQK/64 column blocks of [MLA_BN rows][64 features] (128-byte rows, 8 pieces
// of 16 bytes).  The same bytes are the A-operand of S^T = KV Q^T (ds_read_b128: lane = key row, one
// piece) and, for the latent part, of O^T = V^T P^T (ds_read_b64_tr_b16: 32 lanes = 4 consecutive
// rows x 64 bytes).  Piece c of row r sits at piece position c ^ mla_swizzle(r).  The LDS serves a
// ds_read_b128 in four passes of 16 lanes, and within each half of the wave the 4-lane blocks
// {0, 3, 5, 6} form one pass and {1, 2, 4, 7} the other (measured: two such blocks on the same banks
// cost a cycle, blocks of different passes do not); the transposing read takes two passes of 32
// consecutive lanes.  With this swizzle the rows of every pass of either read cover all 64 banks.
__device__ __forceinline__ int mla_swizzle(int row) {
  return (((row >> 1) & 1) << 2) | ((row >> 3) & 3);
}

// ---- O in fixed accumulation registers ------------------------------------------------------------
// O^T of a wave is 512 x 32 fp32 = all 256 accumulation registers of the SIMD.  They are addressed by
// number from assembly and never handed to the register allocator (which, asked to keep 16 tuples
// of 16 in that file across a loop that also touches them from the vector ALU, moves them into
// ordinary registers and spills the Q fragments): block db is a[16*db : 16*db+15].  The compiler
// therefore knows nothing of the matrix instructions on them, and the wait states it would insert
// around accumulation-register reads and writes are written out where they are needed.  The file
// must be compiled with -mllvm -amdgpu-spill-vgpr-to-agpr=0 so that no spill lands in these
// registers.
// Every statement that touches them names all 256 as clobbered: a value of the compiler's own can then
// not sit in one across such a statement (under register pressure it parks values there otherwise), and
// check_mla_isa.py verifies on the generated assembly that none does in between either.
#define MLA_ACC_REGS \
  "a0", "a1", "a2", "a3", "a4", "a5", "a6", "a7", "a8", "a9", "a10", "a11", "a12", "a13", "a14", "a15", \
  "a16", "a17", "a18", "a19", "a20", "a21", "a22", "a23", "a24", "a25", "a26", "a27", "a28", "a29", "a30", "a31", \
  "a32", "a33", "a34", "a35", "a36", "a37", "a38", "a39", "a40", "a41", "a42", "a43", "a44", "a45", "a46", "a47", \
  "a48", "a49", "a50", "a51", "a52", "a53", "a54", "a55", "a56", "a57", "a58", "a59", "a60", "a61", "a62", "a63", \
  "a64", "a65", "a66", "a67", "a68", "a69", "a70", "a71", "a72", "a73", "a74", "a75", "a76", "a77", "a78", "a79", \
  "a80", "a81", "a82", "a83", "a84", "a85", "a86", "a87", "a88", "a89", "a90", "a91", "a92", "a93", "a94", "a95", \
  "a96", "a97", "a98", "a99", "a100", "a101", "a102", "a103", "a104", "a105", "a106", "a107", "a108", "a109", "a110", "a111", \
  "a112", "a113", "a114", "a115", "a116", "a117", "a118", "a119", "a120", "a121", "a122", "a123", "a124", "a125", "a126", "a127", \
  "a128", "a129", "a130", "a131", "a132", "a133", "a134", "a135", "a136", "a137", "a138", "a139", "a140", "a141", "a142", "a143", \
  "a144", "a145", "a146", "a147", "a148", "a149", "a150", "a151", "a152", "a153", "a154", "a155", "a156", "a157", "a158", "a159", \
  "a160", "a161", "a162", "a163", "a164", "a165", "a166", "a167", "a168", "a169", "a170", "a171", "a172", "a173", "a174", "a175", \
  "a176", "a177", "a178", "a179", "a180", "a181", "a182", "a183", "a184", "a185", "a186", "a187", "a188", "a189", "a190", "a191", \
  "a192", "a193", "a194", "a195", "a196", "a197", "a198", "a199", "a200", "a201", "a202", "a203", "a204", "a205", "a206", "a207", \
  "a208", "a209", "a210", "a211", "a212", "a213", "a214", "a215", "a216", "a217", "a218", "a219", "a220", "a221", "a222", "a223", \
  "a224", "a225", "a226", "a227", "a228", "a229", "a230", "a231", "a232", "a233", "a234", "a235", "a236", "a237", "a238", "a239", \
  "a240", "a241", "a242", "a243", "a244", "a245", "a246", "a247", "a248", "a249", "a250", "a251", "a252", "a253", "a254", "a255"
template <int R>
__device__ __forceinline__ void acc_mfma_32x32x16(half8_t a, half8_t b) {  // a[R:R+15] += a * b
  asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]" : : "v"(a), "v"(b), "n"(R), "n"(R + 15) : MLA_ACC_REGS);
}
// The same with an order token: `tok` is an operand the instruction does not touch.  Vector work that
// is made to depend on it (pin_after) cannot be scheduled before this matrix instruction, and a
// matrix instruction whose token depends on that work's result cannot be scheduled before the work:
// program order then alternates matrix and vector instructions, which a single wave needs in order
// to use both pipes at once (it issues in order).
template <int R>
__device__ __forceinline__ void acc_mfma_32x32x16(half8_t a, half8_t b, float& tok) {
  asm volatile("v_mfma_f32_32x32x16_f16 a[%3:%4], %1, %2, a[%3:%4]" : "+v"(tok) : "v"(a), "v"(b), "n"(R), "n"(R + 15) : MLA_ACC_REGS);
}
__device__ __forceinline__ void pin_after(float& x, float on) { asm("" : "+v"(x) : "v"(on)); }  // no instruction

template <int R>
__device__ __forceinline__ void acc_zero() {
  asm volatile("v_accvgpr_write_b32 a[%0], 0" : : "n"(R) : MLA_ACC_REGS);
}
template <int R>
__device__ __forceinline__ float acc_read() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(R) : MLA_ACC_REGS);
  return x;
}
template <int R>
__device__ __forceinline__ void acc_scale(float factor) {
  float t;
  asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_mul_f32 %0, %0, %1\n\tv_accvgpr_write_b32 a[%2], %0"
               : "=&v"(t) : "v"(factor), "n"(R) : MLA_ACC_REGS);
}
// wait states between the last matrix instruction that writes an accumulation register and a vector
// instruction that reads it (or the reverse), more than any case needs
__device__ __forceinline__ void acc_settle() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

template <class F, int... I>
__device__ __forceinline__ void static_for_impl(F&& f, std::integer_sequence<int, I...>) {
  (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class F>
__device__ __forceinline__ void static_for(F&& f) {  // f(integral_constant<int, 0>) ... f(integral_constant<int, N-1>)
  static_for_impl(f, std::make_integer_sequence<int, N>{});
}

// ---- the split of a decode-shaped call ---------------------------------------------------------------
constexpr int MLA_MAX_SPLIT_BATCH = 128;  // two sequences per lane

// What a lane knows of the two sequences it looks after (lane and lane + 64).
struct MlaSeqInfo {
  int q_start, qo_len, pbeg, npages, kv_len;
  int cost;  // KV tiles a split launch has to walk: 0 for a sequence that is empty or not a decode step
};
__device__ __forceinline__ MlaSeqInfo mla_seq_info(const MlaParams& p, int b) {
  MlaSeqInfo s{0, 0, 0, 0, 0, 0};
  if (b < p.batch_size && p.tokens_of > 0) {
    // token b of the call as a one-token sequence: under the causal mask token j of n sees the first
    // L - n + j + 1 of its sequence's L keys (python/tvm/relax/frontend/nn/llm/_kernel_common.py:130-135),
    // which is plain attention over that many keys
    const int token = p.token_base + b;
    int lo = 0, hi = p.tokens_of - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (p.q_indptr[mid] <= token) {
        lo = mid;
      } else {
        hi = mid - 1;
      }
    }
    const int first = p.q_indptr[lo];
    const int n = p.q_indptr[lo + 1] - first;
    const int npages = p.page_indptr[lo + 1] - p.page_indptr[lo];
    const int len = npages > 0 ? (npages - 1) * p.page_size + p.last_page_len[lo] : 0;
    s.q_start = token;
    s.qo_len = 1;
    s.pbeg = p.page_indptr[lo];
    s.kv_len = p.causal ? max(0, min(len, len - n + (token - first) + 1)) : len;
    s.npages = (s.kv_len + p.page_size - 1) / p.page_size;
    s.cost = (s.kv_len + MLA_BN - 1) / MLA_BN;
  } else if (b < p.batch_size) {
    s.q_start = p.q_indptr[b];
    s.qo_len = p.q_indptr[b + 1] - s.q_start;
    s.pbeg = p.page_indptr[b];
    s.npages = p.page_indptr[b + 1] - s.pbeg;
    s.kv_len = s.npages > 0 ? (s.npages - 1) * p.page_size + p.last_page_len[b] : 0;
    s.cost = s.qo_len == 1 ? (s.kv_len + MLA_BN - 1) / MLA_BN : 0;
  }
  return s;
}
// ceil(a / c) for 0 <= a < 2^22, c >= 1, rc = 1.0f / c: the float product is off by less than one
__device__ __forceinline__ int mla_ceil_div(int a, int c, float rc) {
  const int x = a + c - 1;
  int q = static_cast<int>(static_cast<float>(x) * rc);
  const int r = x - q * c;
  q += r >= c ? 1 : 0;
  q -= r < 0 ? 1 : 0;
  return q;
}
__device__ __forceinline__ int mla_lane_value(int v0, int v1, int b) {  // b is the same in every lane
  return b < 64 ? __builtin_amdgcn_readlane(v0, b) : __builtin_amdgcn_readlane(v1, b - 64);
}

struct MlaSplit {
  int b, chunk, nchunks;  // nchunks == 0: the slot is not in use
  int first;              // first chunk slot of the sequence
};
// Sum over the wave of small non-negative integers (exact: the total stays below 2^24).
__device__ __forceinline__ int mla_wave_sum(int x) {
  const uint32_t rows = __float_as_uint(group_sum<16>(static_cast<float>(x)));  // every lane: the sum of its row of 16
  return static_cast<int>(__uint_as_float(__builtin_amdgcn_readlane(rows, 0)) + __uint_as_float(__builtin_amdgcn_readlane(rows, 16)) +
                          __uint_as_float(__builtin_amdgcn_readlane(rows, 32)) + __uint_as_float(__builtin_amdgcn_readlane(rows, 48)));
}
// Chunk slots: sequence b gets n_b = max(1, ceil(cost_b / c)) consecutive slots, c being the smallest
// chunk length (in tiles, at least p.min_chunk_tiles) for which all of them fit into `slots`; its tiles
// are divided evenly among its n_b chunks.  The total cost T bounds c from both sides, ceil(T / slots) <= c
// <= ceil(T / (slots - batch)), and a bisection of that (narrow) range finds it, every lane working out the
// chunks of its own two sequences.  Integer arithmetic on values every workgroup reads alike: all
// workgroups, and the merge kernel, arrive at the same plan.
__device__ __forceinline__ MlaSplit mla_split_plan(const MlaParams& p, const MlaSeqInfo& s0, const MlaSeqInfo& s1,
                                                   int slots, int cslot, int lane) {
  const int batch = p.batch_size;
  const bool have0 = lane < batch, have1 = lane + 64 < batch;
  int n0 = 0, n1 = 0;
  auto chunks_with = [&](int c) {
    const float rc = 1.0f / static_cast<float>(c);
    n0 = have0 ? max(1, mla_ceil_div(s0.cost, c, rc)) : 0;
    n1 = have1 ? max(1, mla_ceil_div(s1.cost, c, rc)) : 0;
    return mla_wave_sum(n0 + n1);
  };
  const int total = mla_wave_sum(s0.cost + s1.cost);
  int lo = max(p.min_chunk_tiles, (total + slots - 1) / slots);
  int hi = max(lo, (total + (slots - batch) - 1) / (slots - batch));  // fits: at most total / hi + batch chunks
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (chunks_with(mid) <= slots) {
      hi = mid;
    } else {
      lo = mid + 1;
    }
  }
  chunks_with(hi);
  int first = 0;
  for (int b = 0; b < batch; ++b) {
    const int n = mla_lane_value(n0, n1, b);
    if (cslot < first + n) return MlaSplit{b, cslot - first, n, first};
    first += n;
  }
  return MlaSplit{0, 0, 0, 0};
}

// Merge of the chunk states of heads [h_lo, h_hi) of a one-token sequence: out = sum_c w_c O_c / sum_c w_c
// with w_c = 2^(lse_c - max lse), the arithmetic of merge_state_inplace (_decode_kernels.py:441-450) over
// all chunks, CB at a time with a running maximum.  A wave takes four heads at once, 16 lanes and 32
// features per lane each, and every lane works out the weights of its head for itself: no exchange
// between lanes, and the loads of CB chunks (CB log-sum-exps and 4 CB x 16 bytes per lane) are in
// flight together -- the merge is a chain of memory round trips and nothing else.
template <int DV, int CB>
__device__ __forceinline__ void mla_merge_heads(const MlaParams& p, int q_row, int first, int nchunks, int h_lo, int h_hi,
                                                int wave, int waves, int lane) {
  static_assert(DV == 512, "16 lanes x 32 features");
  const int sub = lane >> 4;   // which of the wave's four heads
  const int part = lane & 15;  // features part*32 .. +31
  // Few heads mean many chunks (a block merges h_q / nchunks heads): then a wave takes one head and its
  // four lane groups share the head's chunks, 4 CB of them in flight, and fold their states at the end.
  const bool share = h_hi - h_lo <= waves;
  const int heads_per_wave = share ? 1 : 4;
  const int cstep = share ? 4 : 1, cfirst = share ? sub : 0;
  for (int h0 = h_lo; h0 < h_hi; h0 += waves * heads_per_wave) {
    const int h = share ? h0 + wave : h0 + wave * 4 + sub;
    const bool valid = h < h_hi;
    const int hh = valid ? h : h_lo;  // lanes without a head repeat a valid one and drop the result
    float acc[32];
#pragma unroll
    for (int e = 0; e < 32; ++e) acc[e] = 0.f;
    float top = -3.0e38f, wsum = 0.f;
    for (int c0 = cfirst; c0 < nchunks; c0 += CB * cstep) {
      float lse_c[CB];
      half8_t o_c[CB][4];
#pragma unroll
      for (int k = 0; k < CB; ++k) {
        const int c = min(c0 + k * cstep, nchunks - 1);  // past the end: the last chunk again, with weight 0
        const int64_t row = static_cast<int64_t>(first + c) * p.h_q + hh;
        lse_c[k] = p.part_lse[row];
#pragma unroll
        for (int j = 0; j < 4; ++j) o_c[k][j] = *reinterpret_cast<const half8_t*>(p.part_o + row * DV + part * 32 + j * 8);
      }
      float block_top = top;
#pragma unroll
      for (int k = 0; k < CB; ++k) block_top = fmaxf(block_top, c0 + k * cstep < nchunks ? lse_c[k] : -3.0e38f);
      const float keep = fast_exp2(top - block_top);  // 0 in the first round
      top = block_top;
      wsum *= keep;
#pragma unroll
      for (int e = 0; e < 32; ++e) acc[e] *= keep;
#pragma unroll
      for (int k = 0; k < CB; ++k) {
        const float w = c0 + k * cstep < nchunks ? fast_exp2(lse_c[k] - top) : 0.f;
        wsum += w;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[j * 8 + e] = fmaf(static_cast<float>(o_c[k][j][e]), w, acc[j * 8 + e]);
        }
      }
    }
    if (share) {  // (wave-uniform) fold the states of the four lane groups; a group without chunks has weight 0
      float top_all = fmaxf(top, __shfl_xor(top, 16, 64));
      top_all = fmaxf(top_all, __shfl_xor(top_all, 32, 64));
      const float keep = fast_exp2(top - top_all);
      top = top_all;
      wsum *= keep;
      wsum += __shfl_xor(wsum, 16, 64);
      wsum += __shfl_xor(wsum, 32, 64);
#pragma unroll
      for (int e = 0; e < 32; ++e) {
        float a = acc[e] * keep;
        a += __shfl_xor(a, 16, 64);
        a += __shfl_xor(a, 32, 64);
        acc[e] = a;
      }
    }
    if (valid && (!share || sub == 0)) {
      const float inv = 1.0f / wsum;  // the chunk that holds the maximum weighs 1
      const int64_t grow = static_cast<int64_t>(q_row) * p.h_q + h;
      half_t* out = p.output + grow * DV + part * 32;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        half8_t out8;
#pragma unroll
        for (int e = 0; e < 8; ++e) out8[e] = static_cast<half_t>(acc[j * 8 + e] * inv);
        *reinterpret_cast<half8_t*>(out + j * 8) = out8;
      }
      if (part == 0) p.lse[grow] = top + fast_log2(wsum);
    }
  }
}

// POW2: the page size is a power of two (p.page_shift), so that a token's page and slot are a shift
// and a mask; the general form divides, per copy instruction, and costs about as much again as the
// matrix work of a tile.
template <int DQK, int DV, bool POW2>
__global__ __launch_bounds__(MLA_WAVES * 64, 1) void mla_paged_kernel(MlaParams p) {
  constexpr int BN = MLA_BN;
  static_assert(BN == 32 && MLA_BM == MLA_WAVES * 32 && DQK % 64 == 0 && DV % 64 == 0 && DV <= DQK, "tile shape");
  constexpr int KS = DQK / 16;               // k-steps of the score product (v_mfma_f32_32x32x16_f16)
  constexpr int DB = DV / 32;                // 32-wide output feature blocks
  constexpr int NBLK = DQK / 64;             // column blocks of a tile
  constexpr int BLK = BN * 64;               // halfs per column block
  constexpr int STAGE = NBLK * BLK;          // halfs per stage
  constexpr int NSTAGE = MLA_STAGES;
  constexpr int NCOPY = NBLK * (BN / 8);     // copy instructions (8 rows x 128 B) per tile
  static_assert(NCOPY % MLA_WAVES == 0 && NSTAGE == 4, "copy split / pipeline depth");
  constexpr int COPIES = NCOPY / MLA_WAVES;  // per wave and tile

  extern __shared__ __attribute__((aligned(16))) half_t lds_tiles[];
  // (no static LDS beside it: the fragment addressing XORs address bits and needs the stages at offset 0)
  asm volatile("" ::: "a0", "a255");  // the kernel uses every accumulation register (by number, see above)

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // a scalar: the bounds derived from it steer wave-uniform branches
  const int h_q = p.h_q;

  // Work item.  Normal mode: a row-tile slot.  Split mode: (chunk slot, row tile of a one-token
  // sequence), the grid holding exactly the items in use: a workgroup takes a whole compute unit
  // (LDS, registers) and runs long, and workgroups that only find out they have nothing to do
  // still disturb the placement of the others.
  int b, r0, chunk = 0, nchunks = 1, cslot = 0, row_step = 0, first_slot = 0;
  int q_start, qo_len, pbeg, npages, kv_len;
  if (p.split) {
    // Workgroup ids go round the XCDs; chunk slots are numbered so that consecutive ones -- the chunks
    // of a sequence -- land on one XCD.
    const int slots = gridDim.x / p.row_tiles;
    const int wg = blockIdx.x / p.row_tiles;
    cslot = slots % 8 == 0 ? (wg % 8) * (slots / 8) + wg / 8 : wg;
    r0 = (blockIdx.x - wg * p.row_tiles) * MLA_BM;
    row_step = p.row_tiles * MLA_BM;
    const int plan_lane = tid & 63;
    const MlaSeqInfo s0 = mla_seq_info(p, plan_lane), s1 = mla_seq_info(p, plan_lane + 64);
    const MlaSplit plan = mla_split_plan(p, s0, s1, slots, cslot, plan_lane);
    if (tid == 0 && r0 == 0) {  // what the merge kernel needs to know of this slot (nchunks <= 1: nothing to merge)
      p.slot_plan[cslot] = make_int4(mla_lane_value(s0.q_start, s1.q_start, plan.b), plan.chunk, plan.nchunks, plan.first);
    }
    if (plan.nchunks == 0) return;  // a slot the plan does not use
    b = plan.b;
    chunk = plan.chunk;
    nchunks = plan.nchunks;
    first_slot = plan.first;
    q_start = mla_lane_value(s0.q_start, s1.q_start, b);
    qo_len = mla_lane_value(s0.qo_len, s1.qo_len, b);
    pbeg = mla_lane_value(s0.pbeg, s1.pbeg, b);
    npages = mla_lane_value(s0.npages, s1.npages, b);
    kv_len = mla_lane_value(s0.kv_len, s1.kv_len, b);
  } else {
    const int slot = blockIdx.x;
    int lo = 0, hi = p.batch_size - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (mla_tile_slot_begin(p.q_indptr, mid, h_q) <= slot) {
        lo = mid;
      } else {
        hi = mid - 1;
      }
    }
    b = lo;
    r0 = (slot - mla_tile_slot_begin(p.q_indptr, b, h_q)) * MLA_BM;
    q_start = p.q_indptr[b];
    qo_len = p.q_indptr[b + 1] - q_start;
    pbeg = p.page_indptr[b];
    npages = p.page_indptr[b + 1] - pbeg;
    kv_len = npages > 0 ? (npages - 1) * p.page_size + p.last_page_len[b] : 0;
  }
  const int rows = qo_len * h_q;
  // (a sequence of a split call that is not a decode step is one chunk: its workgroup walks all its row tiles)
  if (!p.split) {
    // a sequence's row tiles from the last to the first: under the causal mask the last rows see the most
    // keys, and the workgroups that start last decide when the kernel ends
    const int tiles = (rows + MLA_BM - 1) / MLA_BM;
    const int local = r0 / MLA_BM;
    if (local < tiles) r0 = (tiles - 1 - local) * MLA_BM;
  }

  const int ps = p.page_size;

  // normal mode: one pass; split mode: one pass per row tile this workgroup owns (one, for a decode step)
  for (; r0 < rows; r0 += row_step) {
  // Everything that depends on the lane is derived inside the pass from a value the compiler
  // cannot see through: hoisted out of this (rarely taken) loop, the per-lane addresses would stay
  // live across the epilogue, be spilled there, and be reloaded in the tile loop.
  int lane = tid & 63;
  asm volatile("" : "+v"(lane));
  const int col = lane & 31;   // query row of the wave (MFMA column) / key row of an A-fragment
  const int half = lane >> 5;  // contraction slots 8*half .. 8*half+7
  const int my_row = r0 + wave * 32 + col;
  const bool row_valid = my_row < rows;
  const int my_pos = my_row / h_q;
  const int my_head = my_row % h_q;
  const int causal_shift = kv_len - qo_len + 1;
  const int my_limit = row_valid ? (p.causal ? min(kv_len, causal_shift + my_pos) : kv_len) : 0;
  const int last_row_wg = min(rows, r0 + MLA_BM) - 1;
  const int kv_end = p.causal ? max(0, min(kv_len, causal_shift + last_row_wg / h_q)) : kv_len;
  const int first_row_wave = r0 + wave * 32;
  const int last_row_wave = min(rows, first_row_wave + 32) - 1;
  const bool wave_active = first_row_wave < rows;
  const int wave_limit_max = !wave_active ? 0 : (p.causal ? min(kv_len, causal_shift + last_row_wave / h_q) : kv_len);
  const int wave_limit_min = !wave_active ? 0 : (p.causal ? min(kv_len, causal_shift + first_row_wave / h_q) : kv_len);

  // tiles of this chunk: an even split of all tiles of the sequence, clipped by the causal bound
  const int tiles_all = (kv_len + BN - 1) / BN;
  const int tile_lo = static_cast<int>(static_cast<int64_t>(chunk) * tiles_all / nchunks);
  const int tile_hi = min(static_cast<int>(static_cast<int64_t>(chunk + 1) * tiles_all / nchunks), (kv_end + BN - 1) / BN);

  // The page ids of the first tiles are asked for ahead of the query rows: the first copies wait for them,
  // and a wait for a load is a wait for every load issued before it.
  const int last_tok = kv_len - 1;
  int page_ids = 0;
  auto load_page_ids = [&](int tile) {  // of 16 consecutive tiles (4 row groups each), lane = 4*tile + row group
    const int t = min((tile + (lane >> 2)) * BN + (lane & 3) * 8, last_tok);
    page_ids = p.page_values[pbeg + (POW2 ? t >> p.page_shift : t / ps)];
  };
  if (tile_lo < tile_hi) load_page_ids(tile_lo);
  __builtin_amdgcn_sched_barrier(0);
  // Q^T fragments (B operand): column = query col, contraction slots = features ks*16 + half*8 .. +7;
  // filled below, through LDS
  half8_t qf[KS];
  // O^T accumulators: register 16*db + j is feature db*32 + (j/4)*8 + half*4 + j%4 of query col
  static_assert(DB * 16 == 256, "O fills the accumulation registers");
  static_for<DB * 16>([&](auto r) { acc_zero<decltype(r)::value>(); });
  float m = kNegInit, lsum = 0.f;

  // ---- tile copy: global -> LDS -------------------------------------------------------------
  // Copy instruction n of a tile (n = 0 .. NCOPY-1, COPIES consecutive ones per wave) moves rows
  // 8*(n%4) .. +7 of column block n/4.  Rows past the end of the sequence repeat its last token
  // (masked scores; P = 0 times a finite value).  The page ids of 16 consecutive tiles (4 row
  // groups each) are fetched by one vector load, lane = 4*tile + row group: the wait for that load
  // also waits for every copy in flight, so it must be rare.
  const int copy_first = wave * COPIES;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)lds_tiles));
  // Per-lane part of a copy's source offset for rows that need no clamping: row lane/8 of the
  // 8-row group rg, piece (lane%8) ^ swizzle(rg*8 + lane/8) = this value ^ (rg << 4).
  const uint32_t copy_lane_off = (lane >> 3) * (DQK * 2) + (((lane & 7) ^ ((((lane >> 3) >> 1) & 1) << 2)) << 4);
  // General form of a tile's copies: a page id per 8-row group, rows past the end clamped.
  auto issue_tile = [&](int tile) {
    const int w = tile - tile_lo;
    if (w != 0 && (w & 15) == 0) load_page_ids(tile);  // the wait for it also waits for every copy in flight: rare
    const int kv0 = tile * BN;
    const uint32_t stage = lds_base + (w % NSTAGE) * (STAGE * 2);
#pragma unroll
    for (int j = 0; j < COPIES; ++j) {
      const int n = copy_first + j;
      const int blk = n >> 2;
      const int rg = n & 3;
      const int page = __builtin_amdgcn_readlane(page_ids, (w & 15) * 4 + rg);
      const half_t* base = p.pages + static_cast<int64_t>(page) * ps * DQK;
      const int row = rg * 8 + (lane >> 3);
      const int piece = (lane & 7) ^ mla_swizzle(row);
      const uint32_t t = min(kv0 + row, last_tok);
      const uint32_t off = (POW2 ? t & (ps - 1) : t % ps) * (DQK * 2) + (blk * 64 + piece * 8) * 2;
      copy16_to_lds(base, off, stage + (blk * BLK + rg * 8 * 64) * 2);
    }
  };
  // Fast form, for a tile that lies inside one page (pages of 32 tokens or more) and inside the
  // sequence: one scalar base per tile, and a copy is two vector and a few scalar instructions,
  // which fit beside one matrix instruction of the score product.
  const bool tile_in_page = POW2 && ps >= BN;
  const half_t* tile_base = p.pages;
  uint32_t tile_stage = lds_base;
  uint32_t tile_lane_off = 0;
  auto fast_copy_prepare = [&](int tile) {
    // a copy of the per-lane offset that the compiler cannot see through: the nine offsets derived
    // from it are then computed where they are used instead of being kept in nine registers
    tile_lane_off = copy_lane_off;
    asm volatile("" : "+v"(tile_lane_off));
    const int w = tile - tile_lo;
    if ((w & 15) == 0) load_page_ids(tile);
    const int page = __builtin_amdgcn_readlane(page_ids, (w & 15) * 4);
    tile_base = p.pages + (static_cast<int64_t>(page) * ps + ((tile * BN) & (ps - 1))) * DQK;
    tile_stage = lds_base + (w % NSTAGE) * (STAGE * 2);
  };
  auto fast_copy_step = [&](auto jc) {  // copy instruction j (of COPIES) of this wave
    constexpr int j = decltype(jc)::value;
    const int n = copy_first + j;
    const int blk = n >> 2;
    const int rg = n & 3;
    copy16_to_lds(tile_base, (tile_lane_off ^ (rg << 4)) + (rg * 8 * DQK + blk * 64) * 2, tile_stage + (blk * BLK + rg * 8 * 64) * 2);
  };

  // ---- per-lane fragment addressing (LDS byte addresses) -------------------------------------------
  // A fragment's 16-byte piece sits at (logical piece ^ swizzle of its row); the logical piece is a
  // lane part XOR a part known at compile time, and every other term of the address is a multiple
  // of the 128-byte row.  So each product keeps ONE per-lane offset, adds the stage's base once per
  // tile, and reaches every fragment with an XOR of bits 4..6 and an immediate offset (registers
  // are what this kernel is short of).
  // K A-fragment of k-step ks: key row col, features ks*16 + half*8 .. +7: column block ks/4,
  // logical piece (ks%4)*2 + half.
  const uint32_t k_rel = col * 128 + ((mla_swizzle(col) ^ half) << 4);
  // V^T A-fragment via the transposing read: lane li of a 16-lane group points at 4 features of
  // token (li >> 2) of the group's 4 tokens and receives feature li of the group's 16 for the 4
  // tokens.  Contraction slot half*8 + i of fragment kk holds token kk*16 + (i/4)*8 + half*4 + i%4,
  // the order in which the S^T accumulator registers hold the tokens.  Feature block db: column
  // block db/2, logical piece (db%2)*4 + gg*2 + (li%4)/2; rows v_row + kk*16 + e*8, whose swizzle is
  // that of v_row XOR (kk*2 + e).
  const int li = lane & 15;
  const int gg = (lane >> 4) & 1;
  const int v_row = half * 4 + (li >> 2);
  const uint32_t v_rel = v_row * 128 + (li & 1) * 8 + (((gg * 2 + ((li & 3) >> 1)) ^ mla_swizzle(v_row)) << 4);

  // Both products read their A-fragments from LDS through a ring of RING fragments: the read of
  // fragment t + RING - 1 is issued right after matrix instruction t, i.e. RING - 1 instructions
  // (of 32 cycles each) ahead of its use, which is what the LDS takes under the load of four waves.
  // A scheduling fence after every step keeps the compiler from hoisting all reads of a product
  // (which would not fit the register file).
  constexpr int RING = 8;
  auto read_k_frag = [&](uint32_t k_at, int ks) -> half8_t {  // k_at: stage base + k_rel
    return lds_read_b128_at((k_at ^ (((ks & 3) * 2) << 4)) + (ks >> 2) * (BLK * 2));
  };
  auto read_v_frag = [&](uint32_t v_at, int t) -> half8_t {  // v_at: stage base + v_rel; t = 2*db + kk
    const int db = t >> 1, kk = t & 1;
    half8_t a;
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      const int c = ((db & 1) << 2) | (kk * 2 + e);
      const half4_t part = lds_read_tr16_at((v_at ^ (c << 4)) + (db >> 1) * (BLK * 2) + (kk * 16 + e * 8) * 128);
      a[e * 4 + 0] = part[0]; a[e * 4 + 1] = part[1];
      a[e * 4 + 2] = part[2]; a[e * 4 + 3] = part[3];
    }
    return a;
  };
  // S^T = KV Q^T over all DQK features for the 32 tokens of a tile
  auto qk = [&](uint32_t stage_at, auto&& beside) -> float16_t {  // beside(t): scalar / vector work placed after instruction t
    float16_t acc;
    half8_t a[RING];
    const uint32_t k_at = stage_at + k_rel;
#pragma unroll
    for (int t = 0; t < RING - 1; ++t) a[t] = read_k_frag(k_at, t);
    __builtin_amdgcn_sched_barrier(0);
    static_for<KS>([&](auto tc) {
      constexpr int t = decltype(tc)::value;
      // Written as assembly to put S into ordinary vector registers: with a whole register file per
      // wave the compiler selects the form of the matrix instructions whose results live in
      // accumulation registers, and O fills all 256 of those.
      if constexpr (t == 0) {
        // C = 0 as a literal instead of sixteen zeroed registers; the result must not share
        // registers with the operands
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a[0]), "v"(qf[0]) : MLA_ACC_REGS);
      } else if constexpr (t == KS - 1) {
        // the compiler does not know this is a matrix instruction: the wait states it would put
        // between the last one and the first vector instruction that reads S are spelled out
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 15\n\ts_nop 7" : "+v"(acc) : "v"(a[t % RING]), "v"(qf[t]) : MLA_ACC_REGS);
      } else {
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a[t % RING]), "v"(qf[t]) : MLA_ACC_REGS);
      }
      if constexpr (t + RING - 1 < KS) a[(t + RING - 1) % RING] = read_k_frag(k_at, t + RING - 1);
      beside(tc);
      __builtin_amdgcn_sched_barrier(0);
    });
    return acc;
  };
  // Online softmax of a tile's scores, cut into slots that sit between the matrix instructions of
  // the PV product running beside it (vec_slot<t> follows instruction t).  s[j]: token kv0 + (j/4)*8 +
  // half*4 + j%4, query col.  The reference point only moves when the maximum exceeds it by more
  // than 2^8 (p stays <= 256, same relative precision in fp16), so that after the first tiles no
  // block rescales O; a fully masked row keeps its reference point.  Slots 0 .. 3: row maximum of the
  // lane's 16 scores; 4: the other half's maximum; 5: new reference point, factor for the old
  // state; 6 .. 21: one probability each (a slot must not take longer than the 32 cycles of a matrix
  // instruction, or the matrix pipe waits for the wave), packed in pairs as the B-operand of the
  // next PV product.
  float alpha = 1.0f, row_mx = 0.f;
  auto mask_scores = [&](float16_t& s, int kv0) {
    if (kv0 + BN > wave_limit_min) {  // wave-uniform: the causal diagonal or the end of the sequence
      asm volatile("" ::: "memory");
      const int rel = my_limit - kv0 - half * 4;
#pragma unroll
      for (int j = 0; j < 16; ++j) s[j] = ((j >> 2) * 8 + (j & 3)) < rel ? s[j] : -3.0e38f;
    }
  };
  auto vec_slot = [&](auto tc, float16_t& s, half8_t (&pf)[2], float& tok) {
    constexpr int t = decltype(tc)::value;
    if constexpr (t < 4) {  // a quarter of the lane's 16 scores each
      float mx = t == 0 ? -3.0e38f : row_mx;
      pin_after(mx, tok);  // everything below hangs on it
#pragma unroll
      for (int j = t * 4; j < t * 4 + 4; ++j) mx = fmaxf(mx, s[j]);
      row_mx = mx;
      pin_after(tok, row_mx);
    } else if constexpr (t == 4) {
      pin_after(row_mx, tok);
      row_mx = max_xor32(row_mx);
      pin_after(tok, row_mx);
    } else if constexpr (t == 5) {
      pin_after(row_mx, tok);
      const float cand = fmaxf(row_mx * p.scale_log2, -1.0e30f);
      const float m_new = cand > m + 8.0f ? cand : m;
      alpha = fast_exp2(m - m_new);
      m = m_new;
      lsum *= alpha;
      pin_after(tok, lsum);
    } else if constexpr (t >= 6 && t < 6 + 16) {
      constexpr int j = t - 6;  // one probability per slot, two of them packed in the odd ones
      float mm = m;
      pin_after(mm, tok);
      const float pj = fast_exp2(fmaf(s[j], p.scale_log2, -mm));  // masked: exp2(-huge) = 0
      lsum += pj;
      if constexpr ((j & 1) == 0) {
        s[j] = pj;  // kept until its neighbour is there
      } else {
        pf[j >> 3][(j & 7) - 1] = static_cast<half_t>(s[j - 1]);
        pf[j >> 3][j & 7] = static_cast<half_t>(pj);
      }
      pin_after(tok, lsum);
    }
  };
  auto softmax_alone = [&](float16_t& s, int kv0, half8_t (&pf)[2]) {
    float tok = 0.f;
    mask_scores(s, kv0);
    static_for<22>([&](auto tc) { vec_slot(tc, s, pf, tok); });
  };
  // O^T += V^T P^T (the value is the first DV features of the same rows), optionally with the
  // softmax of the next tile's scores on the vector ALU beside it
  auto pv = [&](uint32_t stage_at, const half8_t (&pf_in)[2], auto with_softmax, float16_t& s, int kv0, half8_t (&pf_out)[2]) {
    half8_t a[RING];
    const uint32_t v_at = stage_at + v_rel;
    float tok = 0.f;
    if (decltype(with_softmax)::value) mask_scores(s, kv0);
#pragma unroll
    for (int t = 0; t < RING - 1; ++t) a[t] = read_v_frag(v_at, t);
    __builtin_amdgcn_sched_barrier(0);
    static_for<DB * 2>([&](auto tc) {
      constexpr int t = decltype(tc)::value;  // instruction t: feature block t/2, tokens (t%2)*16 .. +15
      acc_mfma_32x32x16<(t / 2) * 16>(a[t % RING], pf_in[t & 1], tok);
      if constexpr (t + RING - 1 < DB * 2) a[(t + RING - 1) % RING] = read_v_frag(v_at, t + RING - 1);
      if constexpr (decltype(with_softmax)::value) vec_slot(tc, s, pf_out, tok);
      __builtin_amdgcn_sched_barrier(0);
    });
  };
  auto rescale = [&]() {
    if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.0f))) {  // wave-uniform: skip when no maximum moved
      acc_settle();
      static_for<DB * 16>([&](auto r) { acc_scale<decltype(r)::value>(alpha); });
      acc_settle();
    }
  };

  // The wave is alone on its SIMD, so it overlaps its own matrix and vector work: the PV product of
  // a tile runs one iteration late, beside the softmax of the next tile's scores.  Iteration w:
  // S(w) = K(w) Q^T; then O += V(w-1) P(w-1) on the matrix pipe while the vector ALU turns S(w) into
  // P(w); the rescale of O that a moved reference point asks for (rare) follows the product.
  // Stages: tile w-1 (V in use), tile w, and tiles w+1 / w+2 in flight.  Every wave walks all tiles
  // of the workgroup (a tile beyond a wave's own causal bound is masked like the diagonal one):
  // with 128 heads a workgroup is a single position anyway.
  const int n_tiles = tile_hi - tile_lo;
  // ---- the query rows ---------------------------------------------------------------------------
  // A wave's 32 query rows are 32 consecutive rows of q, 36 KiB: the shape of a tile.  Loaded straight
  // into the fragment layout, every load instruction touches 32 rows x 32 bytes and the texture cache
  // looks up 32 lines for it (10 k cycles for the four waves of a decode step, the longest part of the
  // workgroup's start-up); copied to LDS like a tile, an instruction moves 8 rows x 128 bytes, and
  // the fragments come out of LDS the way the K fragments do.  A wave's rows fill one pipeline stage,
  // and stages 2 and 3 are free until the tiles 2 and 3 are copied: waves 0 and 1 go first, beside the
  // load of the page ids, waves 2 and 3 after them, beside the copies of the first two tiles.
  {
    // the wave's first row (a wave past the end of the rows copies the last row, and zeroes what it reads)
    const int q_first = min(first_row_wave, rows - 1);
    const half_t* q_wave = p.q + (static_cast<int64_t>(q_start) * h_q + q_first) * DQK;
    const int q_last = rows - 1 - q_first;  // rows past it repeat it
    const int q_stage = 2 + (wave & 1);
    const uint32_t q_at = lds_base + q_stage * (STAGE * 2);
    auto copy_q = [&]() {
#pragma unroll
      for (int n = 0; n < NCOPY; ++n) {
        const int blk = n >> 2;
        const int rg = n & 3;
        const int row = rg * 8 + (lane >> 3);
        const int piece = (lane & 7) ^ mla_swizzle(row);
        const uint32_t src = min(row, q_last);
        copy16_to_lds(q_wave, src * (DQK * 2) + (blk * 64 + piece * 8) * 2, q_at + (blk * BLK + rg * 8 * 64) * 2);
      }
    };
    auto read_q = [&]() {
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[ks] = read_k_frag(q_at + k_rel, ks);
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
      if (!row_valid) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) qf[ks] = zero16().h8;
      }
    };
    if (wave < 2) {  // (wave is a scalar: uniform branches)
      copy_q();
      wait_vmcnt<0>();
      read_q();
    }
    __syncthreads();  // stages 2 and 3 are free again
    // the page ids have long arrived; said here, so that the wait the compiler puts in front of their first use
    // (it waits for every load in flight) does not fall behind the copies of the query rows
    asm volatile("" : "+v"(page_ids));
    if (wave >= 2) copy_q();
#pragma unroll
    for (int s = 0; s < 2; ++s) {
      if (s < n_tiles) issue_tile(tile_lo + s);
    }
    if (wave >= 2) {
      // copies complete in order: the query rows are in when no more than the tile copies issued after them are outstanding
      if (n_tiles >= 2) {
        wait_vmcnt<2 * COPIES>();
      } else if (n_tiles == 1) {
        wait_vmcnt<COPIES>();
      } else {
        wait_vmcnt<0>();
      }
      read_q();
    }
    // (the copies of tile 2 into stage 2 are issued after the barrier of tile_ready(0), which every wave reaches
    //  with its query rows in registers)
  }
  auto tile_ready = [&](int w) {
    // copies complete in order: it is enough that no more than the next tile's copies are outstanding
    if (w + 1 < n_tiles) {
      wait_vmcnt<COPIES>();
    } else {
      wait_vmcnt<0>();
    }
    __syncthreads();  // everyone's part of tile w has landed; everyone is done with the stage of tile w-2
  };
  // Where the fast form applies, the copies of tile w+2 go out one by one between the matrix
  // instructions of S(w), which leave the scalar and vector units idle; otherwise before them.
  auto qk_and_copies = [&](int w) -> float16_t {
    const uint32_t stage_at = lds_base + (w % NSTAGE) * (STAGE * 2);
    if (w + 2 < n_tiles) {
      const int tile = tile_lo + w + 2;
      if (tile_in_page && (tile + 1) * BN <= kv_len) {  // wave-uniform
        return qk(stage_at, [&](auto tc) {
          constexpr int t = decltype(tc)::value;
          if constexpr (t == 0) {
            fast_copy_prepare(tile);
          } else if constexpr (t % 3 == 0 && t / 3 <= COPIES) {
            fast_copy_step(std::integral_constant<int, t / 3 - 1>{});
          }
        });
      }
      issue_tile(tile);
    }
    return qk(stage_at, [&](auto) {});
  };
  if (n_tiles > 0) {
    half8_t pf_prev[2];
    float16_t s;
    tile_ready(0);
    s = qk_and_copies(0);
    softmax_alone(s, tile_lo * BN, pf_prev);  // nothing accumulated yet: no rescale
    for (int w = 1; w < n_tiles; ++w) {
      tile_ready(w);
      half8_t pf[2];
      s = qk_and_copies(w);
      pv(lds_base + ((w - 1) % NSTAGE) * (STAGE * 2), pf_prev, std::true_type{}, s, (tile_lo + w) * BN, pf);
      rescale();
      pf_prev[0] = pf[0];
      pf_prev[1] = pf[1];
    }
    half8_t pf_unused[2];
    pv(lds_base + ((n_tiles - 1) % NSTAGE) * (STAGE * 2), pf_prev, std::false_type{}, s, 0, pf_unused);
  }

  // the row sums are per half of the wave: add them up; m is already common
  lsum = sum_xor32(lsum);
  acc_settle();  // the last PV product's results, before the vector ALU reads them
  if (nchunks == 1) {
    if (row_valid) {
      const int64_t grow = static_cast<int64_t>(q_start + my_pos) * h_q + my_head;  // global row
      const float denom = lsum + fast_exp2(kNegInit - m);
      const float inv = 1.0f / denom;
      half_t* orow = p.output + grow * DV + half * 4;
      static_for<DB * 4>([&](auto qc) {
        constexpr int q4 = decltype(qc)::value;  // registers 4*q4 .. 4*q4+3: block q4/4, feature group q4%4
        half4_t out4;
        out4[0] = static_cast<half_t>(acc_read<q4 * 4 + 0>() * inv);
        out4[1] = static_cast<half_t>(acc_read<q4 * 4 + 1>() * inv);
        out4[2] = static_cast<half_t>(acc_read<q4 * 4 + 2>() * inv);
        out4[3] = static_cast<half_t>(acc_read<q4 * 4 + 3>() * inv);
        *reinterpret_cast<half4_t*>(orow + (q4 / 4) * 32 + (q4 % 4) * 8) = out4;
      });
      if (half == 0) p.lse[grow] = m + fast_log2(denom);
    }
  } else {
    // A chunk of a one-token sequence (the row is the head).  Its state goes out normalised, in fp16,
    // with the log-sum-exp beside it.  A lane holds 4 features of a head here and there; the rows are
    // put together in LDS (the tile stages are free by now) and leave as whole 1 KiB rows.
    constexpr int PSTRIDE = DV + 8;  // halfs: consecutive rows start 4 banks apart
    static_assert(MLA_WAVES * 32 * PSTRIDE <= NSTAGE * STAGE, "the tile stages hold the rows of all waves");
    __syncthreads();  // every wave is done with the tiles
    half_t* wave_rows = lds_tiles + wave * (32 * PSTRIDE);
    const float inv = lsum > 0.f ? 1.0f / lsum : 0.f;  // a chunk without a visible token weighs nothing
    static_for<DB * 4>([&](auto qc) {
      constexpr int q4 = decltype(qc)::value;
      half4_t out4;
      out4[0] = static_cast<half_t>(acc_read<q4 * 4 + 0>() * inv);
      out4[1] = static_cast<half_t>(acc_read<q4 * 4 + 1>() * inv);
      out4[2] = static_cast<half_t>(acc_read<q4 * 4 + 2>() * inv);
      out4[3] = static_cast<half_t>(acc_read<q4 * 4 + 3>() * inv);
      *reinterpret_cast<half4_t*>(wave_rows + col * PSTRIDE + (q4 / 4) * 32 + (q4 % 4) * 8 + half * 4) = out4;
    });
    // the rows are read back below through another type: keep the reads behind the writes
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    const int head0 = r0 + wave * 32;
    const int nrows = min(32, rows - head0);
    half_t* dst = p.part_o + (static_cast<int64_t>(cslot) * h_q + head0) * DV + lane * 8;
    for (int r4 = 0; r4 < nrows; r4 += 4) {  // four rows at a time: their LDS reads are in flight together
      Vec16 v[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) v[k].u = *reinterpret_cast<const uint4*>(wave_rows + min(r4 + k, 31) * PSTRIDE + lane * 8);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (r4 + k < nrows) st16(dst + (r4 + k) * DV, v[k]);
      }
    }
    if (row_valid && half == 0) p.part_lse[static_cast<int64_t>(cslot) * h_q + my_head] = lsum > 0.f ? m + fast_log2(lsum) : kNegInit;
  }
  if (row_step == 0) break;
  __syncthreads();  // the LDS stages are reused by the next pass
  }
}

// The merge of a split call: block i merges the i-th slice of the heads of the sequence that chunk slot i
// belongs to (the kernel above left a note of the plan for every slot).
template <int DV>
__global__ __launch_bounds__(256) void mla_merge_kernel(MlaParams p) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int4 plan = p.slot_plan[blockIdx.x];  // {token row, chunk, nchunks, first slot}
  if (plan.z <= 1) return;
  mla_merge_heads<DV, 8>(p, plan.x, plan.w, plan.z, static_cast<int>(static_cast<int64_t>(plan.y) * p.h_q / plan.z),
                         static_cast<int>(static_cast<int64_t>(plan.y + 1) * p.h_q / plan.z), wave, 4, lane);
}

}  // namespace tvmkv

using namespace tvmkv;

// token_count >= 0: the launch covers the tokens token_base .. token_base + token_count - 1 of the call only, each
// planned as a one-token sequence (a part of a call that was cut up, see below); -1: the whole call.
static int mla_entry(const void* q, const int32_t* q_indptr, const void* pages, const int32_t* page_indptr,
                     const int32_t* page_values, const int32_t* length_info, void* output, float* lse, int64_t causal,
                     double sm_scale, int32_t batch_size, int64_t total_q, int64_t nnz_pages, int64_t num_pages,
                     int32_t h_q, int32_t d_latent, int32_t d_rope, int32_t page_size, void* stream, int64_t token_base,
                     int64_t token_count) {
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0) << "batch_prefill_paged_kv_mla: bad shape";
  KV_UNSUPPORTED(d_latent != 512 || d_rope != 64)
      << "batch_prefill_paged_kv_mla: (d_latent, d_rope) = (" << d_latent << ", " << d_rope
      << ") is not built ((512, 64))";
  KV_UNSUPPORTED(page_size <= 0 || page_size % 8 != 0)
      << "batch_prefill_paged_kv_mla: page_size " << page_size << " must be a positive multiple of 8";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && pages && page_indptr && length_info && output && lse)
      << "batch_prefill_paged_kv_mla: NULL tensor";
  KV_CHECK(nnz_pages == 0 || page_values) << "batch_prefill_paged_kv_mla: NULL page table";
  constexpr int DQK = 576, DV = 512;
  // A decode step of more sequences than one split launch plans (two per lane of the planning wave) with
  // long sequences would run one workgroup per sequence, as long as its longest one and in arbitrary
  // order: it is cut into equal parts of at most that many sequences, each a split launch of its own
  // (200 sequences of 2048-8192 tokens: 0.57 ms in one unsplit launch).  The index arrays hold absolute
  // offsets, so a part is the same call on a slice of them.
  const bool parts_fit = static_cast<int64_t>(MLA_MAX_SPLIT_BATCH) * ((h_q + MLA_BM - 1) / MLA_BM) * 2 <= compute_units() &&
                         nnz_pages > 0 && nnz_pages * page_size < (int64_t{1} << 26) &&
                         nnz_pages * page_size / batch_size >= 1024;
  if (token_count < 0 && total_q == batch_size && batch_size > MLA_MAX_SPLIT_BATCH &&
      batch_size <= 4 * MLA_MAX_SPLIT_BATCH && parts_fit) {
    const int parts = (batch_size + MLA_MAX_SPLIT_BATCH - 1) / MLA_MAX_SPLIT_BATCH;
    for (int i = 0; i < parts; ++i) {
      const int lo = static_cast<int>(static_cast<int64_t>(i) * batch_size / parts);
      const int hi = static_cast<int>(static_cast<int64_t>(i + 1) * batch_size / parts);
      const int rc = mla_entry(q, q_indptr + lo, pages, page_indptr + lo, page_values, length_info + lo, output, lse,
                               causal, sm_scale, hi - lo, hi - lo, nnz_pages, num_pages, h_q, d_latent, d_rope, page_size,
                               stream, 0, -1);
      if (rc != TVMKV_OK) return rc;
    }
    return TVMKV_OK;
  }
  // The same for a call with a few tokens per sequence (a draft to verify) and more tokens than one launch plans:
  // parts of at most that many consecutive tokens, each planned as one-token sequences over the whole index arrays.
  if (token_count < 0 && total_q != batch_size && total_q > MLA_MAX_SPLIT_BATCH && total_q <= 4 * MLA_MAX_SPLIT_BATCH &&
      parts_fit) {
    const int parts = static_cast<int>((total_q + MLA_MAX_SPLIT_BATCH - 1) / MLA_MAX_SPLIT_BATCH);
    for (int i = 0; i < parts; ++i) {
      const int64_t lo = i * total_q / parts, hi = (i + 1) * total_q / parts;
      const int rc = mla_entry(q, q_indptr, pages, page_indptr, page_values, length_info, output, lse, causal, sm_scale,
                               batch_size, total_q, nnz_pages, num_pages, h_q, d_latent, d_rope, page_size, stream, lo,
                               hi - lo);
      if (rc != TVMKV_OK) return rc;
    }
    return TVMKV_OK;
  }
  MlaParams p{};
  ScratchLease lease{};  // held until the launches are enqueued
  p.q = static_cast<const half_t*>(q);
  p.q_indptr = q_indptr;
  p.pages = static_cast<const half_t*>(pages);
  p.page_indptr = page_indptr;
  p.page_values = page_values;
  p.last_page_len = length_info;
  p.output = static_cast<half_t*>(output);
  p.lse = lse;
  p.batch_size = batch_size;
  p.h_q = h_q;
  p.page_size = page_size;
  p.causal = causal > 0;
  p.scale_log2 = static_cast<float>(sm_scale) * kLog2e;
  const int64_t slots = total_q * h_q / MLA_BM + (h_q % MLA_BM != 0 ? batch_size : 0);
  KV_CHECK(slots < (int64_t{1} << 31)) << "batch_prefill_paged_kv_mla: too many row tiles";
  // Decode-shaped calls (one token per sequence, as far as the shapes tell) have too few row tiles
  // for the chip, so the KV of the sequences is cut into chunks.  One workgroup per compute unit is
  // resident (LDS): the grid is one round of workgroups, and the kernel fits the chunks to it.
  const int cus = compute_units();
  const int row_tiles = (h_q + MLA_BM - 1) / MLA_BM;
  int64_t grid = slots;
  // A call with a few tokens per sequence (a draft to verify, a short chunk late in a long prompt) is in the
  // same position: its tokens are planned as one-token sequences of their own.
  const int64_t planned = token_count >= 0 ? token_count : total_q;
  KV_CHECK(token_count < 0 || (planned * row_tiles * 2 <= cus && planned <= MLA_MAX_SPLIT_BATCH))
      << "batch_prefill_paged_kv_mla: a part of a call must fit one split launch";
  if (planned * row_tiles * 2 <= cus && planned <= MLA_MAX_SPLIT_BATCH && nnz_pages > 0 &&
      nnz_pages * page_size < (int64_t{1} << 26)) {
    if (token_count >= 0 || total_q != batch_size) {
      p.tokens_of = batch_size;
      p.batch_size = static_cast<int>(planned);
      p.token_base = static_cast<int>(token_base);
    }
    const int64_t cslots = cus / row_tiles;
    p.split = 1;
    p.row_tiles = row_tiles;
    p.min_chunk_tiles = MLA_MIN_CHUNK / MLA_BN;
    if (option(kOptMlaChunkTokens) >= MLA_BN) p.min_chunk_tiles = static_cast<int>(option(kOptMlaChunkTokens) / MLA_BN);  // tuning aid
    grid = cslots * row_tiles;
    const size_t part_rows = static_cast<size_t>(cslots) * h_q;
    const size_t part_o_bytes = part_rows * DV * sizeof(half_t);
    const size_t part_lse_bytes = (part_rows * sizeof(float) + 15) / 16 * 16;
    lease = lease_scratch(kScratchMla, as_stream(stream), part_o_bytes + part_lse_bytes + cslots * sizeof(int4), 0);
    char* ws = lease.ptr;
    p.part_o = reinterpret_cast<half_t*>(ws);
    p.part_lse = reinterpret_cast<float*>(ws + part_o_bytes);
    p.slot_plan = reinterpret_cast<int4*>(ws + part_o_bytes + part_lse_bytes);
  }
  constexpr size_t lds_bytes = static_cast<size_t>(MLA_STAGES) * MLA_BN * DQK * sizeof(half_t);
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&mla_paged_kernel<DQK, DV, true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&mla_paged_kernel<DQK, DV, false>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    attr_set = true;
  }
  hipStream_t s = as_stream(stream);
  KV_CHECK(grid < (int64_t{1} << 31)) << "batch_prefill_paged_kv_mla: too many work items";
  p.page_shift = -1;
  if ((page_size & (page_size - 1)) == 0) {
    p.page_shift = 0;
    while ((1 << p.page_shift) < page_size) ++p.page_shift;
    hipLaunchKernelGGL((mla_paged_kernel<DQK, DV, true>), dim3(static_cast<unsigned>(grid)), dim3(MLA_WAVES * 64),
                       lds_bytes, s, p);
  } else {
    hipLaunchKernelGGL((mla_paged_kernel<DQK, DV, false>), dim3(static_cast<unsigned>(grid)), dim3(MLA_WAVES * 64),
                       lds_bytes, s, p);
  }
  KV_LAUNCH_CHECK();
  if (p.split) {
    hipLaunchKernelGGL(mla_merge_kernel<DV>, dim3(static_cast<unsigned>(grid / row_tiles)), dim3(256), 0, s, p);
    KV_LAUNCH_CHECK();
  }
  KV_API_END();
}

extern "C" int tvmkv_batch_prefill_paged_kv_mla(const void* q, const int32_t* q_indptr, const void* pages,
                                                const int32_t* page_indptr, const int32_t* page_values,
                                                const int32_t* length_info, void* output, float* lse,
                                                int64_t causal, double sm_scale, int32_t batch_size,
                                                int64_t total_q, int64_t nnz_pages, int64_t num_pages, int32_t h_q,
                                                int32_t d_latent, int32_t d_rope, int32_t page_size, void* stream) {
  return mla_entry(q, q_indptr, pages, page_indptr, page_values, length_info, output, lse, causal, sm_scale, batch_size,
                   total_q, nnz_pages, num_pages, h_q, d_latent, d_rope, page_size, stream, 0, -1);
}
