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
// KV split: decode-shaped calls (one token per sequence) have too few row tiles to fill 256 CUs,
// so the KV of a sequence is cut into chunks of about `chunk_tokens` tokens; partial (O, m, l)
// states go to an fp32 buffer indexed by (chunk slot, head) and a second kernel merges them.  The
// chunk slots of a sequence are a pure function of the page table, recomputed by both kernels.
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
  float* part_o;   // (chunk slots, h_q, DV)
  float* part_ml;  // (chunk slots, h_q, 2)
  int batch_size;
  int h_q;
  int page_size;
  int page_shift;    // log2(page_size) when it is a power of two, else -1
  int causal;
  int split;         // 1: decode-shaped call, the KV of a sequence is cut into chunks (see mla_chunk_slot_begin)
  int chunk_tokens;  // target tokens per chunk
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
template <int R>
__device__ __forceinline__ void acc_mfma_32x32x16(half8_t a, half8_t b) {  // a[R:R+15] += a * b
  asm volatile("v_mfma_f32_32x32x16_f16 a[%2:%3], %0, %1, a[%2:%3]" : : "v"(a), "v"(b), "n"(R), "n"(R + 15));
}
// The same with an order token: `tok` is an operand the instruction does not touch.  Vector work that
// is made to depend on it (pin_after) cannot be scheduled before this matrix instruction, and a
// matrix instruction whose token depends on that work's result cannot be scheduled before the work:
// program order then alternates matrix and vector instructions, which a single wave needs in order
// to use both pipes at once (it issues in order).
template <int R>
__device__ __forceinline__ void acc_mfma_32x32x16(half8_t a, half8_t b, float& tok) {
  asm volatile("v_mfma_f32_32x32x16_f16 a[%3:%4], %1, %2, a[%3:%4]" : "+v"(tok) : "v"(a), "v"(b), "n"(R), "n"(R + 15));
}
__device__ __forceinline__ void pin_after(float& x, float on) { asm("" : "+v"(x) : "v"(on)); }  // no instruction

template <int R>
__device__ __forceinline__ void acc_zero() {
  asm volatile("v_accvgpr_write_b32 a[%0], 0" : : "n"(R));
}
template <int R>
__device__ __forceinline__ float acc_read() {
  float x;
  asm volatile("v_accvgpr_read_b32 %0, a[%1]" : "=v"(x) : "n"(R));
  return x;
}
template <int R>
__device__ __forceinline__ void acc_scale(float factor) {
  float t;
  asm volatile("v_accvgpr_read_b32 %0, a[%2]\n\tv_mul_f32 %0, %0, %1\n\tv_accvgpr_write_b32 a[%2], %0"
               : "=&v"(t) : "v"(factor), "n"(R));
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
  asm volatile("" ::: "a0", "a255");  // the kernel uses every accumulation register (by number, see above)

  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // a scalar: the bounds derived from it steer wave-uniform branches
  const int h_q = p.h_q;

  // Work item.  Normal mode: a row-tile slot.  Split mode: (chunk slot, row tile of a one-token
  // sequence), the grid holding exactly the items in use: a workgroup takes a whole compute unit
  // (LDS, registers) and runs long, and workgroups that only find out they have nothing to do
  // still disturb the placement of the others.
  int b, r0, chunk = 0, nchunks = 1, cslot = 0, row_step = 0;
  if (p.split) {
    cslot = blockIdx.x / p.row_tiles;
    r0 = (blockIdx.x - cslot * p.row_tiles) * MLA_BM;
    row_step = p.row_tiles * MLA_BM;
    int lo = 0, hi = p.batch_size - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (mla_chunk_slot_begin(p.page_indptr, mid, p.page_size, p.chunk_tokens) <= cslot) {
        lo = mid;
      } else {
        hi = mid - 1;
      }
    }
    b = lo;
    const int first = mla_chunk_slot_begin(p.page_indptr, b, p.page_size, p.chunk_tokens);
    chunk = cslot - first;
    nchunks = mla_chunk_slot_begin(p.page_indptr, b + 1, p.page_size, p.chunk_tokens) - first;
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
  }
  const int q_start = p.q_indptr[b];
  const int qo_len = p.q_indptr[b + 1] - q_start;
  const int rows = qo_len * h_q;
  if (p.split && qo_len != 1) {
    // not a decode step after all: the workgroups of chunk 0 do the whole sequence, unsplit
    if (chunk != 0) return;
    nchunks = 1;
  }

  const int pbeg = p.page_indptr[b];
  const int npages = p.page_indptr[b + 1] - pbeg;
  const int ps = p.page_size;
  const int kv_len = npages > 0 ? (npages - 1) * ps + p.last_page_len[b] : 0;

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

  // Q^T fragments (B operand): column = query col, contraction slots = features ks*16 + half*8 .. +7
  half8_t qf[KS];
  {
    const half_t* qrow = p.q + (static_cast<int64_t>(q_start + my_pos) * h_q + my_head) * DQK + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = row_valid ? ld16(qrow + ks * 16).h8 : zero16().h8;
  }
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
  const int last_tok = kv_len - 1;
  int page_ids = 0;
  // Per-lane part of a copy's source offset for rows that need no clamping: row lane/8 of the
  // 8-row group rg, piece (lane%8) ^ swizzle(rg*8 + lane/8) = this value ^ (rg << 4).
  const uint32_t copy_lane_off = (lane >> 3) * (DQK * 2) + (((lane & 7) ^ ((((lane >> 3) >> 1) & 1) << 2)) << 4);
  // General form of a tile's copies: a page id per 8-row group, rows past the end clamped.
  auto load_page_ids = [&](int tile) {
    if (((tile - tile_lo) & 15) == 0) {
      const int t = min((tile + (lane >> 2)) * BN + (lane & 3) * 8, last_tok);
      page_ids = p.page_values[pbeg + (POW2 ? t >> p.page_shift : t / ps)];
    }
  };
  auto issue_tile = [&](int tile) {
    load_page_ids(tile);
    const int w = tile - tile_lo;
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
    load_page_ids(tile);
    const int w = tile - tile_lo;
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
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, 0" : "=&v"(acc) : "v"(a[0]), "v"(qf[0]));
      } else if constexpr (t == KS - 1) {
        // the compiler does not know this is a matrix instruction: the wait states it would put
        // between the last one and the first vector instruction that reads S are spelled out
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0\n\ts_nop 15\n\ts_nop 7" : "+v"(acc) : "v"(a[t % RING]), "v"(qf[t]));
      } else {
        asm("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a[t % RING]), "v"(qf[t]));
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
#pragma unroll
  for (int s = 0; s < 2; ++s) {
    if (s < n_tiles) issue_tile(tile_lo + s);
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
  if (row_valid) {
  const int64_t grow = static_cast<int64_t>(q_start + my_pos) * h_q + my_head;  // global row
  if (nchunks == 1) {
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
  } else {
    // only one-token sequences are split: the row is the head
    const int64_t prow_idx = static_cast<int64_t>(cslot) * h_q + my_head;
    float* prow = p.part_o + prow_idx * DV + half * 4;
    static_for<DB * 4>([&](auto qc) {
      constexpr int q4 = decltype(qc)::value;
      const float4_t v4 = {acc_read<q4 * 4 + 0>(), acc_read<q4 * 4 + 1>(), acc_read<q4 * 4 + 2>(), acc_read<q4 * 4 + 3>()};
      *reinterpret_cast<float4_t*>(prow + (q4 / 4) * 32 + (q4 % 4) * 8) = v4;
    });
    if (half == 0) {
      p.part_ml[prow_idx * 2 + 0] = m;
      p.part_ml[prow_idx * 2 + 1] = lsum;
    }
  }
  }
  if (row_step == 0) break;
  __syncthreads();  // the LDS stages are reused by the next pass
  }
}

// One block per (query token, head); DV/4 threads, 4 features each.
template <int DV>
__global__ __launch_bounds__(DV / 4) void mla_merge_kernel(MlaParams p) {
  const int token = blockIdx.x;
  const int head = blockIdx.y;
  int b;
  {
    int lo = 0, hi = p.batch_size - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (p.q_indptr[mid] <= token) {
        lo = mid;
      } else {
        hi = mid - 1;
      }
    }
    b = lo;
  }
  // (sequences with qo_len == 0 share their q_indptr value with the next one: the search returns
  // the last b with q_indptr[b] <= token, which is the one that owns the token)
  if (p.q_indptr[b + 1] - p.q_indptr[b] != 1) return;  // only one-token sequences are split
  const int first = mla_chunk_slot_begin(p.page_indptr, b, p.page_size, p.chunk_tokens);
  const int nchunks = mla_chunk_slot_begin(p.page_indptr, b + 1, p.page_size, p.chunk_tokens) - first;
  if (nchunks == 1) return;
  const int64_t grow = static_cast<int64_t>(token) * p.h_q + head;
  const int64_t prow = static_cast<int64_t>(first) * p.h_q + head;  // + c * h_q for chunk c
  const float* ml = p.part_ml + prow * 2;
  const int64_t cstride = p.h_q;
  float mx = kNegInit;
  for (int c = 0; c < nchunks; ++c) mx = fmaxf(mx, ml[c * cstride * 2]);
  float lsum = 0.f;
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  const int d = threadIdx.x * 4;
  for (int c = 0; c < nchunks; ++c) {
    const float sc = fast_exp2(ml[c * cstride * 2] - mx);
    lsum += ml[c * cstride * 2 + 1] * sc;
    const float4_t po = *reinterpret_cast<const float4_t*>(p.part_o + (prow + c * cstride) * DV + d);
    acc += po * sc;
  }
  const float denom = lsum + fast_exp2(kNegInit - mx);
  const float inv = 1.0f / denom;
  half4_t out4;
#pragma unroll
  for (int e = 0; e < 4; ++e) out4[e] = static_cast<half_t>(acc[e] * inv);
  *reinterpret_cast<half4_t*>(p.output + grow * DV + d) = out4;
  if (threadIdx.x == 0) p.lse[grow] = mx + fast_log2(denom);
}

}  // namespace tvmkv

using namespace tvmkv;

extern "C" int tvmkv_batch_prefill_paged_kv_mla(const void* q, const int32_t* q_indptr, const void* pages,
                                                const int32_t* page_indptr, const int32_t* page_values,
                                                const int32_t* length_info, void* output, float* lse,
                                                int64_t causal, double sm_scale, int32_t batch_size,
                                                int64_t total_q, int64_t nnz_pages, int64_t num_pages, int32_t h_q,
                                                int32_t d_latent, int32_t d_rope, int32_t page_size, void* stream) {
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
  MlaParams p{};
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
  // Decode-shaped calls (one token per sequence, as far as the shapes tell) have too few row
  // tiles for the chip, so the KV of a sequence is cut into chunks of about chunk_tokens tokens.
  // One workgroup per compute unit is resident (LDS), so aim at one round of workgroups:
  // chunk slots = floor(tokens / chunk_tokens) + B, times the row tiles of a sequence, <= CUs.
  const int cus = compute_units();
  const int row_tiles = (h_q + MLA_BM - 1) / MLA_BM;
  const int64_t tokens = nnz_pages * page_size;  // upper bound on the cached tokens
  int64_t grid = slots;
  if (total_q == batch_size && static_cast<int64_t>(batch_size) * row_tiles * 2 <= cus && tokens > 0) {
    const int64_t room = cus / row_tiles - batch_size;
    int64_t ct = (tokens + room - 1) / room;
    ct = std::max<int64_t>(MLA_MIN_CHUNK, (ct + MLA_BN - 1) / MLA_BN * MLA_BN);
    if (option(kOptMlaChunkTokens) >= MLA_BN) ct = option(kOptMlaChunkTokens) / MLA_BN * MLA_BN;  // tuning aid
    const int64_t cslots = tokens / ct + batch_size;
    p.split = 1;
    p.chunk_tokens = static_cast<int>(ct);
    p.row_tiles = row_tiles;
    grid = cslots * row_tiles;
    const size_t part_rows = static_cast<size_t>(cslots) * h_q;
    const size_t part_o_bytes = part_rows * DV * sizeof(float);
    char* ws = lease_scratch(kScratchMla, as_stream(stream), part_o_bytes + part_rows * 2 * sizeof(float), 0).ptr;
    p.part_o = reinterpret_cast<float*>(ws);
    p.part_ml = reinterpret_cast<float*>(ws + part_o_bytes);
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
    hipLaunchKernelGGL(mla_merge_kernel<DV>, dim3(static_cast<unsigned>(total_q), h_q), dim3(DV / 4), 0, s, p);
    KV_LAUNCH_CHECK();
  }
  KV_API_END();
}
