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
// Tiling: 128 rows (position, head) per workgroup of 8 wavefronts, 16 rows per wave with the query
// on the N axis of v_mfma_f32_16x16x32_f16: O^T of one wave is 512 x 16 fp32 = 128 accumulator
// registers, Q is 72 registers of B-fragments, which leaves room for two waves per SIMD.  32-token
// tiles of cached rows are copied from global memory straight into LDS (global_load_lds_dwordx4),
// four stages deep; the same LDS bytes serve as A-operand of S^T = KV Q^T (ds_read_b128) and of
// O^T = V^T P^T (ds_read_b64_tr_b16, which transposes on the way out of LDS).
//
// KV split: decode-shaped calls (one token per sequence) have too few row tiles to fill 256 CUs,
// so the KV of a sequence is cut into chunks of about `chunk_tokens` tokens; partial (O, m, l)
// states go to an fp32 buffer indexed by (chunk slot, head) and a second kernel merges them.  The
// chunk slots of a sequence are a pure function of the page table, recomputed by both kernels.
#include <algorithm>
#include <cstdlib>

#include "kernels_common.cuh"

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

// Split mode: sequence b owns the chunk slots [mla_chunk_slot_begin(b), mla_chunk_slot_begin(b+1)),
// a function of the page table alone (so the grid can be sized from shapes: at most
// floor(nnz_pages * page_size / chunk_tokens) + batch slots, every one of them in use), and its KV
// tiles are divided evenly among them: about chunk_tokens tokens each.
__device__ __forceinline__ int mla_chunk_slot_begin(const int32_t* page_indptr, int b, int page_size, int chunk_tokens) {
  return static_cast<int>(static_cast<int64_t>(page_indptr[b]) * page_size / chunk_tokens) + b;
}

constexpr int MLA_WAVES = 8;    // wavefronts per workgroup, 16 rows each
constexpr int MLA_STAGES = 4;   // 4 x 36 KiB of LDS: three tiles in flight behind the one being multiplied

// LDS image of a tile: DQK/64 column blocks of [MLA_BN rows][64 features] (128-byte rows, 8 pieces
// of 16 bytes).  The same bytes are the A-operand of S^T = KV Q^T (ds_read_b128: 16 lanes = 16
// consecutive rows at one piece) and, for the latent part, of O^T = V^T P^T (ds_read_b64_tr_b16: 32
// lanes = 8 consecutive rows x 32 bytes).  Piece c of row r sits at piece position c ^ (r & 7).
// A ds_read_b128 is served in four passes of 16 lanes, and the passes are not the four quarters of
// the wave: within each half of it, the 4-lane blocks {0, 3, 5, 6} form one pass and {1, 2, 4, 7} the
// other (measured: two such blocks on the same banks cost a cycle, two blocks of different passes do
// not).  For the K fragment that is rows {0-3, 12-15} at one piece and rows {4-11} at the next one;
// with this swizzle the 16 lanes of a pass cover all 64 banks, and so do the 32 lanes of a pass of
// the transposing read.
__device__ __forceinline__ int mla_swizzle(int row) {
  return row & 7;
}

template <int DQK, int DV>
__global__ __launch_bounds__(MLA_WAVES * 64) void mla_paged_kernel(MlaParams p) {
  constexpr int BN = MLA_BN;
  static_assert(BN == 32 && MLA_BM == MLA_WAVES * 16 && DQK % 64 == 0 && DV % 64 == 0 && DV <= DQK, "tile shape");
  constexpr int KS = DQK / 32;               // k-steps of the score product (v_mfma_f32_16x16x32_f16)
  constexpr int DB = DV / 16;                // 16-wide output feature blocks
  constexpr int NBLK = DQK / 64;             // column blocks of a tile
  constexpr int BLK = BN * 64;               // halfs per column block
  constexpr int STAGE = NBLK * BLK;          // halfs per stage
  constexpr int NSTAGE = MLA_STAGES;
  constexpr int NCOPY = NBLK * (BN / 8);     // copy instructions (8 rows x 128 B) per tile
  constexpr int COPIES_HI = (NCOPY + MLA_WAVES - 1) / MLA_WAVES;  // per wave: the first NCOPY % MLA_WAVES waves
  constexpr int COPIES_LO = NCOPY / MLA_WAVES;                    // ... the others
  constexpr int WAVES_HI = NCOPY % MLA_WAVES;

  extern __shared__ __attribute__((aligned(16))) half_t lds_tiles[];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int c16 = lane & 15;   // query row of the wave (MFMA column) / token row of an A-fragment
  const int g4 = lane >> 4;    // lane group: contraction slots 8*g4 .. 8*g4+7
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
  const int my_row = r0 + wave * 16 + c16;
  const bool row_valid = my_row < rows;
  const int my_pos = my_row / h_q;
  const int my_head = my_row % h_q;
  const int causal_shift = kv_len - qo_len + 1;
  const int my_limit = row_valid ? (p.causal ? min(kv_len, causal_shift + my_pos) : kv_len) : 0;
  const int last_row_wg = min(rows, r0 + MLA_BM) - 1;
  const int kv_end = p.causal ? max(0, min(kv_len, causal_shift + last_row_wg / h_q)) : kv_len;
  const int first_row_wave = r0 + wave * 16;
  const int last_row_wave = min(rows, first_row_wave + 16) - 1;
  const bool wave_active = first_row_wave < rows;
  const int wave_limit_max = !wave_active ? 0 : (p.causal ? min(kv_len, causal_shift + last_row_wave / h_q) : kv_len);
  const int wave_limit_min = !wave_active ? 0 : (p.causal ? min(kv_len, causal_shift + first_row_wave / h_q) : kv_len);

  // tiles of this chunk: an even split of all tiles of the sequence, clipped by the causal bound
  const int tiles_all = (kv_len + BN - 1) / BN;
  const int tile_lo = static_cast<int>(static_cast<int64_t>(chunk) * tiles_all / nchunks);
  const int tile_hi = min(static_cast<int>(static_cast<int64_t>(chunk + 1) * tiles_all / nchunks), (kv_end + BN - 1) / BN);

  // Q^T fragments (B operand): column = query c16, contraction slots = features ks*32 + g4*8 .. +7
  half8_t qf[KS];
  {
    const half_t* qrow = p.q + (static_cast<int64_t>(q_start + my_pos) * h_q + my_head) * DQK + g4 * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = row_valid ? ld16(qrow + ks * 32).h8 : zero16().h8;
  }
  // O^T accumulators: o[db][j] is feature db*16 + 4*g4 + j of query c16
  float4_t o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) o[db] = float4_t{0.f, 0.f, 0.f, 0.f};
  float m = kNegInit, lsum = 0.f;

  // ---- tile copy: global -> LDS -------------------------------------------------------------
  // Copy instruction n of a tile (n = 0 .. NCOPY-1, dealt out to the waves in consecutive runs)
  // moves rows 8*(n%4) .. +7 of column block n/4.  Rows past the end of the sequence repeat its last
  // token (masked scores; P = 0 times a finite value).  The page ids of 16 consecutive tiles (4 row
  // groups each) are fetched by one vector load, lane = 4*tile + row group: the wait for that load
  // also waits for every copy in flight, so it must be rare.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const bool copies_hi = wave_u < WAVES_HI;
  const int copy_first = copies_hi ? wave_u * COPIES_HI : WAVES_HI * COPIES_HI + (wave_u - WAVES_HI) * COPIES_LO;
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)lds_tiles));
  const int last_tok = kv_len - 1;
  int page_ids = 0;
  auto issue_tile = [&](int tile) {
    const int w = tile - tile_lo;
    if ((w & 15) == 0) {
      const int t = min((tile + (lane >> 2)) * BN + (lane & 3) * 8, last_tok);
      page_ids = p.page_values[pbeg + t / ps];
    }
    const int kv0 = tile * BN;
    const uint32_t stage = lds_base + (w % NSTAGE) * (STAGE * 2);
#pragma unroll
    for (int j = 0; j < COPIES_HI; ++j) {
      if (j < COPIES_LO || copies_hi) {  // wave-uniform
        const int n = copy_first + j;
        const int blk = n >> 2;
        const int rg = n & 3;
        const int page = __builtin_amdgcn_readlane(page_ids, (w & 15) * 4 + rg);
        const half_t* base = p.pages + static_cast<int64_t>(page) * ps * DQK;
        const int row = rg * 8 + (lane >> 3);
        const int piece = (lane & 7) ^ mla_swizzle(row);
        const uint32_t t = min(kv0 + row, last_tok);
        const uint32_t off = (t % ps) * (DQK * 2) + (blk * 64 + piece * 8) * 2;
        copy16_to_lds(base, off, stage + (blk * BLK + rg * 8 * 64) * 2);
      }
    }
  };

  // ---- per-lane fragment addressing (halfs, relative to a stage) ---------------------------------
  // K A-fragment of k-step ks, token block tb: row tb*16 + c16, features ks*32 + g4*8 .. +7
  const int k_lane_off = c16 * 64;
  const int k_swz = mla_swizzle(c16);  // the same for row + 16
  // V^T A-fragment via the transposing read: lane li of a 16-lane group points at 4 features of
  // token (li >> 2) of the group's 4 tokens and receives feature li of the group's 16 for the 4
  // tokens.  Contraction slot 8*g4 + i holds token (i/4)*16 + 4*g4 + i%4, the order in which the
  // S^T accumulators of the two token blocks hold them.
  const int li = lane & 15;
  const int v_row = 4 * g4 + (li >> 2);               // + 16 for the second half of the fragment
  const int v_swz = mla_swizzle(v_row);               // row + 16 does not change it
  const int v_lane_off = v_row * 64 + (li & 1) * 4;
  const int v_piece = (li & 3) >> 1;                   // + 2 * (feature block % 4)

  const int n_tiles = tile_hi - tile_lo;
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s) {
    if (s < n_tiles) issue_tile(tile_lo + s);
  }
  for (int w = 0; w < n_tiles; ++w) {
    const int kv0 = (tile_lo + w) * BN;
    const half_t* T = lds_tiles + (w % NSTAGE) * STAGE;
    // copies complete in order: it is enough that no more than the later tiles' copies are outstanding
    if (w + NSTAGE - 2 < n_tiles) {
      if (copies_hi) {
        wait_vmcnt<(NSTAGE - 2) * COPIES_HI>();
      } else {
        wait_vmcnt<(NSTAGE - 2) * COPIES_LO>();
      }
    } else {
      wait_vmcnt<0>();
    }
    __syncthreads();  // everyone's part of this tile has landed; everyone is done with the stage of tile w-1
    if (w + NSTAGE - 1 < n_tiles) issue_tile(tile_lo + w + NSTAGE - 1);

    if (kv0 >= wave_limit_max) continue;  // wave-uniform: every row of this wave is masked out

    // ---- S^T = KV Q^T over all DQK features: two blocks of 16 tokens ------------------------------
    float4_t s[2];
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
      s[tb] = float4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const int piece = ((ks & 1) * 4 + g4) ^ k_swz;
        const half8_t a = *reinterpret_cast<const half8_t*>(T + (ks >> 1) * BLK + tb * 16 * 64 + k_lane_off + piece * 8);
        s[tb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, qf[ks], s[tb], 0, 0, 0);
      }
    }
    // s[tb][j]: token kv0 + tb*16 + 4*g4 + j, query c16
    if (kv0 + BN > wave_limit_min) {  // wave-uniform: the causal diagonal or the end of the sequence
      asm volatile("" ::: "memory");
      const int rel = my_limit - kv0 - 4 * g4;
#pragma unroll
      for (int tb = 0; tb < 2; ++tb) {
#pragma unroll
        for (int j = 0; j < 4; ++j) s[tb][j] = (tb * 16 + j) < rel ? s[tb][j] : -3.0e38f;
      }
    }
    float mx = -3.0e38f;
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
#pragma unroll
      for (int j = 0; j < 4; ++j) mx = fmaxf(mx, s[tb][j]);
    }
    mx = max_xor32(max_xor16(mx));
    // The reference point only moves when the maximum exceeds it by more than 2^8 (p stays <= 256,
    // same relative precision in fp16), so that after the first tiles no block rescales O; a fully
    // masked row keeps its reference point.
    const float cand = fmaxf(mx * p.scale_log2, -1.0e30f);
    const float m_new = cand > m + 8.0f ? cand : m;
    const float alpha = fast_exp2(m - m_new);
    m = m_new;
    lsum *= alpha;
    if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.0f))) {  // wave-uniform: skip when no maximum moved
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] *= alpha;
    }
    half8_t pf;
#pragma unroll
    for (int tb = 0; tb < 2; ++tb) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float pj = fast_exp2(fmaf(s[tb][j], p.scale_log2, -m_new));  // masked: exp2(-huge) = 0
        lsum += pj;
        pf[tb * 4 + j] = static_cast<half_t>(pj);
      }
    }
    // ---- O^T += V^T P^T: the value is the first DV features of the same rows ---------------------
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const half_t* vb = T + (db >> 2) * BLK + v_lane_off + (((db & 3) * 2 + v_piece) ^ v_swz) * 8;
      const half4_t lo = lds_read_tr16(vb);
      const half4_t hi = lds_read_tr16(vb + 16 * 64);
      half8_t a;
      a[0] = lo[0]; a[1] = lo[1]; a[2] = lo[2]; a[3] = lo[3];
      a[4] = hi[0]; a[5] = hi[1]; a[6] = hi[2]; a[7] = hi[3];
      o[db] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, pf, o[db], 0, 0, 0);
    }
  }

  // the row sums are per lane group: add them up; m is already common
  lsum = sum_xor32(sum_xor16(lsum));
  if (row_valid) {
  const int64_t grow = static_cast<int64_t>(q_start + my_pos) * h_q + my_head;  // global row
  if (nchunks == 1) {
    const float denom = lsum + fast_exp2(kNegInit - m);
    const float inv = 1.0f / denom;
    half_t* orow = p.output + grow * DV + 4 * g4;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      half4_t out4;
#pragma unroll
      for (int e = 0; e < 4; ++e) out4[e] = static_cast<half_t>(o[db][e] * inv);
      *reinterpret_cast<half4_t*>(orow + db * 16) = out4;
    }
    if (g4 == 0) p.lse[grow] = m + fast_log2(denom);
  } else {
    // only one-token sequences are split: the row is the head
    const int64_t prow_idx = static_cast<int64_t>(cslot) * h_q + my_head;
    float* prow = p.part_o + prow_idx * DV + 4 * g4;
#pragma unroll
    for (int db = 0; db < DB; ++db) *reinterpret_cast<float4_t*>(prow + db * 16) = o[db];
    if (g4 == 0) {
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

struct MlaWorkspace {
  void* ptr = nullptr;
  size_t bytes = 0;
};
static MlaWorkspace g_mla_workspace[64];

static void* mla_workspace(size_t bytes) {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  KV_CHECK(dev >= 0 && dev < 64) << "device ordinal " << dev << " out of range";
  MlaWorkspace& ws = g_mla_workspace[dev];
  if (ws.bytes < bytes) {
    if (ws.ptr) {
      HIP_CHECK(hipDeviceSynchronize());
      HIP_CHECK(hipFree(ws.ptr));
      ws.ptr = nullptr;
      ws.bytes = 0;
    }
    HIP_CHECK(hipMalloc(&ws.ptr, bytes + bytes / 2));
    ws.bytes = bytes + bytes / 2;
  }
  return ws.ptr;
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
    if (const char* e = getenv("TVMKV_MLA_CHUNK_TOKENS")) {  // tuning aid
      if (atoi(e) >= MLA_BN) ct = atoi(e) / MLA_BN * MLA_BN;
    }
    const int64_t cslots = tokens / ct + batch_size;
    p.split = 1;
    p.chunk_tokens = static_cast<int>(ct);
    p.row_tiles = row_tiles;
    grid = cslots * row_tiles;
    const size_t part_rows = static_cast<size_t>(cslots) * h_q;
    const size_t part_o_bytes = part_rows * DV * sizeof(float);
    char* ws = static_cast<char*>(mla_workspace(part_o_bytes + part_rows * 2 * sizeof(float)));
    p.part_o = reinterpret_cast<float*>(ws);
    p.part_ml = reinterpret_cast<float*>(ws + part_o_bytes);
  }
  constexpr size_t lds_bytes = static_cast<size_t>(MLA_STAGES) * MLA_BN * DQK * sizeof(half_t);
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&mla_paged_kernel<DQK, DV>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    attr_set = true;
  }
  hipStream_t s = as_stream(stream);
  KV_CHECK(grid < (int64_t{1} << 31)) << "batch_prefill_paged_kv_mla: too many work items";
  hipLaunchKernelGGL((mla_paged_kernel<DQK, DV>), dim3(static_cast<unsigned>(grid)), dim3(MLA_WAVES * 64), lds_bytes,
                     s, p);
  KV_LAUNCH_CHECK();
  if (p.split) {
    hipLaunchKernelGGL(mla_merge_kernel<DV>, dim3(static_cast<unsigned>(total_q), h_q), dim3(DV / 4), 0, s, p);
    KV_LAUNCH_CHECK();
  }
  KV_API_END();
}
