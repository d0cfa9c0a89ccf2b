// Ragged and paged causal prefill attention on fp16 MFMA tiles for gfx950.
//
// Replaces batch_prefill_ragged_kv and batch_prefill_paged_kv
// (python/tvm/relax/frontend/nn/llm/_prefill_kernels.py:795-923, :217-391), whose inner
// products are scalar FMAs over 32x32 tiles on a fixed grid of 16 x h_kv blocks.  Numerics
// follow the reference macros (python/tvm/relax/frontend/nn/llm/_kernel_common.py:222-334):
// S = QK^T * sm_scale * log2(e), base-2 online softmax with initial state m = -5e4, d = 1,
// fp32 accumulation, out = O/d rounded once to fp16, lse = m + log2(d); rows are the
// (position, head-in-group) pairs of one kv head, interleaved as row = pos*group + head
// (_prefill_kernels.py:331-332); causal mask col < kv_len - qo_len + row_pos + 1
// (_kernel_common.py:130-135).
//
// Tiling: a workgroup of 4 wavefronts owns 128 rows x one kv head; each wave owns 32 rows, one
// row per lane%32, and keeps Q as MFMA B-fragments in registers.  K/V tiles of 64 tokens are
// copied from global memory straight into LDS (global_load_lds_dwordx4: no staging registers, no
// ds_write), row-major and unpadded, two stages deep, so that tile t+1 lands while tile t is
// multiplied.  Bank conflicts are avoided by an XOR swizzle of the 16-byte pieces of a row; the
// copy applies it on the source side (lane L always fills LDS piece L of the 1 KiB an
// instruction writes, and fetches the global piece that belongs there).  S^T = K Q^T and
// O^T = V^T P^T use v_mfma_f32_32x32x16_f16 with the query on the N axis: all per-query softmax
// state (m, l, the O rescale factor) is lane-local, and the S^T accumulator registers are exactly
// the B-operand of the PV product, so P never leaves registers.  The V^T A-fragments come from
// the row-major V tile through ds_read_b64_tr_b16, which hands each lane four consecutive tokens
// of one feature.
//
// Workgroup -> (sequence, row tile) without a prologue kernel: sequence b owns tile slots
//   [floor(q_indptr[b]*group/128) + b, floor(q_indptr[b+1]*group/128) + b + 1)
// found by binary search on q_indptr; the grid is floor(total_q*group/128) + B slots.
#include <cmath>
#include <type_traits>

#include "prefill_common.cuh"
#include "runtime_support.h"
#include "typed_kernels.h"

namespace tvmkv {

// Pipeline depth: as many stages as fit next to the other workgroups of the CU (NW = 4: one more, two
// more at head dim 64, whose kernels need a third of the registers) or alone (NW = 8).
constexpr int prefill_stages(int dqk, int dv) {
  const int stage_bytes = BN * (dqk + dv) * 2;
  const int budget = (NW == 8 ? 160 : (dqk == 64 ? 53 : 80)) * 1024;
  return budget / stage_bytes >= 4 ? 4 : (budget / stage_bytes >= 3 ? 3 : 2);
}

constexpr size_t prefill_lds_bytes(int dqk, int dv) {
  return static_cast<size_t>(prefill_stages(dqk, dv)) * BN * (dqk + dv) * 2;
}

// EXT = false: plain cache, q and k already rotated (or no RoPE).  EXT = true adds
//  * the sliding-window cache, length_info (3, B): the page table covers `sink` tokens at the front,
//    evicted tokens up to `window_offset`, then the window; keys have logical indices (sink tokens,
//    then window tokens) that the masks and RoPE use
//    (python/tvm/relax/frontend/nn/llm/_kernel_common.py:155-170);
//  * the per-layer sliding-window mask of _kernel_common.py:138-144;
//  * inline RoPE: q at q_rope_position[token], key t at k_rope_pos_offset[b] + t
//    (_prefill_kernels.py:119-147);
//  * the token-tree mask of speculative decoding: the last keys of a sequence are the nodes of its
//    token tree, a query node sees the keys before the tree and its ancestors (tree_attn.py:48-65).
// Attention does not depend on the order of the keys, so the tiles are still walked in physical
// order.  Masks are evaluated per element; only a plain cache without RoPE keeps the unmasked
// path, for the tiles in front of the tree.
// SRC: where the keys come from.  kRagged: k / v rows of the call; kPaged: the page pool; kBoth: the
// cached tokens of the page pool, all visible, followed by the k / v rows of the call under the
// causal mask -- a chunked-prefill step in one pass, on one key axis whose paged part is padded to
// a whole number of tiles (the padding is masked like the end of a sequence).
// STREAM: every K/V row of the launch is read by one row tile only (draft chains and small trees per
// sequence, decode-shaped calls): the tiles are copied with the streaming hint like the decode kernel's
// (a 15-node tree per sequence 0.252 -> 0.231 ms).  Where row tiles share K/V rows the hint costs 2-4 %,
// and choosing the copy at run time inside one kernel cost the shared case 1.5 %.
// PAD: the head dim in memory, p.d_mem (80, 96, 112: a multiple of 16 below the template's), is smaller
// than the tile the kernel computes on.  Rows of q, k, v, the pages and the output keep d_mem elements;
// the q fragments of the missing features are zero, the K/V copies fill the missing 16-byte pieces of a
// row with a repeat of its last piece (finite values that meet zeros in the score product and only reach
// output features that are not stored), and the epilogue stores the first d_mem features.
// VARIANT: the in-kernel RoPE takes a frequency variant (a table entry per element, inverse frequencies, a
// magnitude: rope_pair_ex).  A kernel of its own: the general rotation holds more values than the default one,
// and inside one kernel it made every extended launch spill (67-87 registers at head dim 128).
template <int DQK, int DV, int SRC, int PS, bool EXT, bool STREAM = false, bool PAD = false, bool VARIANT = false>
__global__ __launch_bounds__(NW * 64, (NW == 8 || DQK + DV > 320) ? 1 : (DQK == 64 ? 3 : 2)) void prefill_kernel(PrefillParams p, PrefillRopeDivisors div) {
  constexpr bool PAGED = SRC == kPaged, BOTH = SRC == kBoth;
  static_assert(!PAD || (!EXT && !BOTH && DQK == DV), "padded head dims: plain ragged and paged kernels");
  const int dqm = PAD ? p.d_mem : DQK;  // elements per q / k row in memory
  const int dvm = PAD ? p.d_mem : DV;   // elements per v / output row in memory
  auto copy_kv = [](const void* base, uint32_t off, uint32_t dst) {
    if (STREAM) copy16_to_lds_nt(base, off, dst); else copy16_to_lds(base, off, dst);
  };
  static_assert(!(BOTH && EXT), "the combined pass exists for the plain cache only");
  static_assert(DQK % 64 == 0 && DV % 64 == 0, "feature dims must be multiples of 64");
  constexpr int KS = DQK / 16;                  // k-steps of the QK^T product
  constexpr int DB = DV / 32;                   // 32-wide output feature blocks
  constexpr int TB = BN / 32;                   // 32-token blocks per tile
  constexpr int KW = DQK % 128 == 0 ? 128 : 64; // K is kept as DQK/KW column blocks of width KW
  constexpr int KBLK = DQK / KW;
  constexpr int KCH = KW / 8;                   // 16-byte pieces per row of a K block
  constexpr int VW = DV % 128 == 0 ? 128 : 64;
  constexpr int VBLK = DV / VW;
  constexpr int VCH = VW / 8;
  constexpr int STAGE = BN * (DQK + DV);        // halfs per pipeline stage
  constexpr int NSTAGE = prefill_stages(DQK, DV);
  constexpr int COPIES = (DQK + DV) / 8 / NW;   // copy instructions per wave per tile
  static_assert(SRC == kRagged || PS % 16 == 0, "page size must be a multiple of 16");

  // two stages; the workgroup's 4 waves each copy 16 of the 64 token rows of a tile
  extern __shared__ __attribute__((aligned(16))) half_t lds_tiles[];

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int col = lane & 31;
  const int half = lane >> 5;
  // grid = (h_kv, slots): the kv head is the fastest-varying workgroup index, so with 8 kv heads
  // and 8 XCDs (workgroups are dealt round-robin to XCDs) all row tiles of one head share one L2
  const int kvh = blockIdx.x;
  const int group = p.group;

  // ---- which (sequence, row tile) ---------------------------------------------------------
  // Workgroups are dispatched in the order of their index, and the last ones to start decide when
  // the kernel ends: the sequences are walked from the one with the most keys to the one with the
  // fewest (up to 64 sequences: one lane per sequence ranks them), and inside a sequence from the
  // last row tile to the first, since under the causal mask the last rows see the most keys.
  const int slot = blockIdx.y;
  int b, local_slot;
  // the sequence's entries of the index arrays: from the lanes that ranked the sequences where they
  // did (no second round trip to memory), loaded otherwise
  int seq_q0, seq_q1, seq_p0 = 0, seq_p1 = 0, seq_last = 0, seq_k0 = 0, seq_k1 = 0;
  if (p.batch_size <= 64) {
    int my_tiles = 0, my_key = -1;
    int lq0 = 0, lq1 = 0, lp0 = 0, lp1 = 0, llast = 0, lk0 = 0, lk1 = 0;
    if (lane < p.batch_size) {
      lq0 = p.q_indptr[lane];
      lq1 = p.q_indptr[lane + 1];
      if (PAGED || BOTH) {
        lp0 = p.page_indptr[lane];
        lp1 = p.page_indptr[lane + 1];
        llast = p.last_page_len[lane];
      }
      if (!PAGED) {
        lk0 = p.kv_indptr[lane];
        lk1 = p.kv_indptr[lane + 1];
      }
      my_tiles = ((lq1 - lq0) * group + BM - 1) / BM;
      my_key = (lp1 - lp0) * (PS << p.page_shift) + (lk1 - lk0);
    }
    // Row tiles of the sequences ranked before this lane's.  (key, index) is one sortable 32-bit
    // number (keys beyond 2^24 tokens rank equal), compared without branches, four sequences per
    // round with separate sums: every workgroup runs this loop alone on its SIMDs, one dependent
    // instruction after the other, and with short sequences it is a visible part of its life.
    const int my_rank = min(my_key, (1 << 24) - 1) * 64 + (63 - lane);  // negative for the lanes past the batch
    int begin4[4] = {0, 0, 0, 0};
    for (int j = 0; j < p.batch_size; j += 4) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        // lanes past the batch rank below every sequence and have no tiles
        const int rank_j = __builtin_amdgcn_readlane(my_rank, (j + u) & 63);
        const int tiles_j = __builtin_amdgcn_readlane(my_tiles, (j + u) & 63);
        begin4[u] += rank_j > my_rank ? tiles_j : 0;
      }
    }
    const int my_begin = (begin4[0] + begin4[1]) + (begin4[2] + begin4[3]);
    const uint64_t owner = __ballot(lane < p.batch_size && slot >= my_begin && slot < my_begin + my_tiles);
    if (owner == 0) return;  // the grid is sized from shapes alone and has spare slots
    b = __builtin_amdgcn_readfirstlane(__ffsll(static_cast<long long>(owner)) - 1);
    local_slot = slot - __builtin_amdgcn_readlane(my_begin, b);
    seq_q0 = __builtin_amdgcn_readlane(lq0, b);
    seq_q1 = __builtin_amdgcn_readlane(lq1, b);
    seq_p0 = __builtin_amdgcn_readlane(lp0, b);
    seq_p1 = __builtin_amdgcn_readlane(lp1, b);
    seq_last = __builtin_amdgcn_readlane(llast, b);
    seq_k0 = __builtin_amdgcn_readlane(lk0, b);
    seq_k1 = __builtin_amdgcn_readlane(lk1, b);
  } else {
    // the last sequence whose first slot is at or before this one, by a 64-ary search of the wave: the
    // lanes probe 64 evenly spaced sequences of the range that is left, one round trip to memory per
    // factor of 64 in the batch size (tile_slot_begin is increasing and 0 for sequence 0)
    int lo = 0, n = p.batch_size;
    while (n > 64) {
      const int stride = (n + 63) >> 6;
      const int idx = lo + lane * stride;
      const bool le = idx < lo + n && tile_slot_begin(p.q_indptr, idx, group) <= slot;
      const int first = lo + (__popcll(__ballot(le)) - 1) * stride;
      n = min(stride, lo + n - first);
      lo = first;
    }
    const bool le = lane < n && tile_slot_begin(p.q_indptr, lo + lane, group) <= slot;
    b = __builtin_amdgcn_readfirstlane(lo + max(static_cast<int>(__popcll(__ballot(le))), 1) - 1);
    local_slot = slot - tile_slot_begin(p.q_indptr, b, group);
    seq_q0 = p.q_indptr[b];
    seq_q1 = p.q_indptr[b + 1];
    if (PAGED || BOTH) {
      seq_p0 = p.page_indptr[b];
      seq_p1 = p.page_indptr[b + 1];
      seq_last = p.last_page_len[b];
    }
    if (!PAGED) {
      seq_k0 = p.kv_indptr[b];
      seq_k1 = p.kv_indptr[b + 1];
    }
  }
  const int q_start = seq_q0;
  const int qo_len = seq_q1 - q_start;
  const int rows = qo_len * group;
  const int n_row_tiles = (rows + BM - 1) / BM;
  if (local_slot >= n_row_tiles) return;
  const int r0 = (n_row_tiles - 1 - local_slot) * BM;

  // phys_len: tokens the K/V storage of the sequence covers; kv_len: keys attended to (logical)
  // kBoth: the key axis is [cached tokens, padded to prefix_pad][new tokens]
  int phys_len = 0, kv_start = 0, pbeg = 0, sink = 0, win_lo = 0, prefix_len = 0, prefix_pad = 0;
  if (PAGED || BOTH) {
    pbeg = seq_p0;
    const int npages = seq_p1 - pbeg;
    phys_len = npages > 0 ? (npages - 1) * (PS << p.page_shift) + seq_last : 0;
    if (EXT && p.sink_size != nullptr && npages > 0) {
      sink = p.sink_size[b];
      win_lo = p.window_offset[b];
    }
  }
  if (!PAGED) {
    kv_start = seq_k0;
    if (BOTH) {
      prefix_len = phys_len;
      prefix_pad = (prefix_len + BN - 1) / BN * BN;
    }
    phys_len = prefix_pad + seq_k1 - kv_start;
  }
  const int prefix_tiles = prefix_pad / BN;
  const int hole_tile = (BOTH && prefix_len < prefix_pad) ? prefix_tiles - 1 : -1;  // its end is padding
  const int kv_len = phys_len - win_lo + sink;
  // number of logical keys -> physical end of the tokens that hold them
  auto to_phys = [&](int n) { return (!EXT || n <= sink) ? n : n - sink + win_lo; };
  __shared__ float div_lds[DQK > 256 ? 256 : DQK];
  const bool q_rope = (EXT && p.rotary) || (BOTH && p.q_inline_rope != 0);  // uniform over the launch
  if (q_rope) {
    if (tid < DQK && tid < 256) div_lds[tid] = div.v[tid];
    __syncthreads();
  }

  // ---- this lane's query row -------------------------------------------------------------
  const int my_row = r0 + wave * 32 + col;
  const bool row_valid = my_row < rows;
  const int my_pos = my_row / group;
  const int my_head = kvh * group + my_row % group;
  const int causal_shift = kv_len - qo_len + 1;
  // number of visible kv tokens for this row (logical), and with the per-layer window the first one
  const bool layer_mask = EXT && p.causal && p.layer_window > 0;
  const int my_limit = !row_valid ? 0 : (layer_mask ? kv_len : (p.causal ? min(kv_len, causal_shift + my_pos) : kv_len));
  const int my_lo = layer_mask ? max(kv_len - max(p.layer_window - my_pos - 1, 0), 0) : 0;
  // workgroup- and wave-level bounds (uniform)
  const int last_row_wg = min(rows, r0 + BM) - 1;
  const int kv_end = to_phys((p.causal && !layer_mask) ? max(0, min(kv_len, causal_shift + last_row_wg / group)) : kv_len);
  const int first_row_wave = r0 + wave * 32;
  const int last_row_wave = min(rows, first_row_wave + 32) - 1;  // < first_row_wave if the wave is empty
  const bool wave_active = first_row_wave < rows;
  const bool causal_rows = p.causal && !layer_mask;
  // physical bounds: beyond wave_limit_max nothing is visible to any row of the wave, below
  // wave_limit_min everything is visible to all of them (plain cache only)
  const int wave_limit_max = to_phys(!wave_active ? 0 : (causal_rows ? min(kv_len, causal_shift + last_row_wave / group) : kv_len));
  const int wave_limit_min = !wave_active ? 0 : (causal_rows ? min(kv_len, causal_shift + first_row_wave / group) : kv_len);

  // token tree: keys from tree_start on are tree nodes; this row's node is my_pos + tree_len - qo_len
  int tree_len = 0, tree_start = kv_len, child_first = 0;
  const int32_t* tree_base = nullptr;
  if (EXT && p.tree_order != nullptr) {
    const int first_node = p.tree_indptr[b];
    tree_len = p.tree_indptr[b + 1] - first_node;
    tree_start = kv_len - tree_len;
    tree_base = p.tree_order + 2 * static_cast<int64_t>(first_node);
    if (tree_len > 0) child_first = tree_base[2 * min(max(my_pos + tree_len - qo_len, 0), tree_len - 1)];
  }
  // Tiles whose keys every row of the wave sees need no mask at all.  Plain cache: the tiles that end
  // at or before unmasked_limit.  EXT without in-kernel RoPE: a tile that lies wholly among the attention
  // sinks or wholly in the window, in front of the tree nodes and of the causal bound of the wave's first
  // row, and behind the per-layer window start of its last row (logical key indices ext_lo .. ext_hi).
  const int unmasked_limit = !EXT ? wave_limit_min : 0;
  const bool ext_fast = EXT && !p.rotary;
  const int ext_hi = min(wave_limit_min, max(tree_start, 0));
  const int ext_lo = (layer_mask && wave_active) ? max(kv_len - max(p.layer_window - last_row_wave / group - 1, 0), 0) : 0;

  half8_t qf[KS];
  {
    const int64_t q_token_stride = p.q_token_stride != 0 ? p.q_token_stride : static_cast<int64_t>(p.h_q) * dqm;
    const half_t* qrow = p.q + static_cast<int64_t>(q_start + my_pos) * q_token_stride + my_head * dqm + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = (row_valid && (!PAD || ks * 16 < dqm)) ? ld16(qrow + ks * 16).h8 : zero16().h8;
    if (q_rope && row_valid) {
      const float q_pos = static_cast<float>(p.q_rope_position[q_start + my_pos]) * p.rope_scale;
#pragma unroll
      for (int ks = 0; ks < KS / 2; ++ks) {
        if constexpr (VARIANT) {
          rope_pair_ex(qf[ks], qf[ks + KS / 2], q_pos, div_lds + ks * 16 + half * 8, div_lds + DQK / 2 + ks * 16 + half * 8,
                       p.rope_inverse, p.rope_halves_differ, p.rope_magnitude);
        } else {
          rope_pair(qf[ks], qf[ks + KS / 2], q_pos, div_lds + ks * 16 + half * 8);
        }
      }
    }
  }
  const float k_pos0 = (EXT && p.rotary) ? static_cast<float>(p.k_rope_pos_offset[b]) : 0.f;

  float16_t o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int j = 0; j < 16; ++j) o[db][j] = 0.f;
  }
  float m = kNegInit, lsum = 0.f;

  // ---- tile copy: global -> LDS ---------------------------------------------------------------
  // Rows past the end of the sequence repeat its last token: their scores are masked, and P = 0
  // times a finite V is 0 (unwritten page memory could hold NaN patterns).
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const uint32_t lds_base = static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lds_ptr_t)lds_tiles));
  const int last_tok = BOTH ? prefix_len - 1 : phys_len - 1;               // last row of the (paged) source
  const int last_new = BOTH ? phys_len - prefix_pad - 1 : 0;              // kBoth: last row of k / v
  // Page ids of this wave's RPW rows for 64 consecutive tiles, one tile per lane, fetched once per
  // 64 tiles: the wait for this load also waits for every tile copy in flight, so it must be rare.
  int page_ids = 0;
  const int psh = p.page_shift;
  auto load_page_ids = [&](int first_tile) {
    if (PAGED || BOTH) {
      // a page of PS << page_shift tokens is walked as 1 << page_shift runs of PS tokens: the lane
      // keeps (page id, run inside the page), the run in the low 3 bits
      const int pslot = min((first_tile + lane) * BN + wave_u * RPW, last_tok) / PS;
      page_ids = (p.page_values[pbeg + (pslot >> psh)] << 3) | (pslot & ((1 << psh) - 1));
    }
  };
  // Global addresses are a wave-uniform base (scalar registers) plus a 32-bit byte offset per lane.
  // Ragged: the base is the sequence's first K/V row of this head, the offset token * row stride,
  // so one sequence's K (or V) must stay below 4 GiB.  Paged: the base is the page, the offset the
  // row inside it.
  const half_t* k_seq = PAGED ? nullptr : uniform_ptr(p.k + (static_cast<int64_t>(kv_start) * p.h_kv + kvh) * dqm);
  const half_t* v_seq = PAGED ? nullptr : uniform_ptr(p.v + (static_cast<int64_t>(kv_start) * p.h_kv + kvh) * dvm);
  const uint32_t k_stride_bytes = static_cast<uint32_t>(p.h_kv) * dqm * 2;
  const uint32_t v_stride_bytes = static_cast<uint32_t>(p.h_kv) * dvm * 2;
  // Issues copy instructions [FIRST, FIRST + COUNT) of the wave's COPIES for `tile` (K blocks first,
  // then V), so that the caller can spread them over its arithmetic: a burst of all copies of all
  // waves right after the barrier queues up in front of the one address unit of the CU, and the
  // waves stall in issue instead of computing.
  auto issue_copies = [&](int tile, auto first_c, auto count_c) {
    constexpr int FIRST = decltype(first_c)::value;
    constexpr int COUNT = decltype(count_c)::value;
    const bool from_pages = BOTH ? tile < prefix_tiles : PAGED;  // wave-uniform
    const int kv0 = tile * BN - (from_pages ? 0 : prefix_pad);
    const int last_row = (BOTH && !from_pages) ? last_new : last_tok;
    const uint32_t stage = lds_base + (tile % NSTAGE) * (STAGE * 2);  // LDS byte address
    const half_t* kbase = k_seq;
    const half_t* vbase = v_seq;
    if (from_pages) {
      const int page = __builtin_amdgcn_readlane(page_ids, tile & 63);
      kbase = p.pages + (((static_cast<int64_t>(page >> 3) * 2 * p.h_kv + kvh) << psh) + (page & 7)) * (PS * dqm);
      vbase = kbase + (static_cast<int64_t>(p.h_kv) << psh) * (PS * dqm);
    }
#pragma unroll
    for (int blk = 0; blk < KBLK; ++blk) {
      constexpr int RPI = 64 / KCH;  // rows per instruction
#pragma unroll
      for (int i = 0; i < RPW / RPI; ++i) {
        const int idx = blk * (RPW / RPI) + i;
        if (idx < FIRST || idx >= FIRST + COUNT) continue;
        const int row = wave_u * RPW + i * RPI + lane / KCH;
        int piece = (lane % KCH) ^ k_swizzle<KW>(row);
        if (PAD) piece = min(piece, dqm / 8 - 1);
        const uint32_t t = min(kv0 + row, last_row);
        const uint32_t off = (from_pages ? (t % PS) * (dqm * 2) : __umul24(t, k_stride_bytes)) + (blk * KW + piece * 8) * 2;
        copy_kv(kbase, off, stage + (blk * (BN * KW) + (wave_u * RPW + i * RPI) * KW) * 2);
      }
    }
#pragma unroll
    for (int blk = 0; blk < VBLK; ++blk) {
      constexpr int RPI = 64 / VCH;
#pragma unroll
      for (int i = 0; i < RPW / RPI; ++i) {
        const int idx = DQK / 8 / NW + blk * (RPW / RPI) + i;
        if (idx < FIRST || idx >= FIRST + COUNT) continue;
        const int row = wave_u * RPW + i * RPI + lane / VCH;
        int piece = (lane % VCH) ^ v_swizzle<VW>(row);
        if (PAD) piece = min(piece, dvm / 8 - 1);
        const uint32_t t = min(kv0 + row, last_row);
        const uint32_t off = (from_pages ? (t % PS) * (dvm * 2) : __umul24(t, v_stride_bytes)) + (blk * VW + piece * 8) * 2;
        copy_kv(vbase, off, stage + (BN * DQK + blk * (BN * VW) + (wave_u * RPW + i * RPI) * VW) * 2);
      }
    }
  };
  // The same copies for head dim 128 and a tile whose 64 rows all exist in the source (every tile
  // but the last of a source): nothing to clamp, the wave's 16 rows are one page or 16 consecutive
  // k / v rows, the 4 rows of a copy instruction are selected through the scalar base, and per lane
  // only the row inside the instruction and the swizzled piece remain -- a handful of vector
  // instructions per tile instead of five per copy, and no branches.
  auto issue_full_tile = [&](int tile) {
    const bool from_pages = BOTH ? tile < prefix_tiles : PAGED;  // wave-uniform
    const uint32_t stage = lds_base + (tile % NSTAGE) * (STAGE * 2) + wave_u * (RPW * 128 * 2);
    const half_t* kbase;
    const half_t* vbase;
    uint32_t row_bytes;
    if (from_pages) {
      const int page = __builtin_amdgcn_readlane(page_ids, tile & 63);
      kbase = p.pages + (((static_cast<int64_t>(page >> 3) * 2 * p.h_kv + kvh) << psh) + (page & 7)) * (PS * 128);
      vbase = kbase + (static_cast<int64_t>(p.h_kv) << psh) * (PS * 128);
      row_bytes = 256;
    } else {
      const int64_t first_row = static_cast<int64_t>(tile) * BN - prefix_pad + wave_u * RPW;
      kbase = k_seq + first_row * p.h_kv * 128;
      vbase = v_seq + first_row * p.h_kv * 128;
      row_bytes = k_stride_bytes;
    }
    const uint32_t row_off = (lane >> 4) * row_bytes;
    const uint32_t k_piece = (lane & 15) ^ (lane >> 4);              // copy i: ^ (i << 2), see k_swizzle
    const uint32_t v_off = row_off + (((lane & 15) ^ (((lane >> 4) & 3) << 2)) << 4);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      copy_kv(kbase + static_cast<int64_t>(i) * 2 * row_bytes, row_off + ((k_piece ^ (i << 2)) << 4),
              stage + i * (4 * 128 * 2));
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      copy_kv(vbase + static_cast<int64_t>(i) * 2 * row_bytes, v_off, stage + BN * 128 * 2 + i * (4 * 128 * 2));
    }
  };
  auto issue_tile = [&](int tile) {
    if ((PAGED || (BOTH && tile < prefix_tiles)) && (tile & 63) == 0) load_page_ids(tile);
    if constexpr (DQK == 128 && DV == 128 && NW == 4 && PS == 16 && !PAD) {
      const bool from_pages = BOTH ? tile < prefix_tiles : PAGED;
      const int rows_left = from_pages ? last_tok + 1 - tile * BN : (BOTH ? last_new + 1 - (tile * BN - prefix_pad)
                                                                          : last_tok + 1 - tile * BN);
      if (rows_left >= BN) {  // wave-uniform
        issue_full_tile(tile);
        return;
      }
    }
    issue_copies(tile, std::integral_constant<int, 0>{}, std::integral_constant<int, COPIES>{});
  };

  // ---- per-lane fragment addressing (halfs, relative to the K / V part of a stage) -----------
  // K A-fragment of k-step ks, token block tb: row tb*32 + col, features ks*16 + half*8 .. +7
  const int k_swz = k_swizzle<KW>(col);  // same for col + 32
  // V^T A-fragment via the transposing read: lane li of a 16-lane group points at 4 features of
  // token (li >> 2) of the group's 4 tokens; the group as a whole covers 16 features, and lane li
  // receives feature li of them for the 4 tokens.
  const int li = lane & 15;
  const int gg = (lane >> 4) & 1;
  const int v_row = half * 4 + (li >> 2);           // + tb*32 + kk*16 + {0, 8}
  const int v_swz = v_swizzle<VW>(v_row);           // the added terms are multiples of 8
  const int v_lane_off = v_row * VW + (li & 1) * 4; // halfs

  auto read_k = [&](const half_t* Ks, int tb, half8_t (&kf)[KS]) {
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      constexpr int SPB = KW / 16;  // k-steps per column block
      const int piece = ((ks % SPB) * 2 + half) ^ k_swz;
      kf[ks] = *reinterpret_cast<const half8_t*>(Ks + (ks / SPB) * (BN * KW) + (tb * 32 + col) * KW + piece * 8);
    }
  };
  // contraction slot half*8+i of fragment kk holds token kk*16 + (i/4)*8 + half*4 + i%4 of the block,
  // the order in which the S^T accumulator registers hold the tokens
  auto read_v = [&](const half_t* Vs, int tb, half8_t (&vf)[DB][2]) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      constexpr int BPB = VW / 32;  // feature blocks per column block
      const int piece = (((db % BPB) * 4 + gg * 2 + ((li & 3) >> 1)) ^ v_swz);
      const half_t* vp = Vs + (db / BPB) * (BN * VW) + v_lane_off + piece * 8 + tb * 32 * VW;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const half4_t lo = lds_read_tr16(vp + (kk * 16) * VW);
        const half4_t hi = lds_read_tr16(vp + (kk * 16 + 8) * VW);
        vf[db][kk][0] = lo[0]; vf[db][kk][1] = lo[1]; vf[db][kk][2] = lo[2]; vf[db][kk][3] = lo[3];
        vf[db][kk][4] = hi[0]; vf[db][kk][5] = hi[1]; vf[db][kk][6] = hi[2]; vf[db][kk][7] = hi[3];
      }
    }
  };
  // S^T = K Q^T for one 32-token block
  auto qk = [&](const half8_t (&kf)[KS]) -> float16_t {
    float16_t acc;
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], qf[ks], acc, 0, 0, 0);
    return acc;
  };
  // online softmax, lane-local per query; the scale is folded into the exponent: p = exp2(s*scale - m)
  auto row_max = [&](const float16_t& acc) -> float {
    float mx = -3.0e38f;
#pragma unroll
    for (int j = 0; j < 16; ++j) mx = fmaxf(mx, acc[j]);
    return max_xor32(mx);
  };
  // The reference point m of the running softmax only has to bound the scores from above up to a
  // factor that fp16 holds comfortably: it moves when a row's maximum exceeds it by more than
  // kMaxSlack (p <= 2^kMaxSlack), so that after the first tiles almost no block rescales O.  Softmax
  // is invariant to the shift, and p is rounded to fp16 with the same relative precision.
  constexpr float kMaxSlack = 8.0f;
  auto advance_max = [&](float mx_raw) -> float {  // returns the factor that rescales the old state
    // a fully masked row keeps its old maximum (the scaled sentinel is far below -5e4)
    const float cand = fmaxf(mx_raw * p.scale_log2, -1.0e30f);
    const float m_new = cand > m + kMaxSlack ? cand : m;
    const float alpha = fast_exp2(m - m_new);
    m = m_new;
    lsum *= alpha;
    return alpha;
  };
  auto rescale = [&](float alpha) {
    if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.0f))) {  // wave-uniform: skip when no maximum moved
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int j = 0; j < 16; ++j) o[db][j] *= alpha;
      }
    }
  };
  auto probs = [&](const float16_t& acc, half8_t (&pf)[2]) {  // uses the current m
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float pj = fast_exp2(fmaf(acc[j], p.scale_log2, -m));  // masked: exp2(-3e38*scale - m) = 0
      lsum += pj;
      pf[j >> 3][j & 7] = static_cast<half_t>(pj);
    }
  };
  // O^T += V^T P^T for one 32-token block
  auto pv = [&](const half8_t (&vf)[DB][2], const half8_t (&pf)[2]) {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[db][kk], pf[kk], o[db], 0, 0, 0);
    }
  };

  // This workgroup's key tiles [tile_lo, n_tiles): all of the row tile's, or its share of them
  int tile_lo = 0, n_tiles = (kv_end + BN - 1) / BN;
  if (SRC != kRagged && p.kv_splits > 1) {  // (ragged launches are never split)
    const int per_split = (n_tiles + p.kv_splits - 1) / p.kv_splits;
    tile_lo = min(static_cast<int>(blockIdx.z) * per_split, n_tiles);
    n_tiles = min(tile_lo + per_split, n_tiles);
    // the page ids are held for windows of 64 tiles that start at multiples of 64
    if ((PAGED || (BOTH && tile_lo < prefix_tiles)) && (tile_lo & 63) != 0 && tile_lo < n_tiles) load_page_ids(tile_lo & ~63);
  }
  // Tiles tile .. tile+NSTAGE-2 are in flight or landed at the top of iteration `tile`.
#pragma unroll
  for (int s = 0; s < NSTAGE - 1; ++s) {
    if (tile_lo + s < n_tiles) issue_tile(tile_lo + s);
  }
  for (int tile = tile_lo; tile < n_tiles; ++tile) {
    const int kv0 = tile * BN;
    const half_t* Ks = lds_tiles + (tile % NSTAGE) * STAGE;
    const half_t* Vs = Ks + BN * DQK;
    // Wait until this wave's part of the tile has landed (copies complete in order, so it is enough
    // that no more than the later tiles' copies are outstanding); after the barrier everyone's
    // has, and every wave is done reading the stage of tile-1, which the next copy overwrites.
    // Copies complete in order, so it is enough that no more than the later tiles' copies (the
    // NSTAGE-2 iterations before this one issued COPIES each, where those tiles exist) are
    // outstanding.  The count passed to s_waitcnt must never exceed what was really issued.
    if (NSTAGE > 2 && tile + NSTAGE - 2 < n_tiles) {
      wait_vmcnt<(NSTAGE - 2) * COPIES>();
    } else {
      wait_vmcnt<0>();
    }
    __syncthreads();
    // no prefetch across a 64-tile window of page ids: the ids held are those of the last copy issued
    const int next = tile + NSTAGE - 1;  // the tile whose copy this iteration issues
    const bool has_next = next < n_tiles;
    // bounds of this tile: those of the wave and the lane, except in the tile that ends in the
    // padding between the cached and the new tokens, which ends at the last cached token for all
    const bool hole = BOTH && tile == hole_tile;
    const int t_limit_max = hole ? (wave_active ? prefix_len : 0) : wave_limit_max;
    const int t_limit_min = hole ? t_limit_max : wave_limit_min;
    const int t_my_limit = hole ? (row_valid ? prefix_len : 0) : my_limit;
    bool unmasked = TB == 2 && kv0 < t_limit_max && kv0 + BN <= (hole ? t_limit_max : unmasked_limit);  // wave-uniform
    if (EXT) {
      const bool in_sink = kv0 + BN <= sink;
      const bool in_window = kv0 >= win_lo && kv0 + BN <= phys_len;
      const int first_key = in_sink ? kv0 : kv0 - win_lo + sink;  // logical index of the tile's first key
      unmasked = TB == 2 && ext_fast && kv0 < t_limit_max && (in_sink || in_window) && first_key >= ext_lo &&
                 first_key + BN <= ext_hi;
    }
    if (has_next) issue_tile(next);

    if (kv0 >= t_limit_max) continue;  // wave-uniform: every row of this wave is masked out

    // The two 32-token halves of a tile, software-pipelined so that the wave's own matrix and vector
    // work overlap: S1 = K1 Q^T runs under the softmax of S0, and O += V0 P0 under the softmax of S1.
    // MASKED: rows of the wave see different parts of the tile (plain cache: the tiles on the causal
    // diagonal and at the end of a source), each lane masks its row's scores against its own bound.
    auto two_halves = [&](auto masked_c) {
      constexpr bool MASKED = decltype(masked_c)::value;
      auto mask = [&](float16_t& acc, int t0) {
        const int rel = t_my_limit - t0 - half * 4;  // element j is token t0 + half*4 + (j/4)*8 + j%4
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] = ((j >> 2) * 8 + (j & 3)) < rel ? acc[j] : -3.0e38f;
      };
      half8_t kf[KS];
      half8_t vf[DB][2];
      half8_t pf[2];
      read_k(Ks, 0, kf);
      __builtin_amdgcn_sched_barrier(0);
      float16_t s0 = qk(kf);
      read_k(Ks, 1, kf);
      read_v(Vs, 0, vf);
      if (MASKED) mask(s0, kv0);
      const float a0 = advance_max(row_max(s0));
      rescale(a0);
      __builtin_amdgcn_sched_barrier(0);
      float16_t s1 = qk(kf);
      probs(s0, pf);
      interleave_mfma_valu<KS>();
      __builtin_amdgcn_sched_barrier(0);
      if (MASKED) mask(s1, kv0 + 32);
      const float a1 = advance_max(row_max(s1));
      pv(vf, pf);
      probs(s1, pf);
      interleave_mfma_valu<2 * DB>();
      __builtin_amdgcn_sched_barrier(0);
      read_v(Vs, 1, vf);
      rescale(a1);
      pv(vf, pf);
    };
    if constexpr (DQK <= 128) {
      if (unmasked) {  // every row of the wave sees the whole tile (all tiles left of the causal diagonal)
        two_halves(std::false_type{});
        continue;
      }
      if constexpr (!EXT && TB == 2) {
        if (kv0 + 32 < t_limit_max) {  // wave-uniform: both halves hold keys that some row sees
          two_halves(std::true_type{});
          continue;
        }
      }
    } else if (unmasked) {
      // d_qk 192 has no register to spare: the same unmasked pipeline written out, which the compiler
      // allocates without spilling (as a call of the generic form above it spills ten registers)
      half8_t kf[KS];
      half8_t vf[DB][2];
      half8_t pf[2];
      read_k(Ks, 0, kf);
      __builtin_amdgcn_sched_barrier(0);
      float16_t s0 = qk(kf);
      read_k(Ks, 1, kf);
      read_v(Vs, 0, vf);
      const float a0 = advance_max(row_max(s0));
      rescale(a0);
      __builtin_amdgcn_sched_barrier(0);
      float16_t s1 = qk(kf);
      probs(s0, pf);
      interleave_mfma_valu<KS>();
      __builtin_amdgcn_sched_barrier(0);
      const float a1 = advance_max(row_max(s1));
      pv(vf, pf);
      probs(s1, pf);
      interleave_mfma_valu<2 * DB>();
      __builtin_amdgcn_sched_barrier(0);
      read_v(Vs, 1, vf);
      rescale(a1);
      pv(vf, pf);
      continue;
    }

    // Tiles on the causal diagonal or at the end of the sequence: one 32-token block at a time,
    // masked.  The LDS reads of a block are issued in two batches ahead of their MFMAs (K
    // fragments, then the V^T fragments, whose latency hides behind the softmax arithmetic).
#pragma unroll
    for (int tb = 0; tb < TB; ++tb) {
      const int t0 = kv0 + tb * 32;
      if (t0 >= t_limit_max) break;  // wave-uniform
      half8_t kf[KS];
      half8_t vf[DB][2];
      half8_t pf[2];
      read_k(Ks, tb, kf);
      if (EXT && p.rotary) {
        // this lane's key row is physical token t0 + col; its logical index is its position
        const int t = min(t0 + col, last_tok);
        const int logical = t < sink ? t : t - win_lo + sink;
        float pos = (k_pos0 + static_cast<float>(logical)) * p.rope_scale;
        if (!PAGED && p.k_pos_from_q) pos = static_cast<float>(p.q_rope_position[kv_start + t]) * p.rope_scale;
#pragma unroll
        for (int ks = 0; ks < KS / 2; ++ks) {
          if constexpr (VARIANT) {
            rope_pair_ex(kf[ks], kf[ks + KS / 2], pos, div_lds + ks * 16 + half * 8, div_lds + DQK / 2 + ks * 16 + half * 8,
                         p.rope_inverse, p.rope_halves_differ, p.rope_magnitude);
          } else {
            rope_pair(kf[ks], kf[ks + KS / 2], pos, div_lds + ks * 16 + half * 8);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      float16_t acc = qk(kf);
      read_v(Vs, tb, vf);
      __builtin_amdgcn_sched_barrier(0);
      if (EXT) {
        // element j is physical token t0 + half*4 + (j/4)*8 + j%4
        const int block_last = t0 + 31;
        const bool in_tree = tree_len > 0 && (block_last < sink ? block_last : block_last - win_lo + sink) >= tree_start;  // wave-uniform
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const int t = t0 + half * 4 + (j >> 2) * 8 + (j & 3);
          const bool cached = t < sink || (t >= win_lo && t < phys_len);
          const int logical = t < sink ? t : t - win_lo + sink;
          bool visible = cached && logical < my_limit && logical >= my_lo;
          if (in_tree) {
            const int node = min(max(logical - tree_start, 0), tree_len - 1);
            const int first = tree_base[2 * node], second = tree_base[2 * node + 1];
            visible = visible && (logical < tree_start || (child_first >= first && child_first < second));
          }
          acc[j] = visible ? acc[j] : -3.0e38f;
        }
      } else if (t0 + 32 > t_limit_min) {  // wave-uniform
        asm volatile("" ::: "memory");  // keep this a branch: if-converted it costs 5 ops per element everywhere
        const int rel = t_my_limit - t0 - half * 4;  // element j is token t0 + half*4 + (j/4)*8 + j%4
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] = ((j >> 2) * 8 + (j & 3)) < rel ? acc[j] : -3.0e38f;
      }
      rescale(advance_max(row_max(acc)));
      probs(acc, pf);
      pv(vf, pf);
    }
  }

  // ---- epilogue ------------------------------------------------------------------------------
  lsum = sum_xor32(lsum);
  const float denom = lsum + fast_exp2(kNegInit - m);  // the d = 1 of the initial state
  if (row_valid) {
    const float inv = 1.0f / denom;
    const int64_t out_row = (SRC != kRagged && p.kv_splits > 1 ? blockIdx.z * p.split_rows : 0) + static_cast<int64_t>(q_start + my_pos) * p.h_q + my_head;
    half_t* orow = p.output + out_row * dvm + half * 4;
    float* lse_ptr = p.lse + out_row;
    const float my_lse = m + fast_log2(denom);
    if (p.merge_into) {
      // python/tvm/relax/frontend/nn/llm/_decode_kernels.py:441-450 with (v, s) = what the arrays
      // hold and (v_other, s_other) = this kernel's state; both lanes of a row read s before lane
      // `half == 0` overwrites it (one wavefront, program order)
      const float s_prev = *lse_ptr;
      const float s_max = fmaxf(s_prev, my_lse);
      const float w_prev = fast_exp2(s_prev - s_max);
      const float w_mine = fast_exp2(my_lse - s_max);
      const float scale_prev = w_prev / (w_prev + w_mine);
      const float scale_mine = w_mine / (w_prev + w_mine) * inv;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4) {
          if (PAD && db * 32 + j4 * 8 >= dvm) continue;
          half4_t* dst = reinterpret_cast<half4_t*>(orow + db * 32 + j4 * 8);
          const half4_t prev = *dst;
          half4_t out4;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            out4[e] = static_cast<half_t>(static_cast<float>(prev[e]) * scale_prev + o[db][j4 * 4 + e] * scale_mine);
          }
          *dst = out4;
        }
      }
      if (half == 0) *lse_ptr = fast_log2(w_prev + w_mine) + s_max;
    } else {
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int j4 = 0; j4 < 4; ++j4) {
          if (PAD && db * 32 + j4 * 8 >= dvm) continue;
          half4_t out4;
#pragma unroll
          for (int e = 0; e < 4; ++e) out4[e] = static_cast<half_t>(o[db][j4 * 4 + e] * inv);
          *reinterpret_cast<half4_t*>(orow + db * 32 + j4 * 8) = out4;
        }
      }
      if (half == 0) *lse_ptr = my_lse;
    }
  }
}

// Page sizes the paged kernels take: 16 << shift tokens, walked as 1 << shift runs of 16.  -1: not built.
static int paged_page_shift(int32_t page_size) {
  if (page_size < 16 || page_size > 128 || (page_size & (page_size - 1)) != 0) return -1;
  int shift = 0;
  while ((16 << shift) < page_size) ++shift;
  return shift;
}

template <int DQK, int DV, int SRC, int PS, bool EXT, bool STREAM = false, bool PAD = false, bool VARIANT = false>
static void launch_prefill_ext(const PrefillParams& p, int64_t total_q, const PrefillRopeDivisors& div,
                               hipStream_t stream) {
  const int64_t slots = total_q * p.group / BM + p.batch_size;
  if (slots >= 65536) throw Error(TVMKV_EINVAL, "prefill: too many row tiles for one launch");
  constexpr size_t lds_bytes = prefill_lds_bytes(DQK, DV);
  static bool attr_set = false;  // per instantiation; the attribute is per function, not per device
  if (lds_bytes > 48 * 1024 && !attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&prefill_kernel<DQK, DV, SRC, PS, EXT, STREAM, PAD, VARIANT>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    attr_set = true;
  }
  hipLaunchKernelGGL((prefill_kernel<DQK, DV, SRC, PS, EXT, STREAM, PAD, VARIANT>),
                     dim3(p.h_kv, static_cast<unsigned>(slots), static_cast<unsigned>(std::max(1, p.kv_splits))),
                     dim3(NW * 64), lds_bytes, stream, p, div);
}

// ---- split over the keys ---------------------------------------------------------------------
// A launch with few row tiles and long key ranges (a token tree or a short chunk against long cached
// sequences) neither fills the chip nor balances it: a row tile is one workgroup that walks all its
// keys.  Such a launch is split: kv_splits workgroups share a row tile, each writes the attention state
// of its share of the key tiles (normalised output in fp16, lse) to scratch memory, and a second kernel
// merges the states of a row with the arithmetic of merge_state_inplace
// (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:441-450) over kv_splits states at once.  A row
// whose states are all empty (lse = -5e4) stays the empty state: out 0, lse -5e4.
template <int DV>
__global__ __launch_bounds__(256) void prefill_split_merge_kernel(const half_t* __restrict__ part_o,
                                                                  const float* __restrict__ part_lse, half_t* __restrict__ output,
                                                                  float* __restrict__ lse, int64_t rows, int splits,
                                                                  int merge_into) {
  constexpr int TPR = DV / 8;  // threads per row, 8 features each
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (256 / TPR) + threadIdx.x / TPR;
  const int piece = threadIdx.x % TPR;
  if (row >= rows) return;
  // the shares' loads do not depend on each other: unrolled, eight are in flight at once (64 shares of a
  // 64-token chunk: 35 us as a loop of dependent round trips)
  float s_max = kNegInit;
#pragma unroll 8
  for (int i = 0; i < splits; ++i) s_max = fmaxf(s_max, part_lse[i * rows + row]);
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  float w_sum = 0.f;
  const bool any_share = s_max > kNegInit;
  if (merge_into) {
    // output / lse already hold a state of the same rows (the launch was asked to merge into it): it is one more
    // state of the sum; shares that are all empty count as the one empty state (out 0, lse -5e4) an unsplit
    // launch would have merged
    const float s_prev = lse[row];
    s_max = fmaxf(s_max, s_prev);
    const float w = fast_exp2(s_prev - s_max);
    const Vec16 v = ld16(output + row * DV + piece * 8);
    w_sum = w + (any_share ? 0.f : fast_exp2(kNegInit - s_max));
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = w * static_cast<float>(v.h8[e]);
  }
  if (any_share) {
#pragma unroll 8
    for (int i = 0; i < splits; ++i) {
      const float w = fast_exp2(part_lse[i * rows + row] - s_max);
      const Vec16 v = ld16(part_o + (i * rows + row) * DV + piece * 8);
      w_sum += w;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += w * static_cast<float>(v.h8[e]);
    }
  }
  const float inv = w_sum > 0.f ? 1.0f / w_sum : 0.f;
  Vec16 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) out.h8[e] = static_cast<half_t>(acc[e] * inv);
  *reinterpret_cast<Vec16*>(output + row * DV + piece * 8) = out;
  if (piece == 0) lse[row] = w_sum > 0.f ? s_max + fast_log2(w_sum) : kNegInit;
}

// How many ways to split the keys of a launch of total_q query tokens in `batch` sequences whose
// sequences hold avg_keys keys on average (shapes only: no read of the index arrays).  The launch has at
// least max(total_q * group / BM, batch) row tiles, times h_kv workgroups, and the chip holds two
// workgroups per compute unit.
//  * Less than half a round of workgroups: as many shares as fill two rounds.
//  * Up to one round, of row tiles that are at most half full (a draft chain or a small tree per
//    sequence): the K/V stream decides and two shares balance it (64 sequences of 1024-8192 keys with a
//    4-token chain each: 0.241 ms unsplit, 0.217 with 2 shares, 0.226 with 4, 0.239 with 8).
//  * Otherwise none: workgroups that end early leave their compute unit to the one that shares it, and
//    shares only add start-up, epilogue and merge traffic (16 sequences with 128-token chunks on
//    2000-6000 keys, 512 workgroups: 0.171 ms unsplit, 0.183 with 2 shares; a 63-node tree per sequence,
//    1008 workgroups, matrix-bound: 0.409 against 0.442).
// No share shorter than 8 tiles on average, at most 64 shares.
static int pick_kv_splits(int64_t total_q, int group, int batch, int h_kv, int64_t avg_keys) {
  const int64_t forced = option(kOptPrefillKvSplits);
  if (forced > 0) return static_cast<int>(std::min<int64_t>(forced, 64));
  const int64_t resident = static_cast<int64_t>(compute_units()) * 2;
  const int64_t tiles = std::max<int64_t>((total_q * group + BM - 1) / BM, batch);
  const int64_t workgroups = tiles * h_kv;
  int64_t want = 1;
  if (workgroups * 2 <= resident) {
    want = (2 * resident + workgroups - 1) / workgroups;
  } else if (workgroups <= resident && total_q * group * 2 <= tiles * BM) {
    want = 2;
  }
  const int64_t by_length = avg_keys / (8 * BN);
  return static_cast<int>(std::max<int64_t>(1, std::min<int64_t>(std::min(want, by_length), 64)));
}

// Redirects the launch described by p to scratch memory when it is to be split; finish() merges.
struct KvSplit {
  half_t* output;
  float* lse;
  int64_t rows;
  int splits;
  int merge_into = 0;
  ScratchLease lease{};
  KvSplit(PrefillParams& p, int64_t total_q, int64_t avg_keys, int dv, hipStream_t stream)
      : output(p.output), lse(p.lse), rows(total_q * p.h_q), splits(1) {
    // at most one row tile per (sequence, kv head) on average: the paged kernels stream the K/V rows
    p.stream_kv = total_q * p.group <= static_cast<int64_t>(p.batch_size) * BM;
    splits = pick_kv_splits(total_q, p.group, p.batch_size, p.h_kv, avg_keys);
    if (dv % 64 != 0) splits = 1;  // padded head dims (80, 96, 112): the merge kernel is not built for their rows
    if (splits <= 1) return;
    const size_t o_bytes = static_cast<size_t>(splits) * rows * dv * sizeof(half_t);
    const size_t lse_bytes = static_cast<size_t>(splits) * rows * sizeof(float);
    lease = lease_scratch(kScratchPrefill, stream, o_bytes + lse_bytes, 0);  // held until the merge is enqueued
    char* ws = lease.ptr;
    p.output = reinterpret_cast<half_t*>(ws);
    p.lse = reinterpret_cast<float*>(ws + o_bytes);
    p.kv_splits = splits;
    p.split_rows = rows;
    merge_into = p.merge_into;  // the shares write plain states; the merge kernel folds the caller's state in
    p.merge_into = 0;
  }
  void finish(const PrefillParams& p, int dv, hipStream_t stream) const {
    if (splits <= 1) return;
    KV_LAUNCH_CHECK();
    const unsigned rows_per_block = 256 / (dv / 8);
    const dim3 grid(static_cast<unsigned>((rows + rows_per_block - 1) / rows_per_block));
    if (dv == 128) {
      hipLaunchKernelGGL(prefill_split_merge_kernel<128>, grid, dim3(256), 0, stream, p.output, p.lse, output, lse, rows, splits, merge_into);
    } else if (dv == 64) {
      hipLaunchKernelGGL(prefill_split_merge_kernel<64>, grid, dim3(256), 0, stream, p.output, p.lse, output, lse, rows, splits, merge_into);
    } else {
      hipLaunchKernelGGL(prefill_split_merge_kernel<256>, grid, dim3(256), 0, stream, p.output, p.lse, output, lse, rows, splits, merge_into);
    }
  }
};

// The extended kernels (sliding-window cache, per-layer window, inline RoPE) exist for the head
// dims that RoPE models use here; d_qk 192 / d_v 128 is the MLA self-attention, which has neither.
// scaling: the frequency variant of the in-kernel RoPE (NULL: default); used when the launch rotates at all
template <int DQK, int DV, int SRC, int PS>
static void launch_prefill(const PrefillParams& params, int64_t total_q, bool ext, double rope_theta, hipStream_t stream,
                           const tvmkv_rope_scaling* scaling = nullptr) {
  PrefillRopeDivisors div{};
  PrefillParams p = params;
  p.rope_magnitude = 1.0f;
  auto fill_table = [&]() {
    if constexpr (DQK <= 256) {
      const InlineRopeHost table = inline_rope_table(scaling, DQK, rope_theta);
      for (int i = 0; i < DQK; ++i) div.v[i] = table.v[i];
      p.rope_inverse = table.inverse;
      p.rope_halves_differ = table.halves_differ;
      p.rope_magnitude = table.magnitude;
    }
  };
  if (!ext) {
    if (p.q_inline_rope) fill_table();
    if constexpr (SRC == kPaged) {
      if (p.stream_kv) {
        launch_prefill_ext<DQK, DV, SRC, PS, false, true>(p, total_q, div, stream);
        return;
      }
    }
    launch_prefill_ext<DQK, DV, SRC, PS, false>(p, total_q, div, stream);
    return;
  }
  if constexpr (DQK == DV && SRC != kBoth) {
    if (p.rotary) fill_table();
    // the default frequencies (one divisor per pair, position / divisor) have the kernel without the general rotation
    const bool variant = p.rotary && (p.rope_inverse != 0 || p.rope_halves_differ != 0 || p.rope_magnitude != 1.0f);
    if constexpr (SRC == kPaged) {
      if (p.stream_kv) {
        if (variant) {
          launch_prefill_ext<DQK, DV, SRC, PS, true, true, false, true>(p, total_q, div, stream);
        } else {
          launch_prefill_ext<DQK, DV, SRC, PS, true, true>(p, total_q, div, stream);
        }
        return;
      }
    }
    if (variant) {
      launch_prefill_ext<DQK, DV, SRC, PS, true, false, false, true>(p, total_q, div, stream);
    } else {
      launch_prefill_ext<DQK, DV, SRC, PS, true>(p, total_q, div, stream);
    }
  } else {
    throw Error(TVMKV_EUNSUPPORTED, "prefill: inline RoPE / sliding window are not built for this head shape");
  }
}

// Head dims 80, 96 and 112: the head dim 128 kernel on rows of d elements (plain cache, no in-kernel RoPE)
static bool padded_head_dim(int d) { return d == 80 || d == 96 || d == 112; }

template <int SRC>
static void launch_prefill_padded(PrefillParams p, int64_t total_q, int d, bool ext, const char* what, hipStream_t stream) {
  if (ext) {
    throw Error(TVMKV_EUNSUPPORTED, std::string(what) + ": head_dim " + std::to_string(d) +
                                        " is built for the plain cache only (no sliding window, inline RoPE or token tree)");
  }
  p.d_mem = d;
  launch_prefill_ext<128, 128, SRC, 16, false, false, true>(p, total_q, PrefillRopeDivisors{}, stream);
}

}  // namespace tvmkv

using namespace tvmkv;

extern "C" {

static int ragged_prefill(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                          const int32_t* kv_indptr, const int32_t* q_rope_position,
                          const int32_t* k_rope_pos_offset, void* output, float* lse, int64_t causal,
                          int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                          int32_t batch_size, int64_t total_q, int32_t h_q, int32_t h_kv, int32_t d_qk,
                          int32_t d_v, const tvmkv_rope_scaling* scaling, void* stream) {
  // head dims the tuned kernel is not built for (80 / 96 / 112 with RoPE inside the kernel among them): the generic
  // matrix-core kernel
  if (d_qk == d_v && !(rotary_mode == 0 ? tuned_head_dim(d_qk) : (d_qk == 64 || d_qk == 128 || d_qk == 256))) {
    GenericAttention a;
    a.what = "batch_prefill_ragged_kv";
    a.rotary_mode = rotary_mode;
    a.q_rope_position = q_rope_position;
    a.k_rope_pos_offset = k_rope_pos_offset;
    a.rope_scale = rope_scale;
    a.rope_theta = rope_theta;
    a.rope_scaling = scaling;
    a.q = q;
    a.q_indptr = q_indptr;
    a.k = k;
    a.v = v;
    a.kv_indptr = kv_indptr;
    a.out = output;
    a.lse = lse;
    a.total_q = total_q;
    a.batch = batch_size;
    a.h_q = h_q;
    a.h_kv = h_kv;
    a.d = d_qk;
    a.causal = causal > 0;
    a.sm_scale = sm_scale;
    return generic_attention(a, stream);
  }
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0)
      << "batch_prefill_ragged_kv: bad shape";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && k && v && kv_indptr && output && lse) << "batch_prefill_ragged_kv: NULL tensor";
  KV_CHECK(rotary_mode == 0 || (q_rope_position && k_rope_pos_offset))
      << "batch_prefill_ragged_kv: inline RoPE needs the position arrays";
  PrefillParams p{};
  p.q = static_cast<const half_t*>(q);
  p.q_indptr = q_indptr;
  p.k = static_cast<const half_t*>(k);
  p.v = static_cast<const half_t*>(v);
  p.kv_indptr = kv_indptr;
  p.output = static_cast<half_t*>(output);
  p.lse = lse;
  p.batch_size = batch_size;
  p.h_q = h_q;
  p.h_kv = h_kv;
  p.group = h_q / h_kv;
  p.causal = causal > 0;
  p.scale_log2 = static_cast<float>(sm_scale) * kLog2e;
  p.rotary = rotary_mode != 0;
  p.rope_scale = static_cast<float>(rope_scale);
  p.q_rope_position = q_rope_position;
  p.k_rope_pos_offset = k_rope_pos_offset;
  const bool ext = p.rotary != 0;
  hipStream_t s = as_stream(stream);
  if (d_qk == 128 && d_v == 128) {
    launch_prefill<128, 128, kRagged, 16>(p, total_q, ext, rope_theta, s, scaling);
  } else if (d_qk == 64 && d_v == 64) {
    launch_prefill<64, 64, kRagged, 16>(p, total_q, ext, rope_theta, s, scaling);
  } else if (d_qk == 256 && d_v == 256) {
    launch_prefill<256, 256, kRagged, 16>(p, total_q, ext, rope_theta, s, scaling);
  } else if (d_qk == 192 && d_v == 128) {
    launch_prefill<192, 128, kRagged, 16>(p, total_q, ext, rope_theta, s);
  } else if (d_qk == d_v && padded_head_dim(d_qk)) {
    launch_prefill_padded<kRagged>(p, total_q, d_qk, ext, "batch_prefill_ragged_kv", s);
  } else {
    KV_UNSUPPORTED(true) << "batch_prefill_ragged_kv: (d_qk, d_v) = (" << d_qk << ", " << d_v
                         << ") is not built ((64,64), (80,80), (96,96), (112,112), (128,128), (192,128), (256,256))";
  }
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_batch_prefill_ragged_kv(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                  const int32_t* kv_indptr, const int32_t* q_rope_position,
                                  const int32_t* k_rope_pos_offset, void* output, float* lse, int64_t causal,
                                  int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                  int32_t batch_size, int64_t total_q, int32_t h_q, int32_t h_kv, int32_t d_qk,
                                  int32_t d_v, void* stream) {
  return ragged_prefill(q, q_indptr, k, v, kv_indptr, q_rope_position, k_rope_pos_offset, output, lse, causal, rotary_mode,
                        rope_scale, rope_theta, sm_scale, batch_size, total_q, h_q, h_kv, d_qk, d_v, nullptr, stream);
}

int tvmkv_batch_prefill_ragged_kv_scaled(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                         const int32_t* kv_indptr, const int32_t* q_rope_position,
                                         const int32_t* k_rope_pos_offset, void* output, float* lse, int64_t causal,
                                         int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                         int32_t batch_size, int64_t total_q, int32_t h_q, int32_t h_kv, int32_t d_qk,
                                         int32_t d_v, const tvmkv_rope_scaling* rope_scaling, void* stream) {
  return ragged_prefill(q, q_indptr, k, v, kv_indptr, q_rope_position, k_rope_pos_offset, output, lse, causal, rotary_mode,
                        rope_scale, rope_theta, sm_scale, batch_size, total_q, h_q, h_kv, d_qk, d_v, rope_scaling, stream);
}

static int paged_prefill(const void* q, const int32_t* q_indptr, const void* pages, const int32_t* page_indptr,
                         const int32_t* page_values, const int32_t* length_info, const int32_t* k_rope_pos_offset,
                         const int32_t* q_rope_position, void* output, float* lse, int64_t causal,
                         int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                         int32_t batch_size, int64_t total_q, int64_t nnz_pages, int64_t num_pages, int32_t h_q,
                         int32_t h_kv, int32_t d, int32_t page_size, int32_t sliding_window,
                         int32_t sliding_window_size, bool merge_into, void* stream,
                         const tvmkv_rope_scaling* scaling = nullptr) {
  // pages other than 16 / 32 / 64 / 128 tokens, other head dims (80 / 96 / 112 with a sliding-window cache or RoPE
  // inside the kernel among them): the generic matrix-core kernel (its caller merges states with merge_state_inplace)
  const bool plain = rotary_mode == 0 && sliding_window == 0;
  if (!merge_into && (!tuned_page_size(page_size) || !(plain ? tuned_head_dim(d) : (d == 64 || d == 128 || d == 256)))) {
    GenericAttention a;
    a.what = "batch_prefill_paged_kv";
    a.sliding_window = sliding_window;
    a.layer_window = sliding_window_size;
    a.rotary_mode = rotary_mode;
    a.q_rope_position = q_rope_position;
    a.k_rope_pos_offset = k_rope_pos_offset;
    a.rope_scale = rope_scale;
    a.rope_theta = rope_theta;
    a.rope_scaling = scaling;
    a.q = q;
    a.q_indptr = q_indptr;
    a.pages = pages;
    a.page_indptr = page_indptr;
    a.page_values = page_values;
    a.last_page_len = length_info;
    a.out = output;
    a.lse = lse;
    a.total_q = total_q;
    a.nnz_pages = nnz_pages;
    a.num_pages = num_pages;
    a.batch = batch_size;
    a.h_q = h_q;
    a.h_kv = h_kv;
    a.d = d;
    a.page_size = page_size;
    a.causal = causal > 0;
    a.sm_scale = sm_scale;
    return generic_attention(a, stream);
  }
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0)
      << "batch_prefill_paged_kv: bad shape";
  const int page_shift = paged_page_shift(page_size);
  KV_UNSUPPORTED(page_shift < 0) << "batch_prefill_paged_kv: page_size " << page_size << " is not built (16, 32, 64, 128)";
  KV_CHECK(num_pages < (int64_t{1} << 28)) << "batch_prefill_paged_kv: page ids must stay below 2^28";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && pages && page_indptr && length_info && output && lse)
      << "batch_prefill_paged_kv: NULL tensor";
  KV_CHECK(nnz_pages == 0 || page_values) << "batch_prefill_paged_kv: NULL page table";
  KV_CHECK(rotary_mode == 0 || (q_rope_position && k_rope_pos_offset))
      << "batch_prefill_paged_kv: inline RoPE needs the position arrays";
  PrefillParams p{};
  p.page_shift = page_shift;
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
  p.h_kv = h_kv;
  p.group = h_q / h_kv;
  p.causal = causal > 0;
  p.scale_log2 = static_cast<float>(sm_scale) * kLog2e;
  p.rotary = rotary_mode != 0;
  p.rope_scale = static_cast<float>(rope_scale);
  p.q_rope_position = q_rope_position;
  p.k_rope_pos_offset = k_rope_pos_offset;
  p.merge_into = merge_into;
  if (sliding_window != 0) {  // length_info is (3, B): last_page_len, window offset, sink size
    p.window_offset = length_info + batch_size;
    p.sink_size = length_info + 2 * static_cast<int64_t>(batch_size);
    p.layer_window = sliding_window_size;
  }
  const bool ext = p.rotary != 0 || sliding_window != 0;
  hipStream_t s = as_stream(stream);
  const KvSplit split(p, total_q, nnz_pages * page_size / batch_size, d, s);
  if (d == 128) {
    launch_prefill<128, 128, kPaged, 16>(p, total_q, ext, rope_theta, s, scaling);
  } else if (d == 64) {
    launch_prefill<64, 64, kPaged, 16>(p, total_q, ext, rope_theta, s, scaling);
  } else if (d == 256) {
    launch_prefill<256, 256, kPaged, 16>(p, total_q, ext, rope_theta, s, scaling);
  } else if (padded_head_dim(d)) {
    launch_prefill_padded<kPaged>(p, total_q, d, ext, "batch_prefill_paged_kv", s);
  } else {
    KV_UNSUPPORTED(true) << "batch_prefill_paged_kv: head_dim " << d << " is not built (64, 80, 96, 112, 128, 256)";
  }
  split.finish(p, d, s);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_batch_prefill_paged_kv(const void* q, const int32_t* q_indptr, const void* pages,
                                 const int32_t* page_indptr, const int32_t* page_values,
                                 const int32_t* length_info, const int32_t* k_rope_pos_offset,
                                 const int32_t* q_rope_position, void* output, float* lse, int64_t causal,
                                 int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                 int32_t batch_size, int64_t total_q, int64_t nnz_pages, int64_t num_pages,
                                 int32_t h_q, int32_t h_kv, int32_t d, int32_t page_size, int32_t sliding_window,
                                 int32_t sliding_window_size, void* stream) {
  return paged_prefill(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position,
                       output, lse, causal, rotary_mode, rope_scale, rope_theta, sm_scale, batch_size, total_q,
                       nnz_pages, num_pages, h_q, h_kv, d, page_size, sliding_window, sliding_window_size,
                       /*merge_into=*/false, stream);
}

int tvmkv_batch_prefill_paged_kv_merge(const void* q, const int32_t* q_indptr, const void* pages,
                                       const int32_t* page_indptr, const int32_t* page_values,
                                       const int32_t* length_info, const int32_t* k_rope_pos_offset,
                                       const int32_t* q_rope_position, void* output, float* lse, int64_t causal,
                                       int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                       int32_t batch_size, int64_t total_q, int64_t nnz_pages, int64_t num_pages,
                                       int32_t h_q, int32_t h_kv, int32_t d, int32_t page_size,
                                       int32_t sliding_window, int32_t sliding_window_size, void* stream) {
  return paged_prefill(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position,
                       output, lse, causal, rotary_mode, rope_scale, rope_theta, sm_scale, batch_size, total_q,
                       nnz_pages, num_pages, h_q, h_kv, d, page_size, sliding_window, sliding_window_size,
                       /*merge_into=*/true, stream);
}

int tvmkv_batch_prefill_paged_kv_scaled(const void* q, const int32_t* q_indptr, const void* pages,
                                        const int32_t* page_indptr, const int32_t* page_values,
                                        const int32_t* length_info, const int32_t* k_rope_pos_offset,
                                        const int32_t* q_rope_position, void* output, float* lse, int64_t causal,
                                        int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                        int32_t batch_size, int64_t total_q, int64_t nnz_pages, int64_t num_pages,
                                        int32_t h_q, int32_t h_kv, int32_t d, int32_t page_size, int32_t sliding_window,
                                        int32_t sliding_window_size, int32_t merge_into,
                                        const tvmkv_rope_scaling* rope_scaling, void* stream) {
  return paged_prefill(q, q_indptr, pages, page_indptr, page_values, length_info, k_rope_pos_offset, q_rope_position,
                       output, lse, causal, rotary_mode, rope_scale, rope_theta, sm_scale, batch_size, total_q,
                       nnz_pages, num_pages, h_q, h_kv, d, page_size, sliding_window, sliding_window_size,
                       merge_into != 0, stream, rope_scaling);
}

static int cached_and_new(const void* q, int64_t q_token_stride, const int32_t* q_rope_position, int64_t apply_rope,
                          double rope_scale, double rope_theta, const int32_t* q_indptr, const void* k, const void* v,
                          const void* pages, const int32_t* page_indptr, const int32_t* page_values,
                          const int32_t* last_page_len, void* output, float* lse, double sm_scale, int32_t batch_size,
                          int64_t total_q, int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv, int32_t d,
                          int32_t page_size, void* stream) {
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0)
      << "batch_prefill_cached_and_new_kv: bad shape";
  const int page_shift = paged_page_shift(page_size);
  KV_UNSUPPORTED(page_shift < 0) << "batch_prefill_cached_and_new_kv: page_size " << page_size << " is not built (16, 32, 64, 128)";
  KV_CHECK(num_pages < (int64_t{1} << 28)) << "batch_prefill_cached_and_new_kv: page ids must stay below 2^28";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && k && v && pages && page_indptr && last_page_len && output && lse)
      << "batch_prefill_cached_and_new_kv: NULL tensor";
  KV_CHECK(nnz_pages == 0 || page_values) << "batch_prefill_cached_and_new_kv: NULL page table";
  KV_CHECK(apply_rope == 0 || q_rope_position) << "batch_prefill_cached_and_new_kv: RoPE needs the position array";
  PrefillParams p{};
  p.page_shift = page_shift;
  p.q = static_cast<const half_t*>(q);
  p.q_token_stride = q_token_stride;
  p.q_inline_rope = apply_rope != 0;
  p.q_rope_position = q_rope_position;
  p.rope_scale = static_cast<float>(rope_scale);
  p.q_indptr = q_indptr;
  p.k = static_cast<const half_t*>(k);
  p.v = static_cast<const half_t*>(v);
  p.kv_indptr = q_indptr;  // the new tokens are the queries' own
  p.pages = static_cast<const half_t*>(pages);
  p.page_indptr = page_indptr;
  p.page_values = page_values;
  p.last_page_len = last_page_len;
  p.output = static_cast<half_t*>(output);
  p.lse = lse;
  p.batch_size = batch_size;
  p.h_q = h_q;
  p.h_kv = h_kv;
  p.group = h_q / h_kv;
  p.causal = 1;
  p.scale_log2 = static_cast<float>(sm_scale) * kLog2e;
  hipStream_t s = as_stream(stream);
  const KvSplit split(p, total_q, (nnz_pages * page_size + total_q) / batch_size, d, s);
  if (d == 128) {
    launch_prefill<128, 128, kBoth, 16>(p, total_q, false, rope_theta, s);
  } else if (d == 64) {
    launch_prefill<64, 64, kBoth, 16>(p, total_q, false, rope_theta, s);
  } else if (d == 256) {
    launch_prefill<256, 256, kBoth, 16>(p, total_q, false, rope_theta, s);
  } else {
    KV_UNSUPPORTED(true) << "batch_prefill_cached_and_new_kv: head_dim " << d << " is not built (64, 128, 256)";
  }
  split.finish(p, d, s);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_batch_prefill_cached_and_new_kv(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                          const void* pages, const int32_t* page_indptr,
                                          const int32_t* page_values, const int32_t* last_page_len, void* output,
                                          float* lse, double sm_scale, int32_t batch_size, int64_t total_q,
                                          int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                                          int32_t d, int32_t page_size, void* stream) {
  return cached_and_new(q, 0, nullptr, 0, 1.0, 1e4, q_indptr, k, v, pages, page_indptr, page_values, last_page_len,
                        output, lse, sm_scale, batch_size, total_q, nnz_pages, num_pages, h_q, h_kv, d, page_size,
                        stream);
}

int tvmkv_batch_prefill_cached_and_new_kv_fused_q(const void* qkv, const int32_t* q_rope_position, int64_t apply_rope,
                                                  double rope_scale, double rope_theta, const int32_t* q_indptr,
                                                  const void* k, const void* v, const void* pages,
                                                  const int32_t* page_indptr, const int32_t* page_values,
                                                  const int32_t* last_page_len, void* output, float* lse,
                                                  double sm_scale, int32_t batch_size, int64_t total_q,
                                                  int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                                                  int32_t d, int32_t page_size, void* stream) {
  return cached_and_new(qkv, static_cast<int64_t>(h_q + 2 * h_kv) * d, q_rope_position, apply_rope, rope_scale,
                        rope_theta, q_indptr, k, v, pages, page_indptr, page_values, last_page_len, output, lse, sm_scale,
                        batch_size, total_q, nnz_pages, num_pages, h_q, h_kv, d, page_size, stream);
}

static int tree_attn_ragged(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                            const int32_t* kv_indptr, const int32_t* q_rope_position, const int32_t* mn_indptr,
                            const int32_t* mask, void* output, float* lse, int64_t rotary_mode, double rope_scale,
                            double rope_theta, double sm_scale, int32_t batch_size, int64_t total_q, int32_t h_q,
                            int32_t h_kv, int32_t d, const tvmkv_rope_scaling* scaling, void* stream) {
  if (d != 64 && d != 128 && d != 256) {  // the generic matrix-core kernel
    GenericAttention a;
    a.what = "batch_tree_attn";
    a.rotary_mode = rotary_mode;  // key t of sequence b sits at q_rope_position[kv_indptr[b] + t]
    a.q_rope_position = q_rope_position;
    a.rope_scale = rope_scale;
    a.rope_theta = rope_theta;
    a.rope_scaling = scaling;
    a.q = q;
    a.q_indptr = q_indptr;
    a.k = k;
    a.v = v;
    a.kv_indptr = kv_indptr;
    a.tree_indptr = mn_indptr;
    a.tree_labels = mask;
    a.out = output;
    a.lse = lse;
    a.total_q = total_q;
    a.batch = batch_size;
    a.h_q = h_q;
    a.h_kv = h_kv;
    a.d = d;
    a.sm_scale = sm_scale;
    return generic_attention(a, stream);
  }
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0) << "batch_tree_attn: bad shape";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && k && v && kv_indptr && mn_indptr && mask && output && lse) << "batch_tree_attn: NULL tensor";
  KV_CHECK(rotary_mode == 0 || q_rope_position) << "batch_tree_attn: inline RoPE needs the position array";
  PrefillParams p{};
  p.q = static_cast<const half_t*>(q);
  p.q_indptr = q_indptr;
  p.k = static_cast<const half_t*>(k);
  p.v = static_cast<const half_t*>(v);
  p.kv_indptr = kv_indptr;
  p.output = static_cast<half_t*>(output);
  p.lse = lse;
  p.batch_size = batch_size;
  p.h_q = h_q;
  p.h_kv = h_kv;
  p.group = h_q / h_kv;
  p.causal = 0;
  p.scale_log2 = static_cast<float>(sm_scale) * kLog2e;
  p.rotary = rotary_mode != 0;
  p.rope_scale = static_cast<float>(rope_scale);
  p.q_rope_position = q_rope_position;
  p.k_rope_pos_offset = q_indptr;  // not used: keys take their positions from q_rope_position
  p.k_pos_from_q = 1;
  p.tree_indptr = mn_indptr;
  p.tree_order = mask;
  hipStream_t s = as_stream(stream);
  if (d == 128) {
    launch_prefill<128, 128, kRagged, 16>(p, total_q, true, rope_theta, s, scaling);
  } else if (d == 64) {
    launch_prefill<64, 64, kRagged, 16>(p, total_q, true, rope_theta, s, scaling);
  } else if (d == 256) {
    launch_prefill<256, 256, kRagged, 16>(p, total_q, true, rope_theta, s, scaling);
  } else {
    KV_UNSUPPORTED(true) << "batch_tree_attn: head_dim " << d << " is not built (64, 128, 256)";
  }
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_batch_tree_attn(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                          const int32_t* kv_indptr, const int32_t* q_rope_position, const int32_t* mn_indptr,
                          const int32_t* mask, void* output, float* lse, int64_t rotary_mode, double rope_scale,
                          double rope_theta, double sm_scale, int32_t batch_size, int64_t total_q, int32_t h_q,
                          int32_t h_kv, int32_t d, void* stream) {
  return tree_attn_ragged(q, q_indptr, k, v, kv_indptr, q_rope_position, mn_indptr, mask, output, lse, rotary_mode, rope_scale,
                          rope_theta, sm_scale, batch_size, total_q, h_q, h_kv, d, nullptr, stream);
}

int tvmkv_batch_tree_attn_scaled(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                 const int32_t* kv_indptr, const int32_t* q_rope_position, const int32_t* mn_indptr,
                                 const int32_t* mask, void* output, float* lse, int64_t rotary_mode, double rope_scale,
                                 double rope_theta, double sm_scale, int32_t batch_size, int64_t total_q, int32_t h_q,
                                 int32_t h_kv, int32_t d, const tvmkv_rope_scaling* rope_scaling, void* stream) {
  return tree_attn_ragged(q, q_indptr, k, v, kv_indptr, q_rope_position, mn_indptr, mask, output, lse, rotary_mode, rope_scale,
                          rope_theta, sm_scale, batch_size, total_q, h_q, h_kv, d, rope_scaling, stream);
}

int tvmkv_tree_attn_paged_kv(const void* q, const int32_t* q_indptr, const void* pages, const int32_t* page_indptr,
                             const int32_t* page_values, const int32_t* length_info,
                             const int32_t* k_rope_pos_offset, const int32_t* q_rope_position, void* output,
                             float* lse, int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                             const int32_t* tree_order_indptr, const int32_t* tree_order, int32_t batch_size,
                             int64_t total_q, int64_t nnz_pages, int64_t num_pages, int32_t h_q, int32_t h_kv,
                             int32_t d, int32_t page_size, int32_t sliding_window, void* stream) {
  if (rotary_mode == 0 && (!tuned_page_size(page_size) || (d != 64 && d != 128 && d != 256))) {
    GenericAttention a;  // the generic matrix-core kernel
    a.what = "tree_attn_paged_kv";
    a.sliding_window = sliding_window;
    a.q = q;
    a.q_indptr = q_indptr;
    a.pages = pages;
    a.page_indptr = page_indptr;
    a.page_values = page_values;
    a.last_page_len = length_info;
    a.tree_indptr = tree_order_indptr;
    a.tree_labels = tree_order;
    a.out = output;
    a.lse = lse;
    a.total_q = total_q;
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
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0)
      << "tree_attn_paged_kv: bad shape";
  const int page_shift = paged_page_shift(page_size);
  KV_UNSUPPORTED(page_shift < 0) << "tree_attn_paged_kv: page_size " << page_size << " is not built (16, 32, 64, 128)";
  KV_CHECK(num_pages < (int64_t{1} << 28)) << "tree_attn_paged_kv: page ids must stay below 2^28";
  // the reference kernel asserts the same (tree_attn.py:700-702)
  KV_UNSUPPORTED(rotary_mode != 0) << "tree_attn_paged_kv: inline rotary mode is not supported in tree attention";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && pages && page_indptr && length_info && output && lse && tree_order_indptr && tree_order)
      << "tree_attn_paged_kv: NULL tensor";
  KV_CHECK(nnz_pages == 0 || page_values) << "tree_attn_paged_kv: NULL page table";
  PrefillParams p{};
  p.page_shift = page_shift;
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
  p.h_kv = h_kv;
  p.group = h_q / h_kv;
  p.causal = 0;
  p.scale_log2 = static_cast<float>(sm_scale) * kLog2e;
  p.rope_scale = static_cast<float>(rope_scale);
  p.q_rope_position = q_rope_position;
  p.k_rope_pos_offset = k_rope_pos_offset;
  if (sliding_window != 0) {  // length_info is (3, B): last_page_len, window offset, sink size
    p.window_offset = length_info + batch_size;
    p.sink_size = length_info + 2 * static_cast<int64_t>(batch_size);
  }
  p.tree_indptr = tree_order_indptr;
  p.tree_order = tree_order;
  hipStream_t s = as_stream(stream);
  const KvSplit split(p, total_q, nnz_pages * page_size / batch_size, d, s);
  if (d == 128) {
    launch_prefill<128, 128, kPaged, 16>(p, total_q, true, rope_theta, s);
  } else if (d == 64) {
    launch_prefill<64, 64, kPaged, 16>(p, total_q, true, rope_theta, s);
  } else if (d == 256) {
    launch_prefill<256, 256, kPaged, 16>(p, total_q, true, rope_theta, s);
  } else {
    KV_UNSUPPORTED(true) << "tree_attn_paged_kv: head_dim " << d << " is not built (64, 128, 256)";
  }
  split.finish(p, d, s);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

}  // extern "C"
