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
// row per lane%32, and keeps Q as MFMA B-fragments in registers.  K/V tiles of 64 tokens go
// through LDS (K row-major, V transposed so that the token axis is contiguous); the next tile's
// global loads are issued before the current tile's math.  S^T = K Q^T and O^T = V^T P^T use
// v_mfma_f32_32x32x16_f16 with the query on the N axis: all per-query softmax state (m, l, the
// O rescale factor) is lane-local, and the S^T accumulator registers are exactly the B-operand
// of the PV product, so P never leaves registers.
//
// Workgroup -> (sequence, row tile) without a prologue kernel: sequence b owns tile slots
//   [floor(q_indptr[b]*group/128) + b, floor(q_indptr[b+1]*group/128) + b + 1)
// found by binary search on q_indptr; the grid is floor(total_q*group/128) + B slots.
#include "kernels_common.cuh"

namespace tvmkv {

constexpr int BM = 128;  // rows per workgroup
constexpr int BN = 64;   // kv tokens per tile
constexpr int KPAD = 8;  // halfs of padding per K row in LDS
constexpr int VPAD = 4;  // halfs of padding per V^T row in LDS

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
};

__device__ __forceinline__ int tile_slot_begin(const int32_t* q_indptr, int b, int group) {
  return static_cast<int>((static_cast<int64_t>(q_indptr[b]) * group) / BM) + b;
}

template <int DQK, int DV, bool PAGED, int PS>
__global__ __launch_bounds__(256, 2) void prefill_kernel(PrefillParams p) {
  static_assert(DQK % 16 == 0 && DV % 32 == 0, "feature dims must fit the MFMA tiles");
  constexpr int KS = DQK / 16;                  // k-steps of the QK^T product
  constexpr int DB = DV / 32;                   // 32-wide output feature blocks
  constexpr int TB = BN / 32;                   // 32-token blocks per tile
  constexpr int KROW = DQK + KPAD;              // LDS row stride of K (halfs)
  constexpr int VROW = BN + VPAD;               // LDS row stride of V^T (halfs)
  constexpr int KCH = DQK / 8;                  // 16-byte pieces per K row
  constexpr int KLOADS = BN * KCH / 256;        // K pieces per thread per tile
  constexpr int VCH = DV / 8;                   // 16-byte pieces per V row
  constexpr int VUNITS = (BN / 4) * VCH;        // (4 tokens x 8 features) units per tile
  constexpr int VT = (VUNITS + 255) / 256;      // units per thread
  static_assert(BN * KCH % 256 == 0, "K tile must divide evenly over the workgroup");
  static_assert(!PAGED || PS % 4 == 0, "page size must be a multiple of 4");

  // two LDS buffers: tile t+1 is stored while the other waves still read tile t, one barrier per tile
  __shared__ __attribute__((aligned(16))) half_t Ks_buf[2][BN * KROW];
  __shared__ __attribute__((aligned(16))) half_t Vt_buf[2][DV * VROW];

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
  const int slot = blockIdx.y;
  int b;
  {
    int lo = 0, hi = p.batch_size - 1;
    while (lo < hi) {
      int mid = (lo + hi + 1) >> 1;
      if (tile_slot_begin(p.q_indptr, mid, group) <= slot) {
        lo = mid;
      } else {
        hi = mid - 1;
      }
    }
    b = lo;
  }
  const int q_start = p.q_indptr[b];
  const int qo_len = p.q_indptr[b + 1] - q_start;
  const int rows = qo_len * group;
  // tiles of a sequence are handed out last-first: under the causal mask the last rows see the
  // most keys, and the longest workgroups should start first
  const int local_slot = slot - tile_slot_begin(p.q_indptr, b, group);
  const int n_row_tiles = (rows + BM - 1) / BM;
  if (local_slot >= n_row_tiles) return;
  const int r0 = (n_row_tiles - 1 - local_slot) * BM;

  int kv_len, kv_start = 0, pbeg = 0;
  if (PAGED) {
    pbeg = p.page_indptr[b];
    const int npages = p.page_indptr[b + 1] - pbeg;
    kv_len = npages > 0 ? (npages - 1) * PS + p.last_page_len[b] : 0;
  } else {
    kv_start = p.kv_indptr[b];
    kv_len = p.kv_indptr[b + 1] - kv_start;
  }

  // ---- this lane's query row -------------------------------------------------------------
  const int my_row = r0 + wave * 32 + col;
  const bool row_valid = my_row < rows;
  const int my_pos = my_row / group;
  const int my_head = kvh * group + my_row % group;
  const int causal_shift = kv_len - qo_len + 1;
  // number of visible kv tokens for this row
  const int my_limit = row_valid ? (p.causal ? min(kv_len, causal_shift + my_pos) : kv_len) : 0;
  // workgroup- and wave-level bounds (uniform)
  const int last_row_wg = min(rows, r0 + BM) - 1;
  const int kv_end = p.causal ? max(0, min(kv_len, causal_shift + last_row_wg / group)) : kv_len;
  const int first_row_wave = r0 + wave * 32;
  const int last_row_wave = min(rows, first_row_wave + 32) - 1;  // < first_row_wave if the wave is empty
  const bool wave_active = first_row_wave < rows;
  const int wave_limit_max = !wave_active ? 0 : (p.causal ? min(kv_len, causal_shift + last_row_wave / group) : kv_len);
  const int wave_limit_min = !wave_active ? 0 : (p.causal ? min(kv_len, causal_shift + first_row_wave / group) : kv_len);

  half8_t qf[KS];
  {
    const half_t* qrow = p.q + (static_cast<int64_t>(q_start + my_pos) * p.h_q + my_head) * DQK + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = row_valid ? ld16(qrow + ks * 16).h8 : zero16().h8;
  }

  float16_t o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db) {
#pragma unroll
    for (int j = 0; j < 16; ++j) o[db][j] = 0.f;
  }
  float m = kNegInit, lsum = 0.f;

  // ---- tile loaders ----------------------------------------------------------------------
  Vec16 kreg[KLOADS];
  Vec16 vreg[VT][4];
  auto load_tile = [&](int kv0) {
#pragma unroll
    for (int r = 0; r < KLOADS; ++r) {
      const int c = r * 256 + tid;
      const int row = c / KCH;
      const int piece = c % KCH;
      const int t = kv0 + row;
      if (t < kv_len) {
        const half_t* src;
        if (PAGED) {
          const int page = p.page_values[pbeg + t / PS];
          src = p.pages + ((static_cast<int64_t>(page) * 2 * p.h_kv + kvh) * PS + t % PS) * DQK + piece * 8;
        } else {
          src = p.k + (static_cast<int64_t>(kv_start + t) * p.h_kv + kvh) * DQK + piece * 8;
        }
        kreg[r] = ld16(src);
      } else {
        kreg[r] = zero16();
      }
    }
#pragma unroll
    for (int u = 0; u < VT; ++u) {
      const int idx = u * 256 + tid;
      const int dchunk = idx % VCH;
      const int tgroup = idx / VCH;
      const int t0 = kv0 + tgroup * 4;
      const half_t* src = nullptr;
      int64_t tok_stride = 0;
      if (idx < VUNITS && t0 < kv_len) {
        if (PAGED) {
          const int page = p.page_values[pbeg + t0 / PS];
          src = p.pages + ((static_cast<int64_t>(page) * 2 + 1) * p.h_kv + kvh) * (static_cast<int64_t>(PS) * DV) +
                (t0 % PS) * DV + dchunk * 8;
          tok_stride = DV;
        } else {
          src = p.v + (static_cast<int64_t>(kv_start + t0) * p.h_kv + kvh) * DV + dchunk * 8;
          tok_stride = static_cast<int64_t>(p.h_kv) * DV;
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        vreg[u][r] = (src != nullptr && t0 + r < kv_len) ? ld16(src + r * tok_stride) : zero16();
      }
    }
  };
  auto store_tile = [&](half_t* Ks, half_t* Vt) {
#pragma unroll
    for (int r = 0; r < KLOADS; ++r) {
      const int c = r * 256 + tid;
      st16(Ks + (c / KCH) * KROW + (c % KCH) * 8, kreg[r]);
    }
#pragma unroll
    for (int u = 0; u < VT; ++u) {
      const int idx = u * 256 + tid;
      if (idx < VUNITS) {
        const int dchunk = idx % VCH;
        const int tgroup = idx / VCH;
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          // words e2 of the four token rows hold features (2*e2, 2*e2+1)
          const uint32_t w0 = vreg[u][0].w[e2], w1 = vreg[u][1].w[e2], w2 = vreg[u][2].w[e2], w3 = vreg[u][3].w[e2];
          uint2 even, odd;  // 4 tokens of feature 2*e2 / 2*e2+1
          even.x = (w0 & 0xffffu) | (w1 << 16);
          even.y = (w2 & 0xffffu) | (w3 << 16);
          odd.x = (w0 >> 16) | (w1 & 0xffff0000u);
          odd.y = (w2 >> 16) | (w3 & 0xffff0000u);
          *reinterpret_cast<uint2*>(Vt + (dchunk * 8 + 2 * e2) * VROW + tgroup * 4) = even;
          *reinterpret_cast<uint2*>(Vt + (dchunk * 8 + 2 * e2 + 1) * VROW + tgroup * 4) = odd;
        }
      }
    }
  };

  const int n_tiles = (kv_end + BN - 1) / BN;
  if (n_tiles > 0) load_tile(0);
  for (int tile = 0; tile < n_tiles; ++tile) {
    const int kv0 = tile * BN;
    half_t* Ks = Ks_buf[tile & 1];
    half_t* Vt = Vt_buf[tile & 1];
    // buffer (tile & 1) was last read during tile-2; every wave passed the barrier of tile-1 since
    store_tile(Ks, Vt);
    __syncthreads();
    if (tile + 1 < n_tiles) load_tile(kv0 + BN);

    if (kv0 < wave_limit_max) {  // wave-uniform: otherwise every row of this wave is masked out
      // The 64-token tile is consumed as TB sub-tiles of 32 tokens.  Per sub-tile the LDS reads are
      // issued in two batches well ahead of their MFMAs (the compiler otherwise serialises one
      // read per MFMA and exposes the LDS latency 32 times per tile): K fragments first, then the
      // V^T fragments, whose latency hides behind the softmax arithmetic.
#pragma unroll
      for (int tb = 0; tb < TB; ++tb) {
        const int t0 = kv0 + tb * 32;
        if (t0 >= wave_limit_max) break;  // wave-uniform
        half8_t kf[KS];
        {
          const half_t* krow = Ks + (tb * 32 + col) * KROW + half * 8;
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) kf[ks] = ld16(krow + ks * 16).h8;
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- S^T = K Q^T --------------------------------------------------------------------
        float16_t acc;
#pragma unroll
        for (int j = 0; j < 16; ++j) acc[j] = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[ks], qf[ks], acc, 0, 0, 0);
        // ---- V^T fragments: contraction slot half*8+i holds token kk*16 + (i/4)*8 + half*4 + i%4
        half8_t vf[DB][2];
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const half_t* vrow = Vt + (db * 32 + col) * VROW + half * 4 + tb * 32;
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) {
            const half4_t lo = *reinterpret_cast<const half4_t*>(vrow + kk * 16);
            const half4_t hi = *reinterpret_cast<const half4_t*>(vrow + kk * 16 + 8);
            vf[db][kk][0] = lo[0]; vf[db][kk][1] = lo[1]; vf[db][kk][2] = lo[2]; vf[db][kk][3] = lo[3];
            vf[db][kk][4] = hi[0]; vf[db][kk][5] = hi[1]; vf[db][kk][6] = hi[2]; vf[db][kk][7] = hi[3];
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        // ---- mask, online softmax (lane-local per query); the scale is folded into the exponent:
        // p = exp2(acc*scale - m)
        if (t0 + 32 > wave_limit_min) {  // wave-uniform; only tiles on the diagonal or at the tail
          asm volatile("" ::: "memory");  // keep this a branch: if-converted it costs 5 ops per element everywhere
          const int rel = my_limit - t0 - half * 4;  // element j is token t0 + half*4 + (j/4)*8 + j%4
#pragma unroll
          for (int j = 0; j < 16; ++j) acc[j] = ((j >> 2) * 8 + (j & 3)) < rel ? acc[j] : -3.0e38f;
        }
        float mx_raw = -3.0e38f;
#pragma unroll
        for (int j = 0; j < 16; ++j) mx_raw = fmaxf(mx_raw, acc[j]);
        mx_raw = fmaxf(mx_raw, __shfl_xor(mx_raw, 32, 64));
        // a fully masked row keeps its old maximum (the scaled sentinel is far below -5e4)
        const float m_new = fmaxf(m, fmaxf(mx_raw * p.scale_log2, -1.0e30f));
        const float alpha = fast_exp2(m - m_new);
        m = m_new;
        lsum *= alpha;
        if (__builtin_amdgcn_readfirstlane(__any(alpha != 1.0f))) {  // wave-uniform: skip when no maximum moved
#pragma unroll
          for (int db = 0; db < DB; ++db) {
#pragma unroll
            for (int j = 0; j < 16; ++j) o[db][j] *= alpha;
          }
        }
        half8_t pf[2];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
          const float pj = fast_exp2(fmaf(acc[j], p.scale_log2, -m_new));  // masked: exp2(-3e38*scale - m) = 0
          lsum += pj;
          pf[j >> 3][j & 7] = static_cast<half_t>(pj);
        }
        // ---- O^T += V^T P^T -----------------------------------------------------------------
#pragma unroll
        for (int db = 0; db < DB; ++db) {
#pragma unroll
          for (int kk = 0; kk < 2; ++kk) o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[db][kk], pf[kk], o[db], 0, 0, 0);
        }
      }
    }
  }

  // ---- epilogue ------------------------------------------------------------------------------
  lsum += __shfl_xor(lsum, 32, 64);
  const float denom = lsum + fast_exp2(kNegInit - m);  // the d = 1 of the initial state
  if (row_valid) {
    const float inv = 1.0f / denom;
    half_t* orow = p.output + (static_cast<int64_t>(q_start + my_pos) * p.h_q + my_head) * DV + half * 4;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int j4 = 0; j4 < 4; ++j4) {
        half4_t out4;
#pragma unroll
        for (int e = 0; e < 4; ++e) out4[e] = static_cast<half_t>(o[db][j4 * 4 + e] * inv);
        *reinterpret_cast<half4_t*>(orow + db * 32 + j4 * 8) = out4;
      }
    }
    if (half == 0) p.lse[static_cast<int64_t>(q_start + my_pos) * p.h_q + my_head] = m + fast_log2(denom);
  }
}

template <int DQK, int DV, bool PAGED, int PS>
static void launch_prefill(const PrefillParams& p, int64_t total_q, hipStream_t stream) {
  const int64_t slots = total_q * p.group / BM + p.batch_size;
  if (slots >= 65536) throw Error(TVMKV_EINVAL, "prefill: too many row tiles for one launch (65535 x 128 rows)");
  hipLaunchKernelGGL((prefill_kernel<DQK, DV, PAGED, PS>), dim3(p.h_kv, static_cast<unsigned>(slots)), dim3(256), 0,
                     stream, p);
}

}  // namespace tvmkv

using namespace tvmkv;

extern "C" {

int tvmkv_batch_prefill_ragged_kv(const void* q, const int32_t* q_indptr, const void* k, const void* v,
                                  const int32_t* kv_indptr, const int32_t* q_rope_position,
                                  const int32_t* k_rope_pos_offset, void* output, float* lse, int64_t causal,
                                  int64_t rotary_mode, double rope_scale, double rope_theta, double sm_scale,
                                  int32_t batch_size, int64_t total_q, int32_t h_q, int32_t h_kv, int32_t d_qk,
                                  int32_t d_v, void* stream) {
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0)
      << "batch_prefill_ragged_kv: bad shape";
  KV_UNSUPPORTED(rotary_mode != 0) << "batch_prefill_ragged_kv: inline RoPE (rotary_mode=1) is not built";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && k && v && kv_indptr && output && lse) << "batch_prefill_ragged_kv: NULL tensor";
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
  hipStream_t s = as_stream(stream);
  if (d_qk == 128 && d_v == 128) {
    launch_prefill<128, 128, false, 16>(p, total_q, s);
  } else if (d_qk == 64 && d_v == 64) {
    launch_prefill<64, 64, false, 16>(p, total_q, s);
  } else if (d_qk == 192 && d_v == 128) {
    launch_prefill<192, 128, false, 16>(p, total_q, s);
  } else {
    KV_UNSUPPORTED(true) << "batch_prefill_ragged_kv: (d_qk, d_v) = (" << d_qk << ", " << d_v
                         << ") is not built ((64,64), (128,128), (192,128))";
  }
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
  KV_API_BEGIN();
  KV_CHECK(batch_size >= 0 && total_q >= 0 && h_q > 0 && h_kv > 0 && h_q % h_kv == 0)
      << "batch_prefill_paged_kv: bad shape";
  KV_UNSUPPORTED(rotary_mode != 0) << "batch_prefill_paged_kv: inline RoPE (rotary_mode=1) is not built";
  KV_UNSUPPORTED(sliding_window != 0) << "batch_prefill_paged_kv: sliding-window length_info (3, B) is not built";
  KV_UNSUPPORTED(page_size != 16) << "batch_prefill_paged_kv: page_size " << page_size << " is not built (16)";
  if (batch_size == 0 || total_q == 0) return TVMKV_OK;
  KV_CHECK(q && q_indptr && pages && page_indptr && length_info && output && lse)
      << "batch_prefill_paged_kv: NULL tensor";
  KV_CHECK(nnz_pages == 0 || page_values) << "batch_prefill_paged_kv: NULL page table";
  PrefillParams p{};
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
  hipStream_t s = as_stream(stream);
  if (d == 128) {
    launch_prefill<128, 128, true, 16>(p, total_q, s);
  } else if (d == 64) {
    launch_prefill<64, 64, true, 16>(p, total_q, s);
  } else {
    KV_UNSUPPORTED(true) << "batch_prefill_paged_kv: head_dim " << d << " is not built (64, 128)";
  }
  KV_LAUNCH_CHECK();
  KV_API_END();
}

}  // extern "C"
