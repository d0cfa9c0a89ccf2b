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
// Tiling: 128 rows (position, head) per workgroup, 32 rows per wave with the query on the MFMA
// N axis; 32-token KV tiles are read from HBM once per workgroup and written to LDS twice: row
// major (A-operand of S^T = KV Q^T) and transposed (A-operand of O^T = V^T P^T).  O^T of one wave
// is 512 x 32 fp32 = 256 accumulator registers, Q is 144 registers of B-fragments: one wave per
// SIMD.
//
// KV split: decode-shaped calls have too few row tiles to fill 256 CUs, so a sequence's KV may be
// cut into up to `max_chunks` chunks (grid.y), each at least 128 tokens; partial (O, m, l) states
// go to an fp32 buffer indexed by (global row, chunk) and a second kernel merges them.  The chunk
// count of a sequence is a pure function of its kv_len, recomputed by both kernels.
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
  float* part_o;   // (total_rows, max_chunks, DV)
  float* part_ml;  // (total_rows, max_chunks, 2)
  int batch_size;
  int h_q;
  int page_size;
  int causal;
  int max_chunks;
  float scale_log2;
};

__device__ __forceinline__ int mla_tile_slot_begin(const int32_t* q_indptr, int b, int h_q) {
  return static_cast<int>((static_cast<int64_t>(q_indptr[b]) * h_q) / MLA_BM) + b;
}

__device__ __forceinline__ int mla_num_chunks(int kv_len, int max_chunks) {
  return max(1, min(max_chunks, (kv_len + MLA_MIN_CHUNK - 1) / MLA_MIN_CHUNK));
}

template <int DQK, int DV>
__global__ __launch_bounds__(256) void mla_paged_kernel(MlaParams p) {
  constexpr int BN = MLA_BN;
  constexpr int KS = DQK / 16;
  constexpr int DB = DV / 32;
  constexpr int KROW = DQK + 8;
  constexpr int VROW = BN + 4;
  constexpr int FCH = DQK / 8;            // 16-byte pieces per cached row
  constexpr int VCH = DV / 8;             // of which the first VCH belong to the value part
  constexpr int UNITS = (BN / 4) * FCH;   // (4 tokens x 8 features) units per tile
  constexpr int ROUNDS = (UNITS + 255) / 256;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  half_t* Ks = reinterpret_cast<half_t*>(smem_raw);  // [BN][KROW]
  half_t* Vt = Ks + BN * KROW;                       // [DV][VROW]

  const int tid = threadIdx.x;
  const int wave = tid >> 6;
  const int lane = tid & 63;
  const int col = lane & 31;
  const int half = lane >> 5;
  const int h_q = p.h_q;

  const int slot = blockIdx.x;
  int b;
  {
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
  }
  const int q_start = p.q_indptr[b];
  const int qo_len = p.q_indptr[b + 1] - q_start;
  const int rows = qo_len * h_q;
  const int r0 = (slot - mla_tile_slot_begin(p.q_indptr, b, h_q)) * MLA_BM;
  if (r0 >= rows) return;

  const int pbeg = p.page_indptr[b];
  const int npages = p.page_indptr[b + 1] - pbeg;
  const int ps = p.page_size;
  const int kv_len = npages > 0 ? (npages - 1) * ps + p.last_page_len[b] : 0;
  const int nchunks = mla_num_chunks(kv_len, p.max_chunks);
  const int chunk = blockIdx.y;
  if (chunk >= nchunks) return;

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

  half8_t qf[KS];
  {
    const half_t* qrow = p.q + (static_cast<int64_t>(q_start + my_pos) * h_q + my_head) * DQK + half * 8;
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

  Vec16 stage[ROUNDS][4];
  auto load_tile = [&](int kv0) {
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int idx = r * 256 + tid;
      const int piece = idx % FCH;
      const int tgroup = idx / FCH;
      const int t0 = kv0 + tgroup * 4;
      const half_t* src = nullptr;
      if (idx < UNITS && t0 < kv_len) {
        const int page = p.page_values[pbeg + t0 / ps];  // 4 | page_size: the 4 tokens share a page
        src = p.pages + (static_cast<int64_t>(page) * ps + t0 % ps) * DQK + piece * 8;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) stage[r][e] = (src != nullptr && t0 + e < kv_len) ? ld16(src + e * DQK) : zero16();
    }
  };
  auto store_tile = [&]() {
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const int idx = r * 256 + tid;
      if (idx < UNITS) {
        const int piece = idx % FCH;
        const int tgroup = idx / FCH;
#pragma unroll
        for (int e = 0; e < 4; ++e) st16(Ks + (tgroup * 4 + e) * KROW + piece * 8, stage[r][e]);
        if (piece < VCH) {
#pragma unroll
          for (int e2 = 0; e2 < 4; ++e2) {
            const uint32_t w0 = stage[r][0].w[e2], w1 = stage[r][1].w[e2], w2 = stage[r][2].w[e2], w3 = stage[r][3].w[e2];
            uint2 even, odd;
            even.x = (w0 & 0xffffu) | (w1 << 16);
            even.y = (w2 & 0xffffu) | (w3 << 16);
            odd.x = (w0 >> 16) | (w1 & 0xffff0000u);
            odd.y = (w2 >> 16) | (w3 & 0xffff0000u);
            *reinterpret_cast<uint2*>(Vt + (piece * 8 + 2 * e2) * VROW + tgroup * 4) = even;
            *reinterpret_cast<uint2*>(Vt + (piece * 8 + 2 * e2 + 1) * VROW + tgroup * 4) = odd;
          }
        }
      }
    }
  };

  if (tile_lo < tile_hi) load_tile(tile_lo * BN);
  for (int tile = tile_lo; tile < tile_hi; ++tile) {
    const int kv0 = tile * BN;
    __syncthreads();
    store_tile();
    __syncthreads();
    if (tile + 1 < tile_hi) load_tile(kv0 + BN);

    if (kv0 < wave_limit_max) {
      float16_t acc;
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[j] = 0.f;
      const half_t* krow = Ks + col * KROW + half * 8;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const half8_t a = ld16(krow + ks * 16).h8;
        acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, qf[ks], acc, 0, 0, 0);
      }
      const bool need_mask = kv0 + BN > wave_limit_min;
      float mx = kNegInit;
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        float s = acc[j] * p.scale_log2;
        if (need_mask) {
          const int t = kv0 + (j >> 2) * 8 + half * 4 + (j & 3);
          s = t < my_limit ? s : kNegInit;
        }
        acc[j] = s;
        mx = fmaxf(mx, s);
      }
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      const float m_new = fmaxf(m, mx);
      const float alpha = fast_exp2(m - m_new);
      m = m_new;
      lsum *= alpha;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
#pragma unroll
        for (int j = 0; j < 16; ++j) o[db][j] *= alpha;
      }
      half8_t pf[2];
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        float pj = fast_exp2(acc[j] - m_new);
        if (need_mask) {
          const int t = kv0 + (j >> 2) * 8 + half * 4 + (j & 3);
          pj = t < my_limit ? pj : 0.f;
        }
        lsum += pj;
        pf[j >> 3][j & 7] = static_cast<half_t>(pj);
      }
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const half_t* vrow = Vt + (db * 32 + col) * VROW + half * 4;
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
          const half4_t lo = *reinterpret_cast<const half4_t*>(vrow + kk * 16);
          const half4_t hi = *reinterpret_cast<const half4_t*>(vrow + kk * 16 + 8);
          half8_t a;
          a[0] = lo[0]; a[1] = lo[1]; a[2] = lo[2]; a[3] = lo[3];
          a[4] = hi[0]; a[5] = hi[1]; a[6] = hi[2]; a[7] = hi[3];
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pf[kk], o[db], 0, 0, 0);
        }
      }
    }
  }

  lsum += __shfl_xor(lsum, 32, 64);
  if (!row_valid) return;
  const int64_t grow = static_cast<int64_t>(q_start + my_pos) * h_q + my_head;  // global row
  if (nchunks == 1) {
    const float denom = lsum + fast_exp2(kNegInit - m);
    const float inv = 1.0f / denom;
    half_t* orow = p.output + grow * DV + half * 4;
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
    if (half == 0) p.lse[grow] = m + fast_log2(denom);
  } else {
    float* prow = p.part_o + (grow * p.max_chunks + chunk) * DV + half * 4;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
#pragma unroll
      for (int j4 = 0; j4 < 4; ++j4) {
        float4_t out4;
#pragma unroll
        for (int e = 0; e < 4; ++e) out4[e] = o[db][j4 * 4 + e];
        *reinterpret_cast<float4_t*>(prow + db * 32 + j4 * 8) = out4;
      }
    }
    if (half == 0) {
      p.part_ml[(grow * p.max_chunks + chunk) * 2 + 0] = m;
      p.part_ml[(grow * p.max_chunks + chunk) * 2 + 1] = lsum;
    }
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
  // skip sequences with qo_len == 0 that share the q_indptr value: the search above returns the
  // last b with q_indptr[b] <= token, which is the one that owns the token
  const int npages = p.page_indptr[b + 1] - p.page_indptr[b];
  const int kv_len = npages > 0 ? (npages - 1) * p.page_size + p.last_page_len[b] : 0;
  const int nchunks = mla_num_chunks(kv_len, p.max_chunks);
  if (nchunks == 1) return;
  const int64_t grow = static_cast<int64_t>(token) * p.h_q + head;
  const float* ml = p.part_ml + grow * p.max_chunks * 2;
  float mx = kNegInit;
  for (int c = 0; c < nchunks; ++c) mx = fmaxf(mx, ml[c * 2]);
  float lsum = 0.f;
  float4_t acc = {0.f, 0.f, 0.f, 0.f};
  const int d = threadIdx.x * 4;
  for (int c = 0; c < nchunks; ++c) {
    const float sc = fast_exp2(ml[c * 2] - mx);
    lsum += ml[c * 2 + 1] * sc;
    const float4_t po = *reinterpret_cast<const float4_t*>(p.part_o + (grow * p.max_chunks + c) * DV + d);
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
  KV_UNSUPPORTED(page_size <= 0 || page_size % 4 != 0)
      << "batch_prefill_paged_kv_mla: page_size " << page_size << " must be a positive multiple of 4";
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
  const int64_t slots = total_q * h_q / MLA_BM + batch_size;
  KV_CHECK(slots < (int64_t{1} << 31)) << "batch_prefill_paged_kv_mla: too many row tiles";
  // split the KV only when the row tiles alone cannot fill the chip (decode-shaped calls)
  int max_chunks = static_cast<int>(512 / slots);
  max_chunks = max_chunks < 1 ? 1 : (max_chunks > 16 ? 16 : max_chunks);
  p.max_chunks = max_chunks;
  if (max_chunks > 1) {
    const size_t rows = static_cast<size_t>(total_q) * h_q;
    const size_t part_o_bytes = rows * max_chunks * DV * sizeof(float);
    char* ws = static_cast<char*>(mla_workspace(part_o_bytes + rows * max_chunks * 2 * sizeof(float)));
    p.part_o = reinterpret_cast<float*>(ws);
    p.part_ml = reinterpret_cast<float*>(ws + part_o_bytes);
  }
  constexpr size_t lds_bytes = (MLA_BN * (DQK + 8) + DV * (MLA_BN + 4)) * sizeof(half_t);
  static bool attr_set = false;
  if (!attr_set) {
    HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void*>(&mla_paged_kernel<DQK, DV>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes)));
    attr_set = true;
  }
  hipStream_t s = as_stream(stream);
  hipLaunchKernelGGL((mla_paged_kernel<DQK, DV>), dim3(static_cast<unsigned>(slots), max_chunks), dim3(256), lds_bytes,
                     s, p);
  KV_LAUNCH_CHECK();
  if (max_chunks > 1) {
    hipLaunchKernelGGL(mla_merge_kernel<DV>, dim3(static_cast<unsigned>(total_q), h_q), dim3(DV / 4), 0, s, p);
    KV_LAUNCH_CHECK();
  }
  KV_API_END();
}
