// Page-granular data movement kernels of the paged KV cache and the two-way state merge:
// fused qkv split + RoPE, K/V append scatter (MHA and MLA), single-page copy for fork,
// gather for debug reads, compaction copy, and merge_state_inplace.
//
// All of them are HBM-bound byte movers: one thread owns 16 bytes (8 fp16), consecutive
// lanes own consecutive 16-byte pieces of one head vector, so every wavefront access is a
// run of full 128-byte lines.
#include <cmath>

#include <type_traits>

#include "kernels_common.cuh"
#include "typed_kernels.h"
#include "runtime_support.h"

namespace tvmkv {

// ------------------------------------------------------------------------------------------
// fused_rope: split qkv and rotate q,k.
// Reference arithmetic (python/tvm/relax/frontend/nn/llm/position_embedding.py:32-67,493-523):
//   freq = (pos * scale) / pow(theta, (2d mod D) / D);  out[d] = cos(freq)*x[d] + sin(freq)*y[d]
//   y[d] = -x[d + D/2] for d < D/2, x[d - D/2] otherwise; fp32 math, one rounding to fp16.
// The D/2 divisors pow(theta, 2i/D) are computed on the host with the same libm call the CPU
// kernels use and travel as a kernel argument, so the angle is formed by one IEEE division.
// ------------------------------------------------------------------------------------------
// One entry per element of the head: element d and its rotation partner d + D/2 share an angle in
// every variant but yarn, whose blend between interpolated and extrapolated frequencies is indexed
// by the element (position_embedding.py:244-247).
struct RopeDivisors {
  float v[kMaxHeadDim];
};

// One workgroup per token: the D/2 (cos, sin) pairs of the token's position are computed once
// (they are the same for every head; the precise sinf/cosf with their range reduction are by far
// the most expensive part) and shared through LDS, then all heads of the token are streamed.
// APPEND: the rotated k and the v rows also go into their page slots (what transpose_append
// does from the k / v outputs), slot append_position_map[token], -1 = none.
template <int D, bool APPEND>
__global__ __launch_bounds__(256) void fused_rope_kernel(const half_t* __restrict__ qkv,
                                                         const int32_t* __restrict__ position_map,
                                                         half_t* __restrict__ q, half_t* __restrict__ k,
                                                         half_t* __restrict__ v, int64_t seq_len, int num_q_heads,
                                                         int num_kv_heads, int apply_rope, float scale,
                                                         RopeDivisors div, int table_is_inverse, int halves_differ,
                                                         float magnitude,
                                                         const float* __restrict__ ext_factors,
                                                         half_t* __restrict__ pages,
                                                         const int32_t* __restrict__ append_position_map,
                                                         int page_size, int rotary_dim, int interleaved) {
  constexpr int kThreadsPerHead = D / 16;  // a thread owns d-range [8c, 8c+8) and its partner +D/2
  // element d < R = rotary_dim: [0, R/2) for the elements of the lower half, [R/2, R) of the upper half
  __shared__ float cs_lds[D];
  __shared__ float sn_lds[D];
  const int R = rotary_dim;
  const int64_t s = blockIdx.x;  // token
  const int fused_heads = num_q_heads + 2 * num_kv_heads;
  if (apply_rope > 0) {
    const float pos_scaled = static_cast<float>(position_map[s]) * scale;
    for (int i = threadIdx.x; i < (halves_differ ? R : R / 2); i += 256) {
      // default / longrope: position over a divisor (times the model's per-dimension factor, if any);
      // llama3 / yarn: position times an inverse frequency (position_embedding.py:130-255)
      float freq;
      if (table_is_inverse) {
        freq = pos_scaled * div.v[i];
      } else {
        freq = pos_scaled / (ext_factors != nullptr ? ext_factors[i] * div.v[i] : div.v[i]);
      }
      const float cs = cosf(freq) * magnitude, sn = sinf(freq) * magnitude;
      cs_lds[i] = cs;
      sn_lds[i] = sn;
      if (!halves_differ) {
        cs_lds[i + R / 2] = cs;
        sn_lds[i + R / 2] = sn;
      }
    }
    __syncthreads();
  }
  // q == NULL: the q rows are left alone (an attention kernel that reads them from qkv rotates them itself)
  const int first_task = q == nullptr ? num_q_heads * kThreadsPerHead : 0;
  for (int task = first_task + threadIdx.x; task < fused_heads * kThreadsPerHead; task += 256) {
    const int c = task % kThreadsPerHead;
    const int h = task / kThreadsPerHead;
    const half_t* src = qkv + (s * fused_heads + h) * D + c * 8;
    Vec16 lo = ld16(src);
    Vec16 hi = ld16(src + D / 2);
    half_t* dst;
    if (h < num_q_heads) {
      dst = q + (s * num_q_heads + h) * D;
    } else if (h < num_q_heads + num_kv_heads) {
      dst = k + (s * num_kv_heads + (h - num_q_heads)) * D;
    } else {
      dst = v + (s * num_kv_heads + (h - num_q_heads - num_kv_heads)) * D;
    }
    if (apply_rope > 0 && h < num_q_heads + num_kv_heads && interleaved) {
      // gptj pairing (position_embedding.py:509-514): element 2i rotates with 2i + 1, both in one vector
      Vec16 out_lo = lo, out_hi = hi;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int dl = c * 8 + e, dh = D / 2 + c * 8 + e;
        if (dl < R) {
          const float other = (e & 1) == 0 ? -static_cast<float>(lo.h[e + 1]) : static_cast<float>(lo.h[e - 1]);
          out_lo.h[e] = static_cast<half_t>(cs_lds[dl] * static_cast<float>(lo.h[e]) + sn_lds[dl] * other);
        }
        if (dh < R) {
          const float other = (e & 1) == 0 ? -static_cast<float>(hi.h[e + 1]) : static_cast<float>(hi.h[e - 1]);
          out_hi.h[e] = static_cast<half_t>(cs_lds[dh] * static_cast<float>(hi.h[e]) + sn_lds[dh] * other);
        }
      }
      lo = out_lo;
      hi = out_hi;
    } else if (apply_rope > 0 && h < num_q_heads + num_kv_heads && R < D) {
      // only the first R features rotate, in pairs (d, d + R/2) that are no longer this thread's two
      // vectors (python/tvm/relax/frontend/nn/llm/position_embedding.py:507-520): element by element, the
      // partner read from the input row
      const half_t* row = qkv + (s * fused_heads + h) * D;
      Vec16 out_lo = lo, out_hi = hi;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int dl = c * 8 + e, dh = D / 2 + c * 8 + e;
        if (dl < R) {
          const float other = dl < R / 2 ? -static_cast<float>(row[dl + R / 2]) : static_cast<float>(row[dl - R / 2]);
          out_lo.h[e] = static_cast<half_t>(cs_lds[dl] * static_cast<float>(lo.h[e]) + sn_lds[dl] * other);
        }
        if (dh < R) {
          const float other = dh < R / 2 ? -static_cast<float>(row[dh + R / 2]) : static_cast<float>(row[dh - R / 2]);
          out_hi.h[e] = static_cast<half_t>(cs_lds[dh] * static_cast<float>(hi.h[e]) + sn_lds[dh] * other);
        }
      }
      lo = out_lo;
      hi = out_hi;
    } else if (apply_rope > 0 && h < num_q_heads + num_kv_heads) {
      Vec16 out_lo, out_hi;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xl = static_cast<float>(lo.h[e]);
        const float xh = static_cast<float>(hi.h[e]);
        out_lo.h[e] = static_cast<half_t>(cs_lds[c * 8 + e] * xl + sn_lds[c * 8 + e] * (-xh));
        out_hi.h[e] = static_cast<half_t>(cs_lds[D / 2 + c * 8 + e] * xh + sn_lds[D / 2 + c * 8 + e] * xl);
      }
      lo = out_lo;
      hi = out_hi;
    }
    st16(dst + c * 8, lo);
    st16(dst + D / 2 + c * 8, hi);
    if (APPEND && h >= num_q_heads) {
      const int32_t slot = append_position_map[s];
      if (slot != -1) {
        const int kv = h >= num_q_heads + num_kv_heads;
        const int head = h - num_q_heads - kv * num_kv_heads;
        half_t* row = pages + ((static_cast<int64_t>(slot / page_size) * 2 + kv) * num_kv_heads + head) *
                                  (static_cast<int64_t>(page_size) * D) + (slot % page_size) * D;
        st16(row + c * 8, lo);
        st16(row + D / 2 + c * 8, hi);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------
// transpose_append: k|v[i, h, :] -> pages[p / ps, 0|1, h, p % ps, :], p = position_map[i] != -1
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void transpose_append_kernel(half_t* __restrict__ pages,
                                                               const half_t* __restrict__ k_data,
                                                               const half_t* __restrict__ v_data,
                                                               const int32_t* __restrict__ position_map,
                                                               int64_t ntoken, int num_kv_heads, int page_size,
                                                               int head_dim) {
  const int chunks = head_dim / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int c = gid % chunks;
  const int64_t row = gid / chunks;  // (token, kv head)
  if (row >= ntoken * num_kv_heads) return;
  const int64_t i = row / num_kv_heads;
  const int h = row % num_kv_heads;
  const int32_t position = position_map[i];
  if (position == -1) return;
  const int64_t page = position / page_size;
  const int slot = position % page_size;
  const int64_t head_stride = static_cast<int64_t>(page_size) * head_dim;
  half_t* kdst = pages + ((page * 2 + 0) * num_kv_heads + h) * head_stride + slot * head_dim + c * 8;
  half_t* vdst = kdst + num_kv_heads * head_stride;
  st16(kdst, ld16(k_data + row * head_dim + c * 8));
  st16(vdst, ld16(v_data + row * head_dim + c * 8));
}

__global__ __launch_bounds__(256) void transpose_append_mla_kernel(half_t* __restrict__ pages,
                                                                   const half_t* __restrict__ kv_data,
                                                                   const int32_t* __restrict__ position_map,
                                                                   int64_t ntoken, int d_qk) {
  const int chunks = d_qk / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int c = gid % chunks;
  const int64_t i = gid / chunks;
  if (i >= ntoken) return;
  const int32_t position = position_map[i];
  if (position == -1) return;
  // pages (num_pages, page_size, d_qk): slot p lives at row p of the flattened (slots, d_qk) view.
  st16(pages + static_cast<int64_t>(position) * d_qk + c * 8, ld16(kv_data + i * d_qk + c * 8));
}

// ------------------------------------------------------------------------------------------
// copy_single_page: first copy_length slots of every head, K and V.
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void copy_single_page_kernel(half_t* __restrict__ pages, int64_t src_page,
                                                               int64_t tgt_page, int copy_length, int num_heads,
                                                               int page_size, int head_dim) {
  const int chunks = head_dim / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t total = static_cast<int64_t>(2) * num_heads * copy_length * chunks;
  if (gid >= total) return;
  const int c = gid % chunks;
  const int slot = (gid / chunks) % copy_length;
  const int kvh = gid / (static_cast<int64_t>(chunks) * copy_length);  // (k|v, head) flattened
  const int64_t page_stride = static_cast<int64_t>(2) * num_heads * page_size * head_dim;
  const int64_t off = (static_cast<int64_t>(kvh) * page_size + slot) * head_dim + c * 8;
  st16(pages + tgt_page * page_stride + off, ld16(pages + src_page * page_stride + off));
}

__global__ __launch_bounds__(256) void copy_single_page_mla_kernel(half_t* __restrict__ pages, int64_t src_page,
                                                                   int64_t tgt_page, int copy_length,
                                                                   int page_size, int d_qk) {
  const int chunks = d_qk / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (gid >= static_cast<int64_t>(copy_length) * chunks) return;
  const int64_t page_stride = static_cast<int64_t>(page_size) * d_qk;
  st16(pages + tgt_page * page_stride + gid * 8, ld16(pages + src_page * page_stride + gid * 8));
}

// ------------------------------------------------------------------------------------------
// debug_get_kv: gather rows by slot id into (num_layers, seqlen, H, D)[layer_id].
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void debug_get_kv_kernel(const half_t* __restrict__ pages,
                                                           const int32_t* __restrict__ position_map,
                                                           half_t* __restrict__ k_data, half_t* __restrict__ v_data,
                                                           int64_t layer_id, int64_t seqlen, int num_kv_heads,
                                                           int page_size, int head_dim) {
  const int chunks = head_dim / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int c = gid % chunks;
  const int64_t row = gid / chunks;  // (p, h)
  if (row >= seqlen * num_kv_heads) return;
  const int64_t p = row / num_kv_heads;
  const int h = row % num_kv_heads;
  const int32_t position = position_map[p];
  const int64_t page = position / page_size;
  const int slot = position % page_size;
  const int64_t head_stride = static_cast<int64_t>(page_size) * head_dim;
  const half_t* ksrc = pages + ((page * 2 + 0) * num_kv_heads + h) * head_stride + slot * head_dim + c * 8;
  const half_t* vsrc = ksrc + num_kv_heads * head_stride;
  const int64_t dst = ((layer_id * seqlen + p) * num_kv_heads + h) * head_dim + c * 8;
  st16(k_data + dst, ld16(ksrc));
  st16(v_data + dst, ld16(vsrc));
}

__global__ __launch_bounds__(256) void debug_get_kv_mla_kernel(const half_t* __restrict__ pages,
                                                               const int32_t* __restrict__ position_map,
                                                               half_t* __restrict__ kv_data, int64_t layer_id,
                                                               int64_t seqlen, int d_qk) {
  const int chunks = d_qk / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int c = gid % chunks;
  const int64_t p = gid / chunks;
  if (p >= seqlen) return;
  st16(kv_data + (layer_id * seqlen + p) * d_qk + c * 8,
       ld16(pages + static_cast<int64_t>(position_map[p]) * d_qk + c * 8));
}

// ------------------------------------------------------------------------------------------
// compact_kv_copy: per batch row, copies run in order (a later destination may be an earlier
// source), so one thread walks the whole list for its (b, k|v, head, 16-byte piece).
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void compact_kv_copy_kernel(half_t* __restrict__ pages,
                                                              const int32_t* __restrict__ copy_length_indptr,
                                                              const int32_t* __restrict__ copy_src_dst_pos,
                                                              int batch_size, int total_copy_length, int num_heads,
                                                              int page_size, int head_dim) {
  const int chunks = head_dim / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t per_batch = static_cast<int64_t>(2) * num_heads * chunks;
  if (gid >= batch_size * per_batch) return;
  const int b = gid / per_batch;
  const int rem = gid % per_batch;
  const int c = rem % chunks;
  const int kvh = rem / chunks;  // (k|v, head) flattened: kv = kvh / num_heads, h = kvh % num_heads
  const int kv = kvh / num_heads;
  const int h = kvh % num_heads;
  const int64_t head_stride = static_cast<int64_t>(page_size) * head_dim;
  for (int i = copy_length_indptr[b]; i < copy_length_indptr[b + 1]; ++i) {
    const int32_t src_pos = copy_src_dst_pos[i];
    const int32_t dst_pos = copy_src_dst_pos[total_copy_length + i];
    const half_t* src = pages + ((static_cast<int64_t>(src_pos / page_size) * 2 + kv) * num_heads + h) * head_stride +
                        (src_pos % page_size) * head_dim + c * 8;
    half_t* dst = pages + ((static_cast<int64_t>(dst_pos / page_size) * 2 + kv) * num_heads + h) * head_stride +
                  (dst_pos % page_size) * head_dim + c * 8;
    st16(dst, ld16(src));
  }
}

// ------------------------------------------------------------------------------------------
// merge_state_inplace (python/tvm/relax/frontend/nn/llm/_decode_kernels.py:497-521):
//   smax = max(s, s'); w = 2^(s-smax), w' = 2^(s'-smax)
//   V = V*w/(w+w') + V'*w'/(w+w') (rounded to fp16);  S = log2(w+w') + smax
// A row (n, h) is owned by D/8 consecutive lanes of ONE wavefront: every lane reads S before
// lane 0 of the group overwrites it (lock-step execution inside the wavefront).
// ------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void merge_state_inplace_kernel(half_t* __restrict__ v, float* __restrict__ s,
                                                                  const half_t* __restrict__ v_other,
                                                                  const float* __restrict__ s_other, int64_t rows,
                                                                  int d, int lanes_per_row) {
  // lanes_per_row: d / 8 rounded up to a divisor of 64, so that the lanes of a row share a wavefront
  const int chunks = d / 8;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int c = gid % lanes_per_row;
  const int64_t row = gid / lanes_per_row;
  if (row >= rows || c >= chunks) return;
  float s_val = s[row];
  float s_other_val = s_other[row];
  const float s_max = fmaxf(s_val, s_other_val);
  s_val = exp2f(s_val - s_max);
  s_other_val = exp2f(s_other_val - s_max);
  const float scale = s_val / (s_val + s_other_val);
  const float other_scale = s_other_val / (s_val + s_other_val);
  Vec16 a = ld16(v + row * d + c * 8);
  const Vec16 b = ld16(v_other + row * d + c * 8);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a.h[e] = static_cast<half_t>(static_cast<float>(a.h[e]) * scale + static_cast<float>(b.h[e]) * other_scale);
  }
  st16(v + row * d + c * 8, a);
  if (c == 0) s[row] = log2f(s_val + s_other_val) + s_max;
}

// The split-rotary kernel for what the vectorised one above is not built for: float32 storage and head dims
// outside its list (any even head dim up to kMaxHeadDim).  The same tables and the same arithmetic, one
// element per thread and step: element e of a rotating head becomes cos * x[e] + sin * partner(e), the partner
// being -x[e + R/2] / x[e - R/2], or -x[e + 1] / x[e - 1] for the gptj pairing.
template <typename T, bool APPEND>
__global__ __launch_bounds__(256) void fused_rope_any_kernel(const T* __restrict__ qkv, const int32_t* __restrict__ position_map,
                                                             T* __restrict__ q, T* __restrict__ k, T* __restrict__ v,
                                                             int num_q_heads, int num_kv_heads, int D, int apply_rope,
                                                             float scale, RopeDivisors div, int table_is_inverse,
                                                             int halves_differ, float magnitude,
                                                             const float* __restrict__ ext_factors, T* __restrict__ pages,
                                                             const int32_t* __restrict__ append_position_map, int page_size,
                                                             int rotary_dim, int interleaved) {
  __shared__ float cs_lds[kMaxHeadDim];
  __shared__ float sn_lds[kMaxHeadDim];
  const int R = rotary_dim;
  const int64_t s = blockIdx.x;  // token
  const int fused_heads = num_q_heads + 2 * num_kv_heads;
  if (apply_rope > 0) {
    const float pos_scaled = static_cast<float>(position_map[s]) * scale;
    for (int i = threadIdx.x; i < (halves_differ ? R : R / 2); i += 256) {
      float freq;
      if (table_is_inverse) {
        freq = pos_scaled * div.v[i];
      } else {
        freq = pos_scaled / (ext_factors != nullptr ? ext_factors[i] * div.v[i] : div.v[i]);
      }
      const float cs = cosf(freq) * magnitude, sn = sinf(freq) * magnitude;
      cs_lds[i] = cs;
      sn_lds[i] = sn;
      if (!halves_differ) {
        cs_lds[i + R / 2] = cs;
        sn_lds[i + R / 2] = sn;
      }
    }
    __syncthreads();
  }
  const int32_t slot = APPEND ? append_position_map[s] : -1;
  const int first = q == nullptr ? num_q_heads * D : 0;  // q == NULL: the q rows are left alone
  for (int idx = first + threadIdx.x; idx < fused_heads * D; idx += 256) {
    const int h = idx / D, e = idx - h * D;
    const T* row = qkv + (s * fused_heads + h) * D;
    float x = static_cast<float>(row[e]);
    T result = row[e];
    if (apply_rope > 0 && h < num_q_heads + num_kv_heads && e < R) {
      float other;
      if (interleaved) {
        other = (e & 1) == 0 ? -static_cast<float>(row[e + 1]) : static_cast<float>(row[e - 1]);
      } else {
        other = e < R / 2 ? -static_cast<float>(row[e + R / 2]) : static_cast<float>(row[e - R / 2]);
      }
      result = static_cast<T>(cs_lds[e] * x + sn_lds[e] * other);
    }
    if (h < num_q_heads) {
      q[(s * num_q_heads + h) * D + e] = result;
      continue;
    }
    const int kv = h >= num_q_heads + num_kv_heads;
    const int head = h - num_q_heads - kv * num_kv_heads;
    (kv ? v : k)[(s * num_kv_heads + head) * D + e] = result;
    if (APPEND && slot != -1) {
      pages[((static_cast<int64_t>(slot / page_size) * 2 + kv) * num_kv_heads + head) * (static_cast<int64_t>(page_size) * D) +
            static_cast<int64_t>(slot % page_size) * D + e] = result;
    }
  }
}

// merge_state_inplace for float32 storage: one thread per 4 features; the threads of a row read S before the
// one that owns piece 0 rewrites it only if they share a wavefront, so S goes through registers first and the
// new value is written after every lane of the row has used the old one (rows never straddle wavefronts: the
// lanes per row are a power of two up to 64).
__global__ __launch_bounds__(256) void merge_state_inplace_f32_kernel(float* __restrict__ v, float* __restrict__ s,
                                                                      const float* __restrict__ v_other,
                                                                      const float* __restrict__ s_other, int64_t rows, int d,
                                                                      int lanes_per_row) {
  const int chunks = d / 4;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int lane_in_row = gid % lanes_per_row;
  const int64_t row = gid / lanes_per_row;
  if (row >= rows) return;
  float s_val = s[row];
  float s_other_val = s_other[row];
  const float s_max = fmaxf(s_val, s_other_val);
  s_val = exp2f(s_val - s_max);
  s_other_val = exp2f(s_other_val - s_max);
  const float scale = s_val / (s_val + s_other_val);
  const float other_scale = s_other_val / (s_val + s_other_val);
  for (int c = lane_in_row; c < chunks; c += lanes_per_row) {
    float4_t a = *reinterpret_cast<const float4_t*>(v + row * d + c * 4);
    const float4_t b = *reinterpret_cast<const float4_t*>(v_other + row * d + c * 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) a[e] = a[e] * scale + b[e] * other_scale;
    *reinterpret_cast<float4_t*>(v + row * d + c * 4) = a;
  }
  if (lane_in_row == 0) s[row] = log2f(s_val + s_other_val) + s_max;
}

inline dim3 grid_for(int64_t threads, int block = 256) { return dim3(static_cast<unsigned>((threads + block - 1) / block)); }

}  // namespace tvmkv

using namespace tvmkv;

extern "C" {

// The table of floats a RoPE variant needs (head_dim / 2, or head_dim when the two halves differ), in
// float32 arithmetic in the reference's order of operations (position_embedding.py:32-67 default,
// :130-161 llama3, :164-188 longrope, :191-255 yarn).  Returns whether the table holds inverse
// frequencies (multiply) or divisors.
static bool rope_table(const tvmkv_rope_scaling* scaling, int head_dim, double rope_theta, int64_t seq_len,
                       const float** ext_factors, RopeDivisors* table, float* magnitude, bool* halves_differ) {
  *halves_differ = false;
  const float theta = static_cast<float>(rope_theta);
  const int type = scaling == nullptr ? TVMKV_ROPE_FREQ_DEFAULT : scaling->rope_type;
  const float d_range = static_cast<float>(head_dim);
  *magnitude = 1.0f;
  auto power = [&](int i) { return powf(theta, static_cast<float>((i * 2) % head_dim) / d_range); };
  if (type == TVMKV_ROPE_FREQ_GPTJ) {  // element d rotates at the frequency of its pair d / 2: one entry per element
    KV_CHECK(*ext_factors == nullptr) << "fused_rope: rope_ext_factors needs a longrope scaling description";
    *halves_differ = true;
    for (int d = 0; d < head_dim; ++d) table->v[d] = powf(theta, static_cast<float>((2 * (d / 2)) % head_dim) / d_range);
    return false;
  }
  if (type == TVMKV_ROPE_FREQ_LLAMA4) {  // position_embedding.py:79-127: one inverse frequency per element, of pair d / 2
    KV_CHECK(*ext_factors == nullptr) << "fused_rope: rope_ext_factors needs a longrope scaling description";
    KV_CHECK(scaling->factor != 0 && scaling->low_freq_factor != 0) << "fused_rope: llama4 scaling needs factor != 0 and low_freq_factor != 0";
    *halves_differ = true;
    const bool hard = scaling->high_freq_factor == scaling->low_freq_factor;
    const double inv_diff = hard ? 0.0 : 1.0 / (scaling->high_freq_factor - scaling->low_freq_factor);
    const float inv_factor = static_cast<float>(1.0 / scaling->factor);
    const float alpha = static_cast<float>(static_cast<double>(scaling->original_max_position_embeddings) / (2 * M_PI) * inv_diff);
    const float beta = static_cast<float>(scaling->low_freq_factor * inv_diff);
    const float threshold = static_cast<float>(static_cast<double>(scaling->original_max_position_embeddings) / scaling->low_freq_factor);
    for (int d = 0; d < head_dim; ++d) {
      const float orig = 1.0f / powf(theta, static_cast<float>(2 * (d / 2)) / d_range);
      if (hard) {
        const float wavelength = static_cast<float>(2 * M_PI) / orig;
        table->v[d] = wavelength > threshold ? orig / static_cast<float>(scaling->factor) : orig;
      } else {
        const float smooth = fmaxf(0.0f, fminf(1.0f, alpha * orig - beta));
        table->v[d] = (1.0f - smooth) * orig * inv_factor + smooth * orig;
      }
    }
    return true;
  }
  if (type == TVMKV_ROPE_FREQ_DEFAULT || type == TVMKV_ROPE_FREQ_LONGROPE) {
    for (int i = 0; i < head_dim / 2; ++i) table->v[i] = power(i);
    if (type == TVMKV_ROPE_FREQ_LONGROPE) {
      KV_CHECK(scaling->original_max_position_embeddings > 0 && scaling->max_position_embeddings > 0)
          << "fused_rope: longrope needs max_position_embeddings and original_max_position_embeddings";
      const double scale = static_cast<double>(scaling->max_position_embeddings) /
                           static_cast<double>(scaling->original_max_position_embeddings);
      if (scale > 1.0) {
        *magnitude = static_cast<float>(
            std::sqrt(1.0 + std::log(scale) / std::log(static_cast<double>(scaling->original_max_position_embeddings))));
      }
      // the factor tensor holds the long factors, then the short ones (position_embedding.py:601-668)
      if (*ext_factors != nullptr && seq_len <= scaling->original_max_position_embeddings) *ext_factors += head_dim / 2;
    } else {
      KV_CHECK(*ext_factors == nullptr) << "fused_rope: rope_ext_factors needs a longrope scaling description";
    }
    return false;
  }
  KV_CHECK(*ext_factors == nullptr) << "fused_rope: rope_ext_factors needs a longrope scaling description";
  if (type == TVMKV_ROPE_FREQ_LLAMA3) {
    KV_CHECK(scaling->high_freq_factor != scaling->low_freq_factor && scaling->factor != 0)
        << "fused_rope: llama3 scaling needs factor != 0 and high_freq_factor != low_freq_factor";
    const double inv_diff = 1.0 / (scaling->high_freq_factor - scaling->low_freq_factor);
    const float inv_factor = static_cast<float>(1.0 / scaling->factor);
    const float alpha = static_cast<float>(static_cast<double>(scaling->original_max_position_embeddings) / (2 * M_PI) * inv_diff);
    const float beta = static_cast<float>(scaling->low_freq_factor * inv_diff);
    for (int i = 0; i < head_dim / 2; ++i) {
      const float orig = 1.0f / power(i);
      const float smooth = fmaxf(0.0f, fminf(1.0f, alpha * orig - beta));
      table->v[i] = (1.0f - smooth) * orig * inv_factor + smooth * orig;
    }
    return true;
  }
  KV_UNSUPPORTED(type != TVMKV_ROPE_FREQ_YARN)
      << "fused_rope: rope type " << type << " is not built (default, llama3, longrope, yarn, gptj, llama4)";
  KV_CHECK(scaling->factor != 0 && rope_theta > 1.0) << "fused_rope: yarn scaling needs factor != 0 and theta > 1";
  const double inv_theta_log_scale = 1.0 / (2.0 * std::log(rope_theta));  // kv_cache.py:363-365
  auto correction_dim = [&](double rotations) {
    return head_dim * std::log(static_cast<double>(scaling->original_max_position_embeddings) / (rotations * 2 * M_PI)) *
           inv_theta_log_scale;
  };
  const float low = static_cast<float>(std::max(correction_dim(scaling->beta_fast), 0.0));
  float high = static_cast<float>(std::min(correction_dim(scaling->beta_slow), static_cast<double>(head_dim - 1)));
  if (low == high) high += 0.001f;
  const float factor = static_cast<float>(scaling->factor);
  // the blend is indexed by the element, not by its frequency: the two halves get different angles
  *halves_differ = true;
  for (int d = 0; d < head_dim; ++d) {
    const float freq_power = power(d);
    const float extra = 1.0f / freq_power;
    const float inter = 1.0f / (factor * freq_power);
    const float mask = 1.0f - fmaxf(fminf((static_cast<float>(d) - low) / (high - low), 1.0f), 0.0f);
    table->v[d] = inter * (1.0f - mask) + extra * mask;
  }
  return true;
}

static int fused_rope_impl(const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                           int64_t apply_rope, const float* ext_factors, const tvmkv_rope_scaling* scaling,
                           int64_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                           int32_t head_dim, double rope_scale, double rope_theta, void* pages,
                           const int32_t* append_position_map, int64_t num_pages, int32_t page_size, void* stream,
                           int elem_bits = 16) {
  KV_API_BEGIN();
  KV_CHECK(seq_len >= 0 && num_q_heads > 0 && num_kv_heads > 0) << "fused_rope: bad shape";
  KV_CHECK(elem_bits == 16 || elem_bits == 32) << "fused_rope: elem_bits must be 16 or 32";
  KV_UNSUPPORTED(head_dim <= 0 || head_dim > kMaxHeadDim || head_dim % 2 != 0)
      << "fused_rope: head_dim " << head_dim << " is not built (even head dims up to " << kMaxHeadDim << ")";
  const bool vectorised = elem_bits == 16 && (head_dim == 64 || head_dim == 128 || head_dim == 256 || head_dim == 80 ||
                                              head_dim == 96 || head_dim == 112);
  if (seq_len == 0) return TVMKV_OK;
  const bool append = pages != nullptr;
  KV_CHECK(qkv && position_map && (q || append) && k && v) << "fused_rope: NULL tensor";
  if (append) {
    KV_CHECK(append_position_map != nullptr && page_size > 0) << "fused_rope_append: NULL position map or bad page size";
    KV_CHECK(num_pages * page_size <= INT32_MAX) << "fused_rope_append: slot ids do not fit int32";
  }
  const int rotary_dim = scaling != nullptr && scaling->rotary_dim > 0 ? scaling->rotary_dim : head_dim;
  KV_CHECK(rotary_dim % 2 == 0 && rotary_dim <= head_dim)
      << "fused_rope: rotary_dim " << rotary_dim << " must be even and at most head_dim " << head_dim;
  RopeDivisors div;
  float magnitude = 1.0f;
  bool halves_differ = false;
  const bool table_is_inverse =
      rope_table(scaling, rotary_dim, rope_theta, seq_len, &ext_factors, &div, &magnitude, &halves_differ);
  KV_CHECK(seq_len < (int64_t{1} << 31)) << "fused_rope: too many tokens for one launch";
  const float scale = static_cast<float>(rope_scale);
  auto launch = [&](auto kernel) {
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(seq_len)), dim3(256), 0, as_stream(stream), static_cast<const half_t*>(qkv),
                       position_map, static_cast<half_t*>(q), static_cast<half_t*>(k), static_cast<half_t*>(v),
                       seq_len, num_q_heads, num_kv_heads, static_cast<int>(apply_rope > 0), scale, div,
                       static_cast<int>(table_is_inverse), static_cast<int>(halves_differ), magnitude, ext_factors,
                       static_cast<half_t*>(pages),
                       append_position_map, page_size, rotary_dim,
                       static_cast<int>(scaling != nullptr && scaling->rope_type == TVMKV_ROPE_FREQ_GPTJ));
  };
  auto launch_any = [&](auto kernel, auto* typed_null) {
    using T = std::remove_pointer_t<decltype(typed_null)>;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(seq_len)), dim3(256), 0, as_stream(stream), static_cast<const T*>(qkv),
                       position_map, static_cast<T*>(q), static_cast<T*>(k), static_cast<T*>(v), num_q_heads, num_kv_heads,
                       head_dim, static_cast<int>(apply_rope > 0), scale, div, static_cast<int>(table_is_inverse),
                       static_cast<int>(halves_differ), magnitude, ext_factors, static_cast<T*>(pages), append_position_map,
                       page_size, rotary_dim, static_cast<int>(scaling != nullptr && scaling->rope_type == TVMKV_ROPE_FREQ_GPTJ));
  };
  if (!vectorised) {
    if (elem_bits == 32) {
      if (append) launch_any(fused_rope_any_kernel<float, true>, static_cast<float*>(nullptr));
      else launch_any(fused_rope_any_kernel<float, false>, static_cast<float*>(nullptr));
    } else {
      if (append) launch_any(fused_rope_any_kernel<half_t, true>, static_cast<half_t*>(nullptr));
      else launch_any(fused_rope_any_kernel<half_t, false>, static_cast<half_t*>(nullptr));
    }
  } else if (head_dim == 64) {
    if (append) launch(fused_rope_kernel<64, true>); else launch(fused_rope_kernel<64, false>);
  } else if (head_dim == 128) {
    if (append) launch(fused_rope_kernel<128, true>); else launch(fused_rope_kernel<128, false>);
  } else if (head_dim == 80) {
    if (append) launch(fused_rope_kernel<80, true>); else launch(fused_rope_kernel<80, false>);
  } else if (head_dim == 96) {
    if (append) launch(fused_rope_kernel<96, true>); else launch(fused_rope_kernel<96, false>);
  } else if (head_dim == 112) {
    if (append) launch(fused_rope_kernel<112, true>); else launch(fused_rope_kernel<112, false>);
  } else {
    if (append) launch(fused_rope_kernel<256, true>); else launch(fused_rope_kernel<256, false>);
  }
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_fused_rope(const void* qkv, const int32_t* position_map, void* q, void* k, void* v, int64_t apply_rope,
                     int64_t seq_len, int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim,
                     double rope_scale, double rope_theta, void* stream) {
  return fused_rope_impl(qkv, position_map, q, k, v, apply_rope, nullptr, nullptr, seq_len, num_q_heads, num_kv_heads,
                         head_dim, rope_scale, rope_theta, nullptr, nullptr, 0, 0, stream);
}

int tvmkv_fused_rope_scaled(const void* qkv, const int32_t* position_map, void* q, void* k, void* v, int64_t apply_rope,
                            const float* rope_ext_factors, const tvmkv_rope_scaling* scaling, int64_t seq_len,
                            int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, double rope_scale,
                            double rope_theta, void* stream) {
  return fused_rope_impl(qkv, position_map, q, k, v, apply_rope, rope_ext_factors, scaling, seq_len, num_q_heads,
                         num_kv_heads, head_dim, rope_scale, rope_theta, nullptr, nullptr, 0, 0, stream);
}

int tvmkv_fused_rope_append_scaled(const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                                   int64_t apply_rope, const float* rope_ext_factors, const tvmkv_rope_scaling* scaling,
                                   void* pages, const int32_t* append_position_map, int64_t seq_len, int32_t num_q_heads,
                                   int32_t num_kv_heads, int32_t head_dim, int64_t num_pages, int32_t page_size,
                                   double rope_scale, double rope_theta, void* stream) {
  if (seq_len > 0 && pages == nullptr) {
    ::tvmkv::SetLastError("fused_rope_append: NULL pages");
    return TVMKV_EINVAL;
  }
  return fused_rope_impl(qkv, position_map, q, k, v, apply_rope, rope_ext_factors, scaling, seq_len, num_q_heads,
                         num_kv_heads, head_dim, rope_scale, rope_theta, pages, append_position_map, num_pages, page_size,
                         stream);
}

int tvmkv_fused_rope_append(const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                            int64_t apply_rope, void* pages, const int32_t* append_position_map, int64_t seq_len,
                            int32_t num_q_heads, int32_t num_kv_heads, int32_t head_dim, int64_t num_pages,
                            int32_t page_size, double rope_scale, double rope_theta, void* stream) {
  if (seq_len > 0 && pages == nullptr) {
    ::tvmkv::SetLastError("fused_rope_append: NULL pages");
    return TVMKV_EINVAL;
  }
  return fused_rope_impl(qkv, position_map, q, k, v, apply_rope, nullptr, nullptr, seq_len, num_q_heads, num_kv_heads,
                         head_dim, rope_scale, rope_theta, pages, append_position_map, num_pages, page_size, stream);
}

static void check_slot_layout(const char* what, int32_t page_size, int32_t head_dim) {
  KV_CHECK(page_size > 0) << what << ": page_size must be positive";
  KV_CHECK(head_dim > 0 && head_dim % 8 == 0) << what << ": feature dim " << head_dim << " must be a multiple of 8";
}

int tvmkv_kv_cache_transpose_append(void* pages, const void* k_data, const void* v_data,
                                    const int32_t* position_map, int64_t ntoken, int64_t num_pages,
                                    int32_t num_kv_heads, int32_t page_size, int32_t head_dim, void* stream) {
  KV_API_BEGIN();
  check_slot_layout("transpose_append", page_size, head_dim);
  KV_CHECK(ntoken >= 0 && num_kv_heads > 0) << "transpose_append: bad shape";
  KV_CHECK(num_pages * page_size <= INT32_MAX) << "transpose_append: slot ids do not fit int32";
  if (ntoken == 0) return TVMKV_OK;
  KV_CHECK(pages && k_data && v_data && position_map) << "transpose_append: NULL tensor";
  const int64_t threads = ntoken * num_kv_heads * (head_dim / 8);
  hipLaunchKernelGGL(transpose_append_kernel, grid_for(threads), dim3(256), 0, as_stream(stream),
                     static_cast<half_t*>(pages), static_cast<const half_t*>(k_data),
                     static_cast<const half_t*>(v_data), position_map, ntoken, num_kv_heads, page_size, head_dim);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_kv_cache_transpose_append_mla(void* pages, const void* kv_data, const int32_t* position_map,
                                        int64_t ntoken, int64_t num_pages, int32_t page_size, int32_t d_qk,
                                        void* stream) {
  KV_API_BEGIN();
  check_slot_layout("transpose_append_mla", page_size, d_qk);
  KV_CHECK(ntoken >= 0) << "transpose_append_mla: bad shape";
  if (ntoken == 0) return TVMKV_OK;
  KV_CHECK(pages && kv_data && position_map) << "transpose_append_mla: NULL tensor";
  hipLaunchKernelGGL(transpose_append_mla_kernel, grid_for(ntoken * (d_qk / 8)), dim3(256), 0, as_stream(stream),
                     static_cast<half_t*>(pages), static_cast<const half_t*>(kv_data), position_map, ntoken, d_qk);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_copy_single_page(void* pages, int64_t src_page_id, int64_t tgt_page_id, int64_t copy_length,
                           int64_t num_pages, int32_t num_kv_heads, int32_t page_size, int32_t head_dim,
                           void* stream) {
  KV_API_BEGIN();
  check_slot_layout("copy_single_page", page_size, head_dim);
  KV_CHECK(src_page_id >= 0 && src_page_id < num_pages && tgt_page_id >= 0 && tgt_page_id < num_pages)
      << "copy_single_page: page id out of range";
  KV_CHECK(copy_length >= 0 && copy_length <= page_size) << "copy_single_page: copy_length out of range";
  if (copy_length == 0) return TVMKV_OK;
  const int64_t threads = 2 * num_kv_heads * copy_length * (head_dim / 8);
  hipLaunchKernelGGL(copy_single_page_kernel, grid_for(threads), dim3(256), 0, as_stream(stream),
                     static_cast<half_t*>(pages), src_page_id, tgt_page_id, static_cast<int>(copy_length),
                     num_kv_heads, page_size, head_dim);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_copy_single_page_mla(void* pages, int64_t src_page_id, int64_t tgt_page_id, int64_t copy_length,
                               int64_t num_pages, int32_t page_size, int32_t d_qk, void* stream) {
  KV_API_BEGIN();
  check_slot_layout("copy_single_page_mla", page_size, d_qk);
  KV_CHECK(src_page_id >= 0 && src_page_id < num_pages && tgt_page_id >= 0 && tgt_page_id < num_pages)
      << "copy_single_page_mla: page id out of range";
  KV_CHECK(copy_length >= 0 && copy_length <= page_size) << "copy_single_page_mla: copy_length out of range";
  if (copy_length == 0) return TVMKV_OK;
  hipLaunchKernelGGL(copy_single_page_mla_kernel, grid_for(copy_length * (d_qk / 8)), dim3(256), 0,
                     as_stream(stream), static_cast<half_t*>(pages), src_page_id, tgt_page_id,
                     static_cast<int>(copy_length), page_size, d_qk);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_kv_cache_debug_get_kv(const void* pages, const int32_t* position_map, void* k_data, void* v_data,
                                int64_t layer_id, int64_t seqlen, int64_t num_pages, int32_t num_kv_heads,
                                int32_t page_size, int32_t head_dim, void* stream) {
  KV_API_BEGIN();
  check_slot_layout("debug_get_kv", page_size, head_dim);
  if (seqlen == 0) return TVMKV_OK;
  KV_CHECK(pages && position_map && k_data && v_data) << "debug_get_kv: NULL tensor";
  hipLaunchKernelGGL(debug_get_kv_kernel, grid_for(seqlen * num_kv_heads * (head_dim / 8)), dim3(256), 0,
                     as_stream(stream), static_cast<const half_t*>(pages), position_map,
                     static_cast<half_t*>(k_data), static_cast<half_t*>(v_data), layer_id, seqlen, num_kv_heads,
                     page_size, head_dim);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_kv_cache_debug_get_kv_mla(const void* pages, const int32_t* position_map, void* kv_data, int64_t layer_id,
                                    int64_t seqlen, int64_t num_pages, int32_t page_size, int32_t d_qk,
                                    void* stream) {
  KV_API_BEGIN();
  check_slot_layout("debug_get_kv_mla", page_size, d_qk);
  if (seqlen == 0) return TVMKV_OK;
  KV_CHECK(pages && position_map && kv_data) << "debug_get_kv_mla: NULL tensor";
  hipLaunchKernelGGL(debug_get_kv_mla_kernel, grid_for(seqlen * (d_qk / 8)), dim3(256), 0, as_stream(stream),
                     static_cast<const half_t*>(pages), position_map, static_cast<half_t*>(kv_data), layer_id,
                     seqlen, d_qk);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_compact_kv_copy(void* pages, const int32_t* copy_length_indptr, const int32_t* copy_src_dst_pos,
                          int32_t batch_size, int32_t total_copy_length, int64_t num_pages, int32_t num_kv_heads,
                          int32_t page_size, int32_t head_dim, void* stream) {
  KV_API_BEGIN();
  check_slot_layout("compact_kv_copy", page_size, head_dim);
  if (batch_size == 0 || total_copy_length == 0) return TVMKV_OK;
  KV_CHECK(pages && copy_length_indptr && copy_src_dst_pos) << "compact_kv_copy: NULL tensor";
  const int64_t threads = static_cast<int64_t>(batch_size) * 2 * num_kv_heads * (head_dim / 8);
  hipLaunchKernelGGL(compact_kv_copy_kernel, grid_for(threads), dim3(256), 0, as_stream(stream),
                     static_cast<half_t*>(pages), copy_length_indptr, copy_src_dst_pos, batch_size,
                     total_copy_length, num_kv_heads, page_size, head_dim);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

int tvmkv_merge_state_inplace(void* v, float* s, const void* v_other, const float* s_other, int64_t n, int32_t h,
                              int32_t d, void* stream) {
  KV_API_BEGIN();
  KV_CHECK(n >= 0 && h > 0) << "merge_state_inplace: bad shape";
  // the lanes of a row share a wavefront: D/8 rounded up to a power of two lanes per row
  KV_UNSUPPORTED(d <= 0 || d % 8 != 0 || d > 512)
      << "merge_state_inplace: head dim " << d << " is not built (a multiple of 8 up to 512)";
  int lanes_per_row = 1;
  while (lanes_per_row < d / 8) lanes_per_row *= 2;
  if (n == 0) return TVMKV_OK;
  KV_CHECK(v && s && v_other && s_other) << "merge_state_inplace: NULL tensor";
  const int64_t rows = n * h;
  hipLaunchKernelGGL(merge_state_inplace_kernel, grid_for(rows * lanes_per_row), dim3(256), 0, as_stream(stream),
                     static_cast<half_t*>(v), s, static_cast<const half_t*>(v_other), s_other, rows, d, lanes_per_row);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

}  // extern "C"

namespace tvmkv {

int typed_fused_rope(int elem_bits, const void* qkv, const int32_t* position_map, void* q, void* k, void* v,
                     int64_t apply_rope, const float* rope_ext_factors, const tvmkv_rope_scaling* scaling, void* pages,
                     const int32_t* append_position_map, int64_t seq_len, int32_t num_q_heads, int32_t num_kv_heads,
                     int32_t head_dim, int64_t num_pages, int32_t page_size, double rope_scale, double rope_theta,
                     void* stream) {
  return fused_rope_impl(qkv, position_map, q, k, v, apply_rope, rope_ext_factors, scaling, seq_len, num_q_heads, num_kv_heads,
                         head_dim, rope_scale, rope_theta, pages, append_position_map, num_pages, page_size, stream, elem_bits);
}

int typed_merge_state_inplace(int elem_bits, void* v, float* s, const void* v_other, const float* s_other, int64_t n,
                              int32_t h, int32_t d, void* stream) {
  if (elem_bits == 16) return tvmkv_merge_state_inplace(v, s, v_other, s_other, n, h, d, stream);
  KV_API_BEGIN();
  KV_CHECK(elem_bits == 32) << "merge_state_inplace: elem_bits must be 16 or 32";
  KV_CHECK(n >= 0 && h > 0) << "merge_state_inplace: bad shape";
  KV_UNSUPPORTED(d <= 0 || d % 4 != 0 || d > 512)
      << "merge_state_inplace: head dim " << d << " is not built (float32: a multiple of 4 up to 512)";
  if (n == 0) return TVMKV_OK;
  KV_CHECK(v && s && v_other && s_other) << "merge_state_inplace: NULL tensor";
  int lanes_per_row = 1;
  while (lanes_per_row < d / 4 && lanes_per_row < 64) lanes_per_row *= 2;
  const int64_t rows = n * h;
  hipLaunchKernelGGL(merge_state_inplace_f32_kernel, grid_for(rows * lanes_per_row), dim3(256), 0, as_stream(stream),
                     static_cast<float*>(v), s, static_cast<const float*>(v_other), s_other, rows, d, lanes_per_row);
  KV_LAUNCH_CHECK();
  KV_API_END();
}

InlineRopeHost inline_rope_table(const ::tvmkv_rope_scaling* scaling, int head_dim, double rope_theta) {
  KV_CHECK(head_dim > 0 && head_dim <= kMaxHeadDim && head_dim % 2 == 0) << "in-kernel RoPE: head_dim " << head_dim;
  InlineRopeHost out{};
  RopeDivisors table{};
  const float* no_factors = nullptr;  // the attention kernels take no factor tensor (_kernel_common.py:115-127)
  bool differ = false;
  tvmkv_rope_scaling whole_head{};
  if (scaling != nullptr) {
    whole_head = *scaling;
    whole_head.rotary_dim = 0;  // the attention kernels rotate the whole head, whatever the split-rotary kernel does
  }
  out.inverse = rope_table(scaling != nullptr ? &whole_head : nullptr, head_dim, rope_theta, /*seq_len=*/0, &no_factors, &table,
                           &out.magnitude, &differ)
                    ? 1
                    : 0;
  out.halves_differ = differ ? 1 : 0;
  for (int d = 0; d < head_dim; ++d) out.v[d] = differ ? table.v[d] : table.v[d % (head_dim / 2)];
  return out;
}

}  // namespace tvmkv
