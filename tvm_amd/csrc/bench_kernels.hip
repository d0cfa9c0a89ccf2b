// Measurement aids of the benchmark, built into their own library (libtvmkv_bench.so) so that the
// product library carries product code only: plain streaming reads and a copy of known size (what the
// memory system of the box delivers; the scale of the hardware traffic counters), a loop of nothing but
// fp16 matrix instructions (what the matrix cores deliver).  None of it has a counterpart in the reference.
#include <hip/hip_runtime.h>

#include <cstdint>

#include "../../include/tvmkv_bench.h"

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));

template <bool NT>  // NT: loads carry the non-temporal hint, as the decode kernel's do
__global__ __launch_bounds__(256) void stream_read_kernel(const uint4* __restrict__ src, int64_t n16,
                                                          uint32_t* __restrict__ sink) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  uint32_t acc = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const u32x4* at = reinterpret_cast<const u32x4*>(src + i);
    const u32x4 v = NT ? __builtin_nontemporal_load(at) : *at;
    acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;  // keeps the loads alive; practically never taken
}

__global__ __launch_bounds__(256) void stream_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                          int64_t n16) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n16; i += stride) dst[i] = src[i];
}

// Every wave runs `iters` rounds of 8 v_mfma_f32_32x32x16_f16 (4 accumulators) on operands it read once
// (8 halfs per lane for A and for B).  Nothing else is in the loop: this is what the matrix pipes of the
// box deliver, and it depends on the operand values (the clock drops with random data).
__global__ __launch_bounds__(256) void mfma_loop_kernel(const _Float16* __restrict__ operands, float* __restrict__ out,
                                                        int iters) {
  const int tid = threadIdx.x;
  const half8 a = *reinterpret_cast<const half8*>(operands + tid * 16);
  const half8 b = *reinterpret_cast<const half8*>(operands + tid * 16 + 8);
  float16v acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
  }
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[j & 3], 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
#pragma unroll
    for (int i = 0; i < 16; ++i) sum += acc[j][i];
  }
  out[static_cast<int64_t>(blockIdx.x) * 256 + tid] = sum;
}

int finish() { return static_cast<int>(hipGetLastError()); }

}  // namespace

extern "C" {

int tvmkvb_stream_read(const void* src, int64_t num_bytes, void* sink, void* stream) {
  if (!src || !sink || num_bytes < 0 || num_bytes % 16 != 0) return -1;
  if (num_bytes == 0) return 0;
  hipLaunchKernelGGL(stream_read_kernel<false>, dim3(256 * 16), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), num_bytes / 16, static_cast<uint32_t*>(sink));
  return finish();
}

int tvmkvb_stream_read_nt(const void* src, int64_t num_bytes, void* sink, void* stream) {
  if (!src || !sink || num_bytes < 0 || num_bytes % 16 != 0) return -1;
  if (num_bytes == 0) return 0;
  hipLaunchKernelGGL(stream_read_kernel<true>, dim3(256 * 16), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), num_bytes / 16, static_cast<uint32_t*>(sink));
  return finish();
}

int tvmkvb_stream_copy(const void* src, void* dst, int64_t num_bytes, void* stream) {
  if (!src || !dst || num_bytes < 0 || num_bytes % 16 != 0) return -1;
  if (num_bytes == 0) return 0;
  hipLaunchKernelGGL(stream_copy_kernel, dim3(256 * 16), dim3(256), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(src), static_cast<uint4*>(dst), num_bytes / 16);
  return finish();
}

int tvmkvb_mfma_loop(const void* operands, float* out, int32_t iters, int32_t workgroups, void* stream) {
  if (!operands || !out || iters < 0 || workgroups <= 0) return -1;
  hipLaunchKernelGGL(mfma_loop_kernel, dim3(static_cast<unsigned>(workgroups)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), static_cast<const _Float16*>(operands), out, iters);
  return finish();
}

}  // extern "C"
