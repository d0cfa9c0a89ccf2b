// Device-side helpers shared by the gfx950 kernels: 16-byte vector access, fp16 packing,
// DPP reductions inside a wavefront row, and the launcher argument checks.
#ifndef TVMKV_CSRC_KERNELS_COMMON_CUH_
#define TVMKV_CSRC_KERNELS_COMMON_CUH_

#include <hip/hip_runtime.h>

#include <cstdint>

#include "common.h"

namespace tvmkv {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kNegInit = -5e4f;  // online-softmax "minus infinity" of the reference kernels

// 16 bytes = 8 fp16, the unit of every global access in these kernels.
union Vec16 {
  uint4 u;
  half8_t h8;
  half2_t h2[4];
  half_t h[8];
  uint32_t w[4];
};

__device__ __forceinline__ Vec16 ld16(const void* p) {
  Vec16 v;
  v.u = *reinterpret_cast<const uint4*>(p);
  return v;
}
__device__ __forceinline__ void st16(void* p, const Vec16& v) { *reinterpret_cast<uint4*>(p) = v.u; }
__device__ __forceinline__ Vec16 zero16() {
  Vec16 v;
  v.u = make_uint4(0, 0, 0, 0);
  return v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }

// x + (x moved inside the 16-lane row by the DPP control CTRL)
template <int CTRL>
__device__ __forceinline__ float dpp_add(float x) {
  int moved = __builtin_amdgcn_update_dpp(0, __float_as_int(x), CTRL, 0xf, 0xf, true);
  return x + __int_as_float(moved);
}
constexpr int kDppXor1 = 0xB1;         // quad_perm [1,0,3,2]
constexpr int kDppXor2 = 0x4E;         // quad_perm [2,3,0,1]
constexpr int kDppRowHalfMirror = 0x141;
constexpr int kDppRowMirror = 0x140;

// Sum over groups of LANES consecutive lanes (LANES = 4, 8 or 16); every lane gets the total.
template <int LANES>
__device__ __forceinline__ float group_sum(float x) {
  x = dpp_add<kDppXor1>(x);
  x = dpp_add<kDppXor2>(x);
  if (LANES >= 8) x = dpp_add<kDppRowHalfMirror>(x);
  if (LANES >= 16) x = dpp_add<kDppRowMirror>(x);
  return x;
}

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

}  // namespace tvmkv

#define KV_LAUNCH_CHECK()                                                                          \
  do {                                                                                             \
    hipError_t _e = hipGetLastError();                                                             \
    if (_e != hipSuccess) {                                                                        \
      throw ::tvmkv::Error(TVMKV_EDEVICE, std::string("kernel launch failed: ") + hipGetErrorString(_e)); \
    }                                                                                              \
  } while (0)

#endif  // TVMKV_CSRC_KERNELS_COMMON_CUH_
