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

// Reductions over the lane pairs (l, l ^ 32) and (l, l ^ 16) with the gfx950 lane-swap
// instructions (vector ALU; a __shfl_xor goes through LDS and its latency).  With both operands
// equal to x, v_permlane32_swap leaves x[l & 31] in one result and x[(l & 31) + 32] in the other
// in every lane, and v_permlane16_swap likewise for the 16-lane rows (0, 1) and (2, 3).
__device__ __forceinline__ float max_xor32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_xor32(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
__device__ __forceinline__ float max_xor16(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_xor16(float x) {
  const auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ---- asynchronous global -> LDS copies, transposing LDS reads (gfx950) -----------------------
typedef __attribute__((address_space(3))) void* lds_ptr_t;

// One global_load_lds_dwordx4: lane L copies the 16 bytes at its own global address to LDS address
// lds_addr + 16*L (lds_addr must be the same in every lane).  The copy is asynchronous and counted
// by vmcnt.  It is issued from inline assembly on purpose: when the compiler knows of a copy in
// flight it puts s_waitcnt vmcnt(0) in front of the next LDS read it cannot tell apart from the
// copy's destination, which would serialise the two-stage pipeline; here the one wait per tile is
// written by hand in front of the workgroup barrier.  The compiler sets M0 itself right before
// each of its own uses, so the asm does not have to restore it.
// src_base (the same in every lane) + byte_off (per lane, unsigned 32 bit) is the global address.
__device__ __forceinline__ void copy16_to_lds(const void* src_base, uint32_t byte_off, uint32_t lds_addr) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               ::"v"(byte_off), "s"(src_base), "s"(lds_addr) : "memory");
}

// The same copy and a 16-byte load with the non-temporal hint, for data that is read exactly once
// (the K/V pages of a decode step): it is streamed through the caches instead of displacing what
// other workgroups reuse, which measured 4 % more bandwidth on the decode kernel.
__device__ __forceinline__ void copy16_to_lds_nt(const void* src_base, uint32_t byte_off, uint32_t lds_addr) {
  lds_addr = __builtin_amdgcn_readfirstlane(lds_addr);
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
               ::"v"(byte_off), "s"(src_base), "s"(lds_addr) : "memory");
}
__device__ __forceinline__ Vec16 ld16_nt(const void* p) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  const u32x4 r = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  Vec16 v;
  v.w[0] = r[0];
  v.w[1] = r[1];
  v.w[2] = r[2];
  v.w[3] = r[3];
  return v;
}

// Tells the compiler that a pointer holds the same value in every lane.
__device__ __forceinline__ const half_t* uniform_ptr(const half_t* p) {
  const uint64_t v = reinterpret_cast<uint64_t>(p);
  const uint32_t lo = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v));
  const uint32_t hi = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(v >> 32));
  return reinterpret_cast<const half_t*>((static_cast<uint64_t>(hi) << 32) | lo);
}
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4_t* lds_short4_ptr_t;

// ds_read_b64_tr_b16: within each group of 16 lanes, lane l receives element l%4 of the four
// 8-byte rows addressed by lanes l/4, 4 + l/4, 8 + l/4 and 12 + l/4 of the group.
__device__ __forceinline__ half4_t lds_read_tr16(const half_t* p) {
  return __builtin_bit_cast(half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr_t)p));
}

// The same reads from an LDS byte address held in a register (plus what the compiler folds into
// the instruction's immediate offset).
typedef __attribute__((address_space(3))) const half8_t* lds_half8_cptr_t;
__device__ __forceinline__ half8_t lds_read_b128_at(uint32_t addr) {
  return *reinterpret_cast<lds_half8_cptr_t>(static_cast<uintptr_t>(addr));
}
__device__ __forceinline__ half4_t lds_read_tr16_at(uint32_t addr) {
  return __builtin_bit_cast(half4_t, __builtin_amdgcn_ds_read_tr16_b64_v4i16(
                                         reinterpret_cast<lds_short4_ptr_t>(static_cast<uintptr_t>(addr))));
}

// s_waitcnt vmcnt(N) alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14, the other counters at their maximum)
template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// Scheduling hint for the region it is placed in: N groups of (1 MFMA, then a few vector ALU ops).
template <int N>
__device__ __forceinline__ void interleave_mfma_valu() {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
    __builtin_amdgcn_sched_group_barrier(0x002, 8, 0);  // VALU
  }
}

// ---- inline RoPE (kernels that rotate q and k themselves) --------------------------------------
// sin and cos of an fp32 angle of any size: two-constant Cody-Waite reduction to [-pi, pi], then
// the hardware functions (which take revolutions).  Absolute error ~1e-6 for |x| up to ~1e5.
__device__ __forceinline__ void sincos_reduced(float x, float& sn, float& cs) {
  const float k = rintf(x * 0.15915494309189535f);
  float r = fmaf(-k, 6.2831854820251465f, x);    // fp32(2 pi)
  r = fmaf(-k, -1.7484555314695172e-7f, r);      // 2 pi - fp32(2 pi)
  const float t = r * 0.15915494309189535f;
  sn = __builtin_amdgcn_sinf(t);
  cs = __builtin_amdgcn_cosf(t);
}

// Rotate-half RoPE of the features (f, f + D/2) held by one lane in two fragments, as the reference
// does it (python/tvm/relax/frontend/nn/llm/_kernel_common.py:115-127): fp32 math, one rounding to fp16.
__device__ __forceinline__ void rope_pair(half8_t& lo, half8_t& hi, float pos_scaled, const float* div8) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float sn, cs;
    sincos_reduced(pos_scaled / div8[i], sn, cs);
    const float xl = static_cast<float>(lo[i]);
    const float xh = static_cast<float>(hi[i]);
    lo[i] = static_cast<half_t>(cs * xl + sn * (-xh));
    hi[i] = static_cast<half_t>(cs * xh + sn * xl);
  }
}

// The table an attention kernel rotates q and k with (in-kernel RoPE, rotate-half pairing over the whole
// head, python/tvm/relax/frontend/nn/llm/_kernel_common.py:115-127).  v[d], d < D: the divisor of element
// d's angle (angle = position / v[d]) or, with `inverse`, its inverse frequency (angle = position * v[d]);
// element d and its partner d + D/2 share an angle unless `halves_differ`; cos and sin are multiplied by
// `magnitude`.  Built on the host in float32 in the reference's order of operations (inline_rope_table).
constexpr int kMaxHeadDim = 256;
struct InlineRopeTable {
  float v[kMaxHeadDim];
  int inverse;
  int halves_differ;
  float magnitude;
};

// rope_pair for any frequency variant: table entries of the 8 elements of `lo` and of `hi`.
__device__ __forceinline__ void rope_pair_ex(half8_t& lo, half8_t& hi, float pos_scaled, const float* tbl_lo8,
                                             const float* tbl_hi8, int inverse, int halves_differ, float magnitude) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    float sn, cs;
    sincos_reduced(inverse ? pos_scaled * tbl_lo8[i] : pos_scaled / tbl_lo8[i], sn, cs);
    sn *= magnitude;
    cs *= magnitude;
    float sn_hi = sn, cs_hi = cs;
    if (halves_differ) {
      sincos_reduced(inverse ? pos_scaled * tbl_hi8[i] : pos_scaled / tbl_hi8[i], sn_hi, cs_hi);
      sn_hi *= magnitude;
      cs_hi *= magnitude;
    }
    const float xl = static_cast<float>(lo[i]);
    const float xh = static_cast<float>(hi[i]);
    lo[i] = static_cast<half_t>(cs * xl + sn * (-xh));
    hi[i] = static_cast<half_t>(cs_hi * xh + sn_hi * xl);
  }
}

// Compute units of the current device (cached per device).
inline int compute_units() {
  static int cached[64] = {0};
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  if (dev < 0 || dev >= 64) return 256;
  if (cached[dev] == 0) {
    int n = 0;
    HIP_CHECK(hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev));
    cached[dev] = n > 0 ? n : 256;
  }
  return cached[dev];
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
