// Shared device helpers for the gfx950 quantization kernels.
//
// Wave size is 64 on CDNA4; every reduction below is written for that.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LCQ_WAVE 64

typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// ---------------------------------------------------------------------------
// bit casts / bf16
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }

// fp32 -> bf16 (round to nearest even) -> fp32, integer form. NaN stays NaN.
__device__ __forceinline__ float bf16_round(float f) {
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return u2f(u | 0x00400000u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return u2f(u & 0xffff0000u);
}
__device__ __forceinline__ uint32_t bf16_bits(float f) {   // upper 16 bits after RNE
  uint32_t u = f2u(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}
__device__ __forceinline__ float bf16_lo(uint32_t w) { return u2f(w << 16); }          // element 0 of a packed pair
__device__ __forceinline__ float bf16_hi(uint32_t w) { return u2f(w & 0xffff0000u); }  // element 1
__device__ __forceinline__ uint32_t bf16_pack(float a, float b) {                      // a,b already bf16-exact
  return (f2u(a) >> 16) | (f2u(b) & 0xffff0000u);
}

// fp32 -> fp16 (RNE) -> fp32
__device__ __forceinline__ float f16_round(float f) { return (float)(_Float16)f; }

// NaN-propagating min / max (torch.amax / clamp semantics)
// (IEEE 754-2019 maximum / minimum: v_maximum3_f32 / v_minimum3_f32 on gfx950, one instruction, no branches)
__device__ __forceinline__ float nan_max(float a, float b) { return __builtin_elementwise_maximum(a, b); }
__device__ __forceinline__ float nan_min(float a, float b) { return __builtin_elementwise_minimum(a, b); }

// ---------------------------------------------------------------------------
// cross-lane: xor butterfly built from DPP (inside a row of 16 lanes),
// ds_swizzle (xor 16, inside 32 lanes) and ds_bpermute (xor 32).
// ---------------------------------------------------------------------------
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return u2f((uint32_t)__builtin_amdgcn_update_dpp(0, (int)f2u(v), CTRL, 0xf, 0xf, true));
}
// value held by lane (id ^ MASK); MASK a power of two below 64.
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
  if constexpr (MASK == 1) return dpp_f<0xB1>(v);        // quad_perm [1,0,3,2]
  else if constexpr (MASK == 2) return dpp_f<0x4E>(v);   // quad_perm [2,3,0,1]
  else if constexpr (MASK == 4) return dpp_f<0x141>(v);  // row_half_mirror: i <-> 7-i  (quads already uniform)
  else if constexpr (MASK == 8) return dpp_f<0x140>(v);  // row_mirror: i <-> 15-i      (octets already uniform)
  else if constexpr (MASK == 16) return u2f((uint32_t)__builtin_amdgcn_ds_swizzle((int)f2u(v), 0x401F));  // bit mode, xor 0x10
  else return u2f((uint32_t)__builtin_amdgcn_ds_bpermute((int)((threadIdx.x ^ 32) << 2), (int)f2u(v)));
}
// NOTE: the MASK==4 / MASK==8 forms are mirrors, not xors; they equal the xor
// butterfly only when applied in increasing MASK order inside a reduction.

template <int TEAM, bool IS_MAX>
__device__ __forceinline__ float team_reduce(float v) {
  // all-reduce over aligned groups of TEAM consecutive lanes (TEAM = 1,2,4,...,64)
  #define LCQ_STEP(M) if constexpr (TEAM > M) { float o = lane_xor<M>(v); v = IS_MAX ? nan_max(v, o) : nan_min(v, o); }
  LCQ_STEP(1) LCQ_STEP(2) LCQ_STEP(4) LCQ_STEP(8) LCQ_STEP(16) LCQ_STEP(32)
  #undef LCQ_STEP
  return v;
}
template <int TEAM>
__device__ __forceinline__ float team_sum(float v) {
  #define LCQ_STEP(M) if constexpr (TEAM > M) { v += lane_xor<M>(v); }
  LCQ_STEP(1) LCQ_STEP(2) LCQ_STEP(4) LCQ_STEP(8) LCQ_STEP(16) LCQ_STEP(32)
  #undef LCQ_STEP
  return v;
}

// ---------------------------------------------------------------------------
// launch check (error codes live in include/lcq.h)
// ---------------------------------------------------------------------------






#define LCQ_CHECK_LAUNCH() do { hipError_t e_ = hipGetLastError(); if (e_ != hipSuccess) return LCQ_ELAUNCH; } while (0)
