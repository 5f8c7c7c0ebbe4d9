// Shared device-side helpers for the gfx950 kernels: vector types, fp8 / bf16
// conversions built on the CDNA4 conversion instructions, wave reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/mi355q.h"

namespace mi355q {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

constexpr float kFp8Max[2] = {448.0f, 57344.0f};  // e4m3fn, e5m2

// Dynamic per-row quantisation computes scale = target / amax.  A row of zeros
// (amax 0) or of values so small that the quotient overflows would give an
// infinite scale, and 0 * inf = NaN would turn every zero of the row into an
// fp8 NaN.  The scale is therefore capped at the largest finite bf16 value
// (0x7f7f0000; finite in fp32 and after the rounding to bf16 that a bf16 input
// applies to it): a zero row then gives zero codes and a finite 1 / scale.  A
// NaN amax (a NaN in the row) compares false and stays NaN.
constexpr float kRowScaleCap = 3.3895313892515355e38f;
__device__ __forceinline__ float row_scale(float target, float amax) {
  const float s = target / amax;  // correctly rounded fp32 division, as on the host
  return s > kRowScaleCap ? kRowScaleCap : s;
}

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 round-to-nearest-even (v_cvt_pk_bf16_f32), returned as fp32.
__device__ __forceinline__ float round_to_bf16(float v) {
  __bf16 h = (__bf16)v;
  return (float)h;
}

// two fp32 -> packed bf16 pair (lo = a, hi = b)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  bf16x2 r = {(__bf16)a, (__bf16)b};
  return __builtin_bit_cast(uint32_t, r);
}

// exp(t) for -87 <= t <= 88 as a fixed sequence of IEEE operations (Cody-Waite
// reduction by ln 2 in two parts, the degree-5 polynomial of Cephes' expf, an
// exact scaling by a power of two): the CPU oracle runs the same sequence and
// gets the same bits, which a library or hardware exp would not guarantee.
// Contraction is off so that no multiply and add merge that the oracle keeps apart.
__device__ __forceinline__ float exp_spelled_out(float t) {
#pragma clang fp contract(off)
  const float n = __builtin_rintf(t * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693145751953125f, t);
  r = __builtin_fmaf(n, -1.42860682030941723212e-6f, r);
  float q = 1.9875691500e-4f;
  q = __builtin_fmaf(q, r, 1.3981999507e-3f);
  q = __builtin_fmaf(q, r, 8.3334519073e-3f);
  q = __builtin_fmaf(q, r, 4.1665795894e-2f);
  q = __builtin_fmaf(q, r, 1.6666665459e-1f);
  q = __builtin_fmaf(q, r, 5.0000001201e-1f);
  float y = __builtin_fmaf(q, r * r, r);
  y = y + 1.0f;
  return __builtin_ldexpf(y, (int)n);
}

// x / (1 + exp(-x)) in fp32, branch-free; results smaller than 3.3e-37 in
// magnitude (x <= -88.5) are -0, NaN stays NaN.
__device__ __forceinline__ float silu_f32(float x) {
#pragma clang fp contract(off)
  const float t = -x;
  // fmin / fmax return the other operand for a NaN, so the exp below never sees one
  float e = exp_spelled_out(__builtin_fminf(__builtin_fmaxf(t, -87.0f), 88.0f));
  e = t > 88.0f ? __builtin_inff() : e;
  e = t < -87.0f ? 0.0f : e;
  return x / (1.0f + e);
}

// Clamp to the finite fp8 range.  minimum/maximum propagate NaN, so a NaN
// input still converts to an fp8 NaN; +-Inf saturates like any overflow.
template <int FMT>
__device__ __forceinline__ float sat_fp8(float v) {
  constexpr float mx = (FMT == MI355Q_E5M2) ? 57344.0f : 448.0f;
  return __builtin_elementwise_minimum(__builtin_elementwise_maximum(v, -mx), mx);
}

// four fp32 -> four fp8 bytes (element 0 in the low byte), RNE, saturating.
// The raw v_cvt_pk_{fp8,bf8}_f32 turns overflow into NaN/Inf, hence the clamp.
template <int FMT>
__device__ __forceinline__ uint32_t cvt_fp8x4(float a, float b, float c, float d) {
  a = sat_fp8<FMT>(a);
  b = sat_fp8<FMT>(b);
  c = sat_fp8<FMT>(c);
  d = sat_fp8<FMT>(d);
  int r;
  if constexpr (FMT == MI355Q_E5M2) {
    r = __builtin_amdgcn_cvt_pk_bf8_f32(a, b, 0, false);
    r = __builtin_amdgcn_cvt_pk_bf8_f32(c, d, r, true);
  } else {
    r = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    r = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, r, true);
  }
  return (uint32_t)r;
}

// Stochastic rounding of four fp32 to fp8 (v_cvt_sr_fp8_f32 / v_cvt_sr_bf8_f32:
// the 32 random bits are added below the kept mantissa before truncation), after
// the same saturating clamp as the round-to-nearest path.
template <int FMT>
__device__ __forceinline__ uint32_t cvt_fp8x4_sr(float a, float b, float c, float d, uint32_t r0,
                                                 uint32_t r1, uint32_t r2, uint32_t r3) {
  a = sat_fp8<FMT>(a);
  b = sat_fp8<FMT>(b);
  c = sat_fp8<FMT>(c);
  d = sat_fp8<FMT>(d);
  int r = 0;
  if constexpr (FMT == MI355Q_E5M2) {
    r = __builtin_amdgcn_cvt_sr_bf8_f32(a, r0, r, 0);
    r = __builtin_amdgcn_cvt_sr_bf8_f32(b, r1, r, 1);
    r = __builtin_amdgcn_cvt_sr_bf8_f32(c, r2, r, 2);
    r = __builtin_amdgcn_cvt_sr_bf8_f32(d, r3, r, 3);
  } else {
    r = __builtin_amdgcn_cvt_sr_fp8_f32(a, r0, r, 0);
    r = __builtin_amdgcn_cvt_sr_fp8_f32(b, r1, r, 1);
    r = __builtin_amdgcn_cvt_sr_fp8_f32(c, r2, r, 2);
    r = __builtin_amdgcn_cvt_sr_fp8_f32(d, r3, r, 3);
  }
  return (uint32_t)r;
}

// 64 random bits for counter `idx` of stream `seed` (the splitmix64 finaliser:
// stateless, so an element's bits depend only on its index and the seed).
__device__ __forceinline__ uint64_t counter_random64(uint64_t seed, uint64_t idx) {
  uint64_t z = seed + (idx + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// four fp8 bytes of one dword -> four fp32 (exact)
template <int FMT>
__device__ __forceinline__ void cvt_f32x4(uint32_t w, float& a, float& b, float& c, float& d) {
  f32x2 lo, hi;
  if constexpr (FMT == MI355Q_E5M2) {
    lo = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, false);
    hi = __builtin_amdgcn_cvt_pk_f32_bf8((int)w, true);
  } else {
    lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
    hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
  }
  a = lo.x; b = lo.y; c = hi.x; d = hi.y;
}

template <int FMT>
__device__ __forceinline__ float cvt_f32x1(uint32_t byte) {
  if constexpr (FMT == MI355Q_E5M2) return __builtin_amdgcn_cvt_f32_bf8((int)byte, 0);
  else return __builtin_amdgcn_cvt_f32_fp8((int)byte, 0);
}

// max over the 64 lanes of a wave of a non-negative-float bit pattern
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) {
    uint32_t o = (uint32_t)__shfl_xor((int)v, off, 64);
    v = v > o ? v : o;
  }
  return v;
}

}  // namespace mi355q
