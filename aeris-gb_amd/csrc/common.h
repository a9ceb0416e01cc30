// Shared device helpers for the gfx950 kernels of libaeris_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace aeris {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

// bf16 <-> f32 on raw bits (round to nearest even; NaN kept quiet)
__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }
__device__ __forceinline__ float bf16_lo(uint32_t packed) { return __uint_as_float(packed << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t packed) { return __uint_as_float(packed & 0xffff0000u); }

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;

// round-to-nearest-even conversions; on gfx950 a pair is one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, 0.f) & 0xffffu; }

// 64-lane wavefront reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float silu_f(float x) { return x * __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }
__device__ __forceinline__ float erf_poly(float x) {
  // Abramowitz-Stegun 7.1.26, abs error <= 1.5e-7 (below bf16 and fp32-accumulation noise)
  const float ax = fabsf(x);
  const float t = __frcp_rn(fmaf(0.3275911f, ax, 1.0f));
  float pol = fmaf(1.061405429f, t, -1.453152027f);
  pol = fmaf(pol, t, 1.421413741f);
  pol = fmaf(pol, t, -0.284496736f);
  pol = fmaf(pol, t, 0.254829592f);
  const float r = 1.0f - pol * t * __expf(-ax * ax);
  return copysignf(r, x);
}
__device__ __forceinline__ float gelu_erf_f(float x) { return 0.5f * x * (1.0f + erf_poly(x * 0.70710678118654752440f)); }

// erf-GELU for results that are rounded to bf16: erf(u) = t * P(t^2), t = clamp(u, -3, 3), P a degree-8 minimax
// polynomial (|error| <= 3.1e-5 in erf, <= 1.6e-5 relative in GELU: 1/100 of a bf16 ulp).  14 VALU operations and no
// transcendental, against about 24 op-equivalents for the 1.5e-7 version above; the GEMM epilogue is VALU-bound.
__device__ __forceinline__ float gelu_bf16_f(float x) {
  const float u = x * 0.70710678118654752440f;
  const float t = __builtin_amdgcn_fmed3f(u, -3.0f, 3.0f);
  const float s = t * t;
  float p = fmaf(4.074150084e-08f, s, -1.944801170e-06f);
  p = fmaf(p, s, 4.106021152e-05f);
  p = fmaf(p, s, -5.110344500e-04f);
  p = fmaf(p, s, 4.235417116e-03f);
  p = fmaf(p, s, -2.510283515e-02f);
  p = fmaf(p, s, 1.110793054e-01f);
  p = fmaf(p, s, -3.753148615e-01f);
  p = fmaf(p, s, 1.128268480e+00f);
  const float hx = 0.5f * x;
  return fmaf(hx, t * p, hx);
}

}  // namespace aeris
