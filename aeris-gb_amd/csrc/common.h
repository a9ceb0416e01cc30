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
// acc + lo + hi of a packed bf16 pair, in fp32 (v_dot2c_f32_bf16 with a pair of ones)
__device__ __forceinline__ float dot2_ones(uint32_t packed, float acc) {
  const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, packed), ones, acc, false);
}

// 64-lane wavefront sum, the same value in every lane.  Data-parallel-primitive adds inside the 16-lane rows (quad
// permutes, half mirror, mirror), two row broadcasts across the rows, total read from lane 63: six VALU operations
// instead of six round trips through the LDS crossbar (ds_bpermute), which a row-per-wave kernel feels twice per row.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_add(float v) {  // v + v[lane selected by CTRL]; rows outside ROW_MASK add 0
  return v + __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, true));
}
__device__ __forceinline__ float wave_sum(float v) {
  v = dpp_add<0xB1, 0xF>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E, 0xF>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141, 0xF>(v);  // row_half_mirror
  v = dpp_add<0x140, 0xF>(v);  // row_mirror: every lane holds the sum of its row
  v = dpp_add<0x142, 0xA>(v);  // row_bcast15: rows 1 and 3 add the row before them
  v = dpp_add<0x143, 0xC>(v);  // row_bcast31: rows 2 and 3 add rows 0 + 1
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// ---- buffer_load_dwordx4 ... lds (16 bytes per lane from global memory straight into LDS, lane l at LDS byte
// m0 + 16 l) as inline assembly.  The compiler's builtin form makes every later LDS access a possible alias of the load
// in the compiler's eyes: it then guards LDS reads with s_waitcnt vmcnt(0) wherever it cannot count the operations in
// between, e.g. inside a loop that is entered with stores still in flight.  Issued from assembly the load is invisible
// to that bookkeeping; what orders it against the LDS reads is the kernels' own counted s_waitcnt + barrier, as
// before.  (Vector memory operations complete in order, so operations the compiler does not know of only make its own
// counted waits stricter.)  The descriptor is built by hand: base, stride 0, size in bytes, raw 32-bit format.
typedef u32x4 lds_dma_rsrc;
__device__ __forceinline__ lds_dma_rsrc make_lds_dma_rsrc(const void* base, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(base);
  lds_dma_rsrc r;
  r.x = __builtin_amdgcn_readfirstlane((uint32_t)a);
  r.y = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32) & 0xffffu);
  r.z = __builtin_amdgcn_readfirstlane(bytes);
  r.w = 0x00020000u;
  return r;
}
// lds_address, soffset: wave-uniform; voffset: per lane; out-of-range lanes (voffset >= size) arrive as zeros
__device__ __forceinline__ void lds_dma_load16(const lds_dma_rsrc& rsrc, uint32_t lds_address, uint32_t voffset, uint32_t soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(lds_address), "v"(voffset), "s"(rsrc), "s"(soffset)
               : "memory");
}

// ---- ds_read_b64_tr_b16 (the LDS read that transposes 4 x 4 blocks of 16-bit elements on the way out) as inline assembly.
// The compiler's builtin form may not be used while a buffer_load ... lds is in flight: the compiler cannot tell that
// the read does not alias the load's destination and puts an s_waitcnt vmcnt(0) in front of it, which makes a wave
// wait for the next unit's (or chunk's) loads in the middle of the arithmetic that they are meant to run under.
// The assembly form is invisible to that analysis - and to the compiler's count of outstanding LDS operations: the
// result registers must pass through lds_tr_wait() (s_waitcnt lgkmcnt(0)) before anything reads them.  ("memory"
// keeps the compiler from moving LDS accesses of its own across the read; its own lgkmcnt waits stay correct, LDS
// operations return in order and extra outstanding ones only make a counted wait stricter.)
// Nor does the compiler keep such a read away from registers that a running MFMA is still writing (see the sweep in
// attention_sweep.h).  Both rules are checked on the emitted assembly by every build (asm_check.py, run by build.py).
__device__ __forceinline__ uint32_t lds_byte_address(const void* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}
template <int OFFSET>
__device__ __forceinline__ u32x2 lds_read_tr16_b64(uint32_t lds_address) {
  u32x2 r;
  asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(r) : "v"(lds_address), "n"(OFFSET) : "memory");
  return r;
}
struct TrFrag { u32x2 lo, hi; };  // two transposing reads = the 8 k slots of one MFMA operand
__device__ __forceinline__ void lds_tr_wait(TrFrag& a, TrFrag& b) {
  asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi));
}
__device__ __forceinline__ void lds_tr_wait(TrFrag& a, TrFrag& b, TrFrag& c, TrFrag& d) {
  asm volatile("s_waitcnt lgkmcnt(0)"
               : "+v"(a.lo), "+v"(a.hi), "+v"(b.lo), "+v"(b.hi), "+v"(c.lo), "+v"(c.hi), "+v"(d.lo), "+v"(d.hi));
}
__device__ __forceinline__ bf16x8 tr_frag_value(const TrFrag& f) {
  return __builtin_bit_cast(bf16x8, u32x4{f.lo.x, f.lo.y, f.hi.x, f.hi.y});
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

// erf-GELU for results that are rounded to bf16: GELU(x) = xm * (0.5 + t * P(t^2)), xm = max(x, -3.5), t = min(xm, 3.5),
// t * P(t^2) = erf(t / sqrt2) / 2 with P a degree-6 minimax polynomial for the error measure |GELU error| / |x| (the
// 1/sqrt2 and the 1/2 are folded into its coefficients): |error| <= 2.0e-4 |x| for x >= -3.5, a tenth of half a bf16 ulp,
// the clamp included (1 - Phi(3.5) = 2.3e-4); below -3.5 the result is the constant -3.5 * 2.3e-4 = -8.1e-4 where the
// exact value decays from -8.1e-4 to 0, so large negative pre-activations cannot leak a term proportional to x.
// On normally distributed inputs 2 % of the bf16 results differ by one ulp from the exactly evaluated and
// once-rounded GELU (0.7 % for a 1.5e-7 evaluation: rounding an fp32 result to bf16 twice), the relative L2 error
// after rounding is the same to four digits.  11 VALU operations and no transcendental, against about 24
// op-equivalents for the 1.5e-7 version above and 12 for a degree-8 polynomial over +-3 sqrt2 (1.6e-5 |x|): the GEMM
// epilogue is VALU-bound, every two operations are worth 1.3 % of the fc1 GEMM.
__device__ __forceinline__ float gelu_bf16_f(float x) {
  const float xm = fmaxf(x, -3.5f);
  const float t = fminf(xm, 3.5f);
  const float s = t * t;
  float p = fmaf(5.387934375e-08f, s, -2.947825681e-06f);
  p = fmaf(p, s, 7.079321479e-05f);
  p = fmaf(p, s, -1.003445996e-03f);
  p = fmaf(p, s, 9.561960235e-03f);
  p = fmaf(p, s, -6.607216932e-02f);
  p = fmaf(p, s, 3.988177931e-01f);
  return xm * fmaf(t, p, 0.5f);
}

}  // namespace aeris
