// Row norm (LayerNorm / RMSNorm) fused with the noise-level scale/shift modulation.  HBM-bound:
// every row of x is read once and every row of y written once, 16 bytes per lane per access, both
// marked non-temporal (streamed once: 4 % faster than with the default cache policy; either one alone is not).
//
// One wavefront owns one row at a time and keeps it in registers (NV vectors of 8 elements per
// lane); the next row's loads are issued before the current row is reduced, so each wave has two
// rows in flight.  Statistics are fp32: mean, then the centred second moment (LayerNorm), or the
// plain second moment (RMSNorm).  The per-column parameters are folded once per wave into
//     pre :  u = x * P1 + P0          (P1 = 1 + scale, P0 = shift;  only for "modulate then norm")
//     post:  y = n(u) * G + Bc        (G = gamma, Bc = beta, or for "norm then modulate"
//                                      G = gamma*(1+scale), Bc = beta*(1+scale) + shift)
// and stay in registers while the wave walks down its rows (re-folded when the batch index, and
// with it the modulation row, changes).
#include "common.h"
#include "kernels.h"

namespace aeris {

struct NormParams {
  const void* x;
  void* y;
  const void* gamma;
  const void* beta;
  int param_f32;
  const float* shift;
  const float* scale;
  int64_t mod_batch_stride;
  int64_t rows;
  int64_t rows_per_batch;
  int d;
  int kind;
  int y_dtype;
  float eps;
};

// FULL: d == NV * 512, every lane holds NV full 16-byte pieces of the row (no per-piece predicates in the loop)
template <int NV, bool X_F32, bool PRE, bool FULL>
__global__ void __launch_bounds__(256) norm_modulate_kernel(NormParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t wave_id = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t n_waves = (int64_t)gridDim.x * 4;
  const int d = p.d;
  const float inv_d = 1.0f / (float)d;

  bool act[NV];
  int col[NV];
#pragma unroll
  for (int v = 0; v < NV; ++v) {
    col[v] = (v * 64 + lane) * 8;
    act[v] = FULL || col[v] < d;
  }

  float G[NV][8], Bc[NV][8], P1[PRE ? NV : 1][8], P0[PRE ? NV : 1][8];
  auto fold = [&](int64_t b) {
    const float* sh = p.shift ? p.shift + b * p.mod_batch_stride : nullptr;
    const float* sc = p.scale ? p.scale + b * p.mod_batch_stride : nullptr;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float g = 1.f, be = 0.f, s1 = 1.f, s0 = 0.f;
        if (act[v]) {
          const int c = col[v] + e;
          if (p.param_f32) {
            g = reinterpret_cast<const float*>(p.gamma)[c];
            if (p.beta) be = reinterpret_cast<const float*>(p.beta)[c];
          } else {
            g = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.gamma)[c]);
            if (p.beta) be = bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p.beta)[c]);
          }
          if (sc) s1 = 1.f + sc[c];
          if (sh) s0 = sh[c];
        }
        if (PRE) {
          P1[v][e] = s1; P0[v][e] = s0; G[v][e] = g; Bc[v][e] = be;
        } else {
          G[v][e] = g * s1; Bc[v][e] = be * s1 + s0;
        }
      }
    }
  };

  struct Raw { u32x4 a, b; };
  auto load_row = [&](int64_t row, Raw (&raw)[NV]) {
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      raw[v].a = u32x4{0u, 0u, 0u, 0u};
      raw[v].b = u32x4{0u, 0u, 0u, 0u};
      if (act[v]) {
        if (X_F32) {
          const float* xp = reinterpret_cast<const float*>(p.x) + row * d + col[v];
          raw[v].a = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xp));
          raw[v].b = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xp + 4));
        } else {
          raw[v].a = __builtin_nontemporal_load(
              reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(p.x) + row * d + col[v]));
        }
      }
    }
  };

  int64_t row = wave_id;
  if (row >= p.rows) return;
  int64_t cur_b = row / p.rows_per_batch;
  fold(p.mod_batch_stride ? cur_b : 0);

  Raw cur[NV], nxt[NV];
  load_row(row, cur);
  for (; row < p.rows; row += n_waves) {
    const int64_t next = row + n_waves;
    if (next < p.rows) load_row(next, nxt);

    if (p.mod_batch_stride) {
      const int64_t b = row / p.rows_per_batch;
      if (b != cur_b) { cur_b = b; fold(b); }
    }

    float u[NV][8];
    float s = 0.f;
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      if (X_F32) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          u[v][e] = __uint_as_float(cur[v].a[e]);
          u[v][4 + e] = __uint_as_float(cur[v].b[e]);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          u[v][2 * e] = bf16_lo(cur[v].a[e]);
          u[v][2 * e + 1] = bf16_hi(cur[v].a[e]);
        }
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if (PRE) u[v][e] = act[v] ? fmaf(u[v][e], P1[v][e], P0[v][e]) : 0.f;
        s += (p.kind == AERIS_NORM_RMS) ? u[v][e] * u[v][e] : u[v][e];
      }
    }
    s = wave_sum(s);
    float mean = 0.f, rstd;
    if (p.kind == AERIS_NORM_RMS) {
      rstd = rsqrtf(s * inv_d + p.eps);
    } else {
      mean = s * inv_d;
      float q = 0.f;
#pragma unroll
      for (int v = 0; v < NV; ++v)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float c = act[v] ? u[v][e] - mean : 0.f;
          q += c * c;
        }
      q = wave_sum(q);
      rstd = rsqrtf(q * inv_d + p.eps);
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) {
      if (!act[v]) continue;
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = fmaf((u[v][e] - mean) * rstd, G[v][e], Bc[v][e]);
      if (p.y_dtype == AERIS_BF16) {
        u32x4 w = {pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7])};
        __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(reinterpret_cast<uint16_t*>(p.y) + row * d + col[v]));
      } else {
        float* yp = reinterpret_cast<float*>(p.y) + row * d + col[v];
        __builtin_nontemporal_store(f32x4{o[0], o[1], o[2], o[3]}, reinterpret_cast<f32x4*>(yp));
        __builtin_nontemporal_store(f32x4{o[4], o[5], o[6], o[7]}, reinterpret_cast<f32x4*>(yp + 4));
      }
    }
#pragma unroll
    for (int v = 0; v < NV; ++v) cur[v] = nxt[v];
  }
}

bool norm_supported(int d) { return d > 0 && d % 8 == 0 && d <= 12 * 512; }

template <int NV>
static hipError_t launch_norm(const NormParams& p, bool x_f32, bool pre, hipStream_t stream) {
  // enough waves to cover HBM latency, few enough that parameter folding is amortised over many rows
  int64_t blocks = (p.rows + 3) / 4;
  const int64_t cap = 256 * 8;
  if (blocks > cap) blocks = cap;
  dim3 grid((unsigned)blocks), block(256);
#define AERIS_NORM_GO(XF, PR)                                                                                   \
  do {                                                                                                          \
    if (p.d == NV * 512) hipLaunchKernelGGL((norm_modulate_kernel<NV, XF, PR, true>), grid, block, 0, stream, p);  \
    else hipLaunchKernelGGL((norm_modulate_kernel<NV, XF, PR, false>), grid, block, 0, stream, p);                 \
  } while (0)
  if (x_f32) {
    if (pre) AERIS_NORM_GO(true, true);
    else AERIS_NORM_GO(true, false);
  } else {
    if (pre) AERIS_NORM_GO(false, true);
    else AERIS_NORM_GO(false, false);
  }
#undef AERIS_NORM_GO
  return hipGetLastError();
}

hipError_t norm_modulate_launch(const void* x, int x_dtype, void* y, int y_dtype, const void* gamma, const void* beta,
                                int param_dtype, const float* shift, const float* scale, int64_t mod_batch_stride, int64_t B,
                                int64_t rows_per_batch, int d, int kind, int order, float eps, hipStream_t stream) {
  NormParams p;
  p.x = x; p.y = y;
  p.gamma = gamma;
  p.beta = beta;
  p.param_f32 = param_dtype == AERIS_F32;
  p.shift = shift; p.scale = scale;
  p.mod_batch_stride = (shift || scale) ? mod_batch_stride : 0;
  p.rows = B * rows_per_batch;
  p.rows_per_batch = rows_per_batch;
  p.d = d; p.kind = kind; p.y_dtype = y_dtype; p.eps = eps;
  const bool pre = (order == AERIS_MOD_THEN_NORM) && (shift || scale);
  const bool xf = x_dtype == AERIS_F32;
  const int nv = (d + 511) / 512;
  switch (nv) {
    case 1: return launch_norm<1>(p, xf, pre, stream);
    case 2: return launch_norm<2>(p, xf, pre, stream);
    case 3: return launch_norm<3>(p, xf, pre, stream);
    case 4: return launch_norm<4>(p, xf, pre, stream);
    case 5: case 6: return launch_norm<6>(p, xf, pre, stream);
    case 7: case 8: return launch_norm<8>(p, xf, pre, stream);
    default: return launch_norm<12>(p, xf, pre, stream);
  }
}

}  // namespace aeris
