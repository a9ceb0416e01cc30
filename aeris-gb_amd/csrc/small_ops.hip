// Small per-step operators: modulation MLP layers (GEMV), sinusoidal noise-level embedding and the
// A-operand preparation of the input embedding.  All are launch- or bandwidth-bound.
#include "common.h"
#include "kernels.h"

namespace aeris {

// y[b, n] = act(dot(W[n, :], x[b, :]) + bias[n]).  One wavefront per output row n; the weight row is
// streamed once (16 B per lane per step) and reused for every batch row b (B <= 8 per pass).
template <bool W_F32>
__global__ void __launch_bounds__(256) modulation_linear_kernel(const float* __restrict__ x, const void* __restrict__ Wv,
                                                               const void* __restrict__ biasv, float* __restrict__ y,
                                                               int B, int N, int K, int act) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (n >= N) return;
  for (int b0 = 0; b0 < B; b0 += 8) {
    const int nb = (B - b0) < 8 ? (B - b0) : 8;
    float accv[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) accv[j] = 0.f;
    for (int k = lane * 8; k < K; k += 512) {
      float w[8];
      if (W_F32) {
        const float* wp = reinterpret_cast<const float*>(Wv) + (int64_t)n * K + k;
        const f32x4 w0 = *reinterpret_cast<const f32x4*>(wp);
        const f32x4 w1 = *reinterpret_cast<const f32x4*>(wp + 4);
        w[0] = w0.x; w[1] = w0.y; w[2] = w0.z; w[3] = w0.w; w[4] = w1.x; w[5] = w1.y; w[6] = w1.z; w[7] = w1.w;
      } else {
        const u32x4 r = *reinterpret_cast<const u32x4*>(reinterpret_cast<const uint16_t*>(Wv) + (int64_t)n * K + k);
#pragma unroll
        for (int e = 0; e < 4; ++e) { w[2 * e] = bf16_lo(r[e]); w[2 * e + 1] = bf16_hi(r[e]); }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        if (j < nb) {
          const float* xp = x + (int64_t)(b0 + j) * K + k;
          const f32x4 x0 = *reinterpret_cast<const f32x4*>(xp);
          const f32x4 x1 = *reinterpret_cast<const f32x4*>(xp + 4);
          accv[j] += w[0] * x0.x + w[1] * x0.y + w[2] * x0.z + w[3] * x0.w + w[4] * x1.x + w[5] * x1.y + w[6] * x1.z +
                     w[7] * x1.w;
        }
      }
    }
    float bias = 0.f;
    if (biasv) bias = W_F32 ? reinterpret_cast<const float*>(biasv)[n]
                            : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(biasv)[n]);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (j < nb) {
        float v = wave_sum(accv[j]) + bias;
        if (act == AERIS_ACT_SILU) v = silu_f(v);
        if (lane == 0) y[(int64_t)(b0 + j) * N + n] = v;
      }
    }
  }
}

hipError_t modulation_linear_launch(const float* x, const void* W, const void* bias, float* y, int B, int N, int K,
                                    int w_dtype, int act, hipStream_t stream) {
  dim3 grid((N + 3) / 4), block(256);
  if (w_dtype == AERIS_F32)
    hipLaunchKernelGGL((modulation_linear_kernel<true>), grid, block, 0, stream, x, W, bias, y, B, N, K, act);
  else
    hipLaunchKernelGGL((modulation_linear_kernel<false>), grid, block, 0, stream, x, W, bias, y, B, N, K, act);
  return hipGetLastError();
}

// emb[b, k] = sin(t_b * f_k), emb[b, half + k] = cos(t_b * f_k), f_k = exp(-ln(max_period) * k / half)
__global__ void timestep_embedding_kernel(const float* __restrict__ t, float* __restrict__ emb, int B, int dim,
                                          float neg_log_period) {
  const int half = dim / 2;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= B * half) return;
  const int b = i / half, k = i - b * half;
  const float f = expf(neg_log_period * (float)k / (float)half);
  const float a = t[b] * f;
  emb[(int64_t)b * dim + k] = sinf(a);
  emb[(int64_t)b * dim + half + k] = cosf(a);
}

hipError_t timestep_embedding_launch(const float* t, float* emb, int B, int dim, float max_period, hipStream_t stream) {
  const int n = B * (dim / 2);
  hipLaunchKernelGGL(timestep_embedding_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, t, emb, B, dim,
                     -logf(max_period));
  return hipGetLastError();
}

// out[m, :] = [x0[m, :] / div0 | x1[m, :]] + ape[m % M_ape, :] as bf16, zero padded to K_pad columns (x1 may be
// absent).  One thread per 8 output columns.
// SPLIT: the C values v are written three times and followed by two ones, [hi | lo | hi | 1 | 1] with hi = bf16(v),
// lo = bf16(v - hi); against a weight matrix laid out [W_hi | W_hi | W_lo | b_hi | b_lo] the bf16 GEMM then returns
// v W^T + b to about 2^-16 relative (hi W_hi + lo W_hi + hi W_lo; only lo W_lo is dropped), which is what keeps the
// embedding at the accuracy of the reference's fp32 Linear.
template <bool SPLIT>
__global__ void __launch_bounds__(256) embed_prepare_kernel(const float* __restrict__ x0, int C0, float div0,
                                                           const float* __restrict__ x1, int C1,
                                                           const float* __restrict__ ape, uint16_t* __restrict__ out,
                                                           int64_t M, int64_t M_ape, int K_pad) {
  const int cpr = K_pad / 8;
  const int C = C0 + C1;
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= M * cpr) return;
  const int64_t m = i / cpr;
  const int k0 = (int)(i - m * cpr) * 8;
  const float* r0 = x0 + m * C0;
  const float* r1 = x1 ? x1 + m * C1 : nullptr;
  const float* ar = ape ? ape + (m % M_ape) * C : nullptr;
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    int k = k0 + e;
    bool lo = false;
    v[e] = 0.f;
    if (SPLIT) {
      if (k >= 3 * C) { if (k < 3 * C + 2) v[e] = 1.f; k = C; }
      else if (k >= 2 * C) k -= 2 * C;
      else if (k >= C) { k -= C; lo = true; }
    }
    if (k < C) {
      const float xv = k < C0 ? (div0 == 1.0f ? r0[k] : r0[k] / div0) : r1[k - C0];
      const float val = xv + (ar ? ar[k] : 0.f);
      v[e] = lo ? val - bf16_bits_to_f32(f32_to_bf16_bits(val)) : val;
    }
  }
  u32x4 w = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
  *reinterpret_cast<u32x4*>(out + m * K_pad + k0) = w;
}

hipError_t embed_prepare_launch(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape, void* out,
                                int64_t M, int64_t M_ape, int K_pad, int split, hipStream_t stream) {
  const int64_t n = M * (K_pad / 8);
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  if (split)
    hipLaunchKernelGGL(embed_prepare_kernel<true>, grid, block, 0, stream, x0, C0, div0, x1, C1, ape,
                       reinterpret_cast<uint16_t*>(out), M, M_ape, K_pad);
  else
    hipLaunchKernelGGL(embed_prepare_kernel<false>, grid, block, 0, stream, x0, C0, div0, x1, C1, ape,
                       reinterpret_cast<uint16_t*>(out), M, M_ape, K_pad);
  return hipGetLastError();
}

}  // namespace aeris
