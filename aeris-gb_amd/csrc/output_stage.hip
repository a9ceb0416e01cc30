// Output stage in one pass over the tokens:  out = head(modulate(norm(x), shift, scale))
// (src/aeris_wp_inference/model.py:421-429: cast to fp32, RMSNorm / LayerNorm, x * (1 + scale) + shift, Linear
// without bias to the output channels).  HBM-bound: x [M, d] is read once, nothing of size M x d is written.
//
// The per-column factors do not depend on the row, so they are folded into the weight once per call:
//     W'[n, k] = W[n, k] * gamma[k] * (1 + scale[k])          u[n] = sum_k W'[n, k]
//     cst[n]   = sum_k W[n, k] * (beta[k] * (1 + scale[k]) + shift[k])
//     out[m, n] = r_m * (sum_k (x[m, k] - c_m) W'[n, k] - (mean_m - c_m) u[n]) + cst[n],   r_m = rsqrt(var_m + eps)
// so one sweep over a row accumulates its statistics and its products together and the normalised row never
// exists.  c_m is a provisional centre taken from the row's first 32 elements (0 for RMSNorm): the products are
// formed on x - c_m, so the correction term (mean_m - c_m) u[n] is small against them whatever the row's mean, and
// the variance is mean((x - c)^2) - (mean - c)^2 without cancellation.
//
// Arithmetic: bf16 MFMA at fp32 accuracy.  x - c and W' are each split into a bf16 head and a bf16 remainder
// (hi = bf16(v), lo = bf16(v - hi)); hi*hi + lo*hi + hi*lo are accumulated in fp32, only lo*lo (2^-16 relative) is
// dropped.  One wave owns 16 rows and all output columns (NF fragments of 16); a workgroup of four waves streams the
// folded weight through LDS in chunks of 64 k, stored in global memory in the order the MFMA operand wants it
// (fragment-ready: 16 bytes per lane, lanes consecutive), so staging is a plain copy and every fragment read is one
// conflict-free ds_read_b128.
#include "common.h"
#include "kernels.h"
#include <mutex>

namespace aeris {

namespace {
constexpr int OS_ROWS = 64, OS_THREADS = 256;

// Scratch of the entry point that allocates nothing (aeris_output_stage_noalloc_fwd): the per-call fold of the
// modulation into the head weight lives in this array instead of a caller's workspace.  Every GPU the library runs
// on holds its own copy until the process ends.  In host code the name below is only a handle: the array's device
// address is looked up once per device with hipGetSymbolAddress and that pointer is what the kernels receive.
constexpr int64_t OS_SCRATCH_BYTES = 2 << 20;
static __device__ __align__(256) unsigned char scratch[OS_SCRATCH_BYTES];
constexpr int OS_MAX_DEVICES = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[OS_MAX_DEVICES] = {};

struct OutStageParams {
  const void* x;
  const unsigned char* wp;  // per modulation batch entry: [d / 32][hi, lo][NF][64 lanes][8] bf16
  const float* u;           // [B_mod][NF * 16]
  const float* cst;         // [B_mod][NF * 16]
  float* out;
  int64_t M;
  int64_t rows_per_batch;
  int batched;
  int N, d;
  float eps;
};

struct FoldParams {
  const float* W;  // [N, d]
  const void* gamma;
  const void* beta;
  int param_f32;
  const float* shift;
  const float* scale;
  int64_t mod_batch_stride;
  int B_mod, N, d, NF;
  unsigned char* wp;
  float* u;
  float* cst;
};

__device__ __forceinline__ float param_at(const void* p, int f32, int k) {
  return f32 ? reinterpret_cast<const float*>(p)[k] : bf16_bits_to_f32(reinterpret_cast<const uint16_t*>(p)[k]);
}

// one thread per 16-byte piece of the fragment-ready split weight
__global__ void __launch_bounds__(256) output_fold_weight_kernel(FoldParams p) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per_ks = 2 * p.NF * 64, per_b = (p.d / 32) * per_ks;
  if (t >= (int64_t)p.B_mod * per_b) return;
  const int b = (int)(t / per_b);
  int r = (int)(t - (int64_t)b * per_b);
  const int ks = r / per_ks;
  r -= ks * per_ks;
  const int part = r / (p.NF * 64);
  r -= part * p.NF * 64;
  const int j = r >> 6, lane = r & 63;
  const int n = 16 * j + (lane & 15), k0 = 32 * ks + 8 * (lane >> 4);
  const float* sc = p.scale ? p.scale + (int64_t)b * p.mod_batch_stride : nullptr;
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int k = k0 + e;
    float w = 0.f;
    if (n < p.N) w = p.W[(int64_t)n * p.d + k] * param_at(p.gamma, p.param_f32, k) * (sc ? 1.f + sc[k] : 1.f);
    const float hi = bf16_bits_to_f32(f32_to_bf16_bits(w));
    v[e] = part ? w - hi : hi;
  }
  const u32x4 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
  *reinterpret_cast<u32x4*>(p.wp + t * 16) = o;
}

// one wave per (batch entry, output column): u and cst
__global__ void __launch_bounds__(256) output_fold_vectors_kernel(FoldParams p) {
  const int lane = threadIdx.x & 63;
  const int nfc = p.NF * 16;
  const int idx = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (idx >= p.B_mod * nfc) return;
  const int b = idx / nfc, n = idx - b * nfc;
  const float* sc = p.scale ? p.scale + (int64_t)b * p.mod_batch_stride : nullptr;
  const float* sh = p.shift ? p.shift + (int64_t)b * p.mod_batch_stride : nullptr;
  float su = 0.f, sc_ = 0.f;
  if (n < p.N) {
    for (int k = lane; k < p.d; k += 64) {
      const float w = p.W[(int64_t)n * p.d + k];
      const float s1 = sc ? 1.f + sc[k] : 1.f;
      const float be = p.beta ? param_at(p.beta, p.param_f32, k) : 0.f;
      su += w * param_at(p.gamma, p.param_f32, k) * s1;
      sc_ += w * (be * s1 + (sh ? sh[k] : 0.f));
    }
  }
  su = wave_sum(su);
  sc_ = wave_sum(sc_);
  if (lane == 0) {
    p.u[idx] = su;
    p.cst[idx] = sc_;
  }
}

template <int NF, bool X_F32, bool LN>
__global__ void __launch_bounds__(OS_THREADS) output_stage_kernel(OutStageParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int NFC = NF * 16;
  constexpr int CHUNK_BYTES = 2 * 2 * NF * 1024;  // two k-steps of 32 x (hi, lo) x NF fragments of 1 KB
  float* const stg = reinterpret_cast<float*>(smem + 2 * CHUNK_BYTES);  // [64][N] results of the tile

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, l15 = lane & 15, q = lane >> 4;
  const int64_t m0 = (int64_t)blockIdx.x * OS_ROWS;
  const int d = p.d, NC = d / 64;
  const int64_t b = p.batched ? m0 / p.rows_per_batch : 0;
  const unsigned char* const wsrc = p.wp + b * (int64_t)d * NFC * 4;
  int64_t row = m0 + wave * 16 + l15;
  if (row > p.M - 1) row = p.M - 1;  // rows below the matrix recompute its last row and are not stored
  const unsigned char* const xrow = reinterpret_cast<const unsigned char*>(p.x) + row * d * (X_F32 ? 4 : 2);

  struct XC { u32x4 a[2], b[2]; };  // a lane's 8 elements of the two k-steps of a chunk
  auto load_x = [&](int c, XC& r) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int off = 64 * c + 32 * kk + 8 * q;
      if (X_F32) {
        r.a[kk] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xrow + off * 4));
        r.b[kk] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xrow + off * 4 + 16));
      } else {
        r.a[kk] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(xrow + off * 2));
        r.b[kk] = u32x4{0u, 0u, 0u, 0u};
      }
    }
  };
  auto unpack = [&](const XC& r, int kk, float (&v)[8]) {
    if (X_F32) {
#pragma unroll
      for (int e = 0; e < 4; ++e) { v[e] = __uint_as_float(r.a[kk][e]); v[4 + e] = __uint_as_float(r.b[kk][e]); }
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) { v[2 * e] = bf16_lo(r.a[kk][e]); v[2 * e + 1] = bf16_hi(r.a[kk][e]); }
    }
  };
  u32x4 wreg[NF];
  auto load_w = [&](int c) {
#pragma unroll
    for (int i = 0; i < NF; ++i)
      wreg[i] = *reinterpret_cast<const u32x4*>(wsrc + (int64_t)c * CHUNK_BYTES + (tid + i * OS_THREADS) * 16);
  };
  auto store_w = [&](int stage) {
#pragma unroll
    for (int i = 0; i < NF; ++i)
      *reinterpret_cast<u32x4*>(smem + stage * CHUNK_BYTES + (tid + i * OS_THREADS) * 16) = wreg[i];
  };

  XC cur, n1, n2;
  load_x(0, cur);
  n1 = cur;
  n2 = cur;
  if (NC > 1) load_x(1, n1);
  load_w(0);
  store_w(0);

  float cen = 0.f;
  if (LN) {  // provisional centre: mean of the row's first 32 elements (held by the four lanes of the row)
    float v[8];
    unpack(cur, 0, v);
    float s = ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    s += __shfl_xor(s, 16);
    s += __shfl_xor(s, 32);
    cen = s * (1.0f / 32.0f);
  }
  __syncthreads();

  f32x4 acc[NF];
#pragma unroll
  for (int j = 0; j < NF; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  float s1 = 0.f, s2 = 0.f;

  for (int c = 0; c < NC; ++c) {
    if (c + 1 < NC) load_w(c + 1);
    if (c + 2 < NC) load_x(c + 2, n2);
    const unsigned char* const ws = smem + (c & 1) * CHUNK_BYTES;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      float v[8];
      unpack(cur, kk, v);
      uint32_t hi[4], lo[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a0 = v[2 * e] - cen, a1 = v[2 * e + 1] - cen;
        s1 += a0 + a1;
        s2 = fmaf(a0, a0, fmaf(a1, a1, s2));
        hi[e] = pack_bf16x2(a0, a1);
        lo[e] = pack_bf16x2(a0 - bf16_lo(hi[e]), a1 - bf16_hi(hi[e]));
      }
      const bf16x8 a_hi = __builtin_bit_cast(bf16x8, u32x4{hi[0], hi[1], hi[2], hi[3]});
      const bf16x8 a_lo = __builtin_bit_cast(bf16x8, u32x4{lo[0], lo[1], lo[2], lo[3]});
#pragma unroll
      for (int j = 0; j < NF; ++j) {
        const bf16x8 w_hi = *reinterpret_cast<const bf16x8*>(ws + ((kk * 2 + 0) * NF + j) * 1024 + lane * 16);
        const bf16x8 w_lo = *reinterpret_cast<const bf16x8*>(ws + ((kk * 2 + 1) * NF + j) * 1024 + lane * 16);
        // weight fragment first: a lane ends up with 4 consecutive output columns of one row
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_hi, a_hi, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_hi, a_lo, acc[j], 0, 0, 0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_lo, a_hi, acc[j], 0, 0, 0);
      }
    }
    if (c + 1 < NC) store_w((c + 1) & 1);
    __syncthreads();
    cur = n1;
    n1 = n2;
  }

  // row statistics: the four lanes of a row (q = 0..3) hold partial sums
  s1 += __shfl_xor(s1, 16);
  s1 += __shfl_xor(s1, 32);
  s2 += __shfl_xor(s2, 16);
  s2 += __shfl_xor(s2, 32);
  const float inv_d = 1.0f / (float)d;
  const float delta = LN ? s1 * inv_d : 0.f;  // mean - centre
  float var = s2 * inv_d - delta * delta;
  if (var < 0.f) var = 0.f;
  const float r = 1.0f / sqrtf(var + p.eps);
  const float* const ub = p.u + b * NFC;
  const float* const cb = p.cst + b * NFC;
  const int N = p.N;
#pragma unroll
  for (int j = 0; j < NF; ++j) {
    const int n0 = 16 * j + 4 * q;
    const f32x4 u4 = *reinterpret_cast<const f32x4*>(ub + n0);
    const f32x4 c4 = *reinterpret_cast<const f32x4*>(cb + n0);
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (n0 + e < N) stg[(wave * 16 + l15) * N + n0 + e] = fmaf(r, acc[j][e] - delta * u4[e], c4[e]);
  }
  __syncthreads();
  // the tile's rows are contiguous in out (row stride N): one linear copy
  int64_t rows_valid = p.M - m0;
  if (rows_valid > OS_ROWS) rows_valid = OS_ROWS;
  const int total = (int)rows_valid * N;
  float* const dst = p.out + m0 * N;
  const int nvec = total >> 2;
  for (int i = tid; i < nvec; i += OS_THREADS)
    reinterpret_cast<f32x4*>(dst)[i] = reinterpret_cast<const f32x4*>(stg)[i];
  for (int i = (nvec << 2) + tid; i < total; i += OS_THREADS) dst[i] = stg[i];
}

template <int NF>
hipError_t launch_main(const OutStageParams& p, bool xf, bool ln, hipStream_t stream) {
  const dim3 grid((unsigned)((p.M + OS_ROWS - 1) / OS_ROWS)), block(OS_THREADS);
  const size_t lds = 2 * (2 * 2 * NF * 1024) + (((size_t)OS_ROWS * p.N * 4 + 15) & ~(size_t)15);
#define GO(XF, LNV) hipLaunchKernelGGL((output_stage_kernel<NF, XF, LNV>), grid, block, lds, stream, p)
  if (xf) { if (ln) GO(true, true); else GO(true, false); }
  else { if (ln) GO(false, true); else GO(false, false); }
#undef GO
  return hipGetLastError();
}
}  // namespace

int64_t output_stage_scratch_capacity() { return OS_SCRATCH_BYTES; }

// Device address of `scratch` on the current device; looked up on the first call per device (hipGetSymbolAddress is
// not a stream operation: make that first call, e.g. through aeris_init, outside any stream capture).
hipError_t output_stage_scratch(void** ptr, bool lookup_allowed) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (dev < 0 || dev >= OS_MAX_DEVICES) return hipErrorInvalidDevice;
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    if (!lookup_allowed) return hipErrorNotReady;
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    g_scratch_ptr[dev] = p;
  }
  *ptr = g_scratch_ptr[dev];
  return hipSuccess;
}

bool output_stage_supported(int N, int d) { return N >= 1 && N <= 80 && d >= 64 && d % 64 == 0; }

int64_t output_stage_workspace_bytes(int N, int d, int B_mod) {
  const int64_t nfc = (int64_t)((N + 15) / 16) * 16;
  return (int64_t)B_mod * ((int64_t)d * nfc * 4 + nfc * 8);
}

hipError_t output_stage_launch(const void* x, int x_dtype, const void* gamma, const void* beta, int param_dtype,
                               const float* shift, const float* scale, int64_t mod_batch_stride, const float* head_w,
                               float* out, int64_t B, int64_t rows_per_batch, int N, int d, int kind, float eps,
                               void* workspace, hipStream_t stream) {
  const int NF = (N + 15) / 16, nfc = NF * 16;
  const bool batched = (shift || scale) && mod_batch_stride != 0 && B > 1;
  const int B_mod = batched ? (int)B : 1;
  unsigned char* ws = reinterpret_cast<unsigned char*>(workspace);
  FoldParams f;
  f.W = head_w; f.gamma = gamma; f.beta = beta; f.param_f32 = param_dtype == AERIS_F32;
  f.shift = shift; f.scale = scale; f.mod_batch_stride = batched ? mod_batch_stride : 0;
  f.B_mod = B_mod; f.N = N; f.d = d; f.NF = NF;
  f.wp = ws;
  f.u = reinterpret_cast<float*>(ws + (int64_t)B_mod * d * nfc * 4);
  f.cst = f.u + (int64_t)B_mod * nfc;
  const int64_t pieces = (int64_t)B_mod * (d / 32) * 2 * NF * 64;
  hipLaunchKernelGGL(output_fold_weight_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, stream, f);
  hipLaunchKernelGGL(output_fold_vectors_kernel, dim3((unsigned)((B_mod * nfc + 3) / 4)), dim3(256), 0, stream, f);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  OutStageParams p;
  p.x = x; p.wp = f.wp; p.u = f.u; p.cst = f.cst; p.out = out;
  p.M = B * rows_per_batch; p.rows_per_batch = rows_per_batch; p.batched = batched ? 1 : 0;
  p.N = N; p.d = d; p.eps = eps;
  const bool xf = x_dtype == AERIS_F32, ln = kind == AERIS_NORM_LAYER;
  switch (NF) {
    case 1: return launch_main<1>(p, xf, ln, stream);
    case 2: return launch_main<2>(p, xf, ln, stream);
    case 3: return launch_main<3>(p, xf, ln, stream);
    case 4: return launch_main<4>(p, xf, ln, stream);
    default: return launch_main<5>(p, xf, ln, stream);
  }
}

}  // namespace aeris
