// Fused windowed multi-head self-attention for gfx950.
//
// One workgroup = one (window, head).  Window partition, window reverse and the cyclic half-window
// shift exist only as address arithmetic: the token at window position p = iy*WS_X + ix of window
// (wy, wx) is row  b*H*W + ((wy*WS_Y + iy + sy) mod H)*W + ((wx*WS_X + ix + sx) mod W)  of the
// natural-order qkv / out matrices, for loads and for stores alike.
//
// Data flow per workgroup (NW waves, wave w owns queries 32w .. 32w+31):
//   K  [L][HD]   global -> LDS rows padded by 16 B (bank-conflict-free ds_read_b128 fragments)
//   V  [L][HD]   global -> registers (4 keys x 8 d per thread) -> 4x8 register transpose ->
//                LDS as V^T [HD][LPAD] so that PV fragments are key-contiguous ds_read_b64
//   bias table   column of this head -> LDS as fp32 4-vectors R4[s] = (R[s..s+3]), R reversed and
//                pre-multiplied by log2(e): the biases of 4 consecutive keys are one ds_read_b128
//   Q            global -> registers (MFMA B operand), never in LDS
//   S^T = K Q^T  v_mfma_f32_32x32x16_bf16, accumulators: lane = one query, 16*NW... keys
//   softmax      in registers; lane = query so the row max / sum need one cross-lane exchange
//                (lane ^ 32); exp2 with scale*log2(e) folded into one FMA
//   O^T = V^T P^T  P^T taken straight from the S^T accumulator registers as the B operand; the
//                k-slot permutation this implies is mirrored in the V^T fragment reads
//   store        4 consecutive d per lane (8 B) to the folded token row
#include "common.h"
#include "kernels.h"

namespace aeris {

struct AttnParams {
  const uint16_t* qkv;
  uint16_t* out;
  const uint16_t* table;  // [(2WS_Y-1)(2WS_X-1), heads] bf16
  int B, H, W, heads;
  int nWy, nWx;
  int sy, sx;
  int use_mask;
  float scale;
};

template <int WS_Y, int WS_X, int HD, bool HAS_BIAS>
struct AttnCfg {
  static constexpr int L = WS_Y * WS_X;
  static constexpr int NW = (L + 31) / 32;
  static constexpr int LPAD = NW * 32;
  static constexpr int NT = NW * 64;
  static constexpr int KROW = HD * 2 + 16;    // bytes
  static constexpr int VROW = LPAD * 2 + 8;   // bytes
  static constexpr int TBL = (2 * WS_Y - 1) * (2 * WS_X - 1);
  static constexpr int K_BYTES = LPAD * KROW;
  static constexpr int V_BYTES = ((HD * VROW + 15) / 16) * 16;
  static constexpr int B_BYTES = HAS_BIAS ? TBL * 16 : 0;
  static constexpr int SMEM = K_BYTES + V_BYTES + B_BYTES;
};

constexpr int attn_threads(int ws_y, int ws_x) { return ((ws_y * ws_x + 31) / 32) * 64; }

template <int WS_Y, int WS_X, int HD, bool HAS_BIAS>
__global__ void __launch_bounds__(attn_threads(WS_Y, WS_X)) window_attention_kernel(AttnParams p) {
  using Cfg = AttnCfg<WS_Y, WS_X, HD, HAS_BIAS>;
  constexpr int L = Cfg::L, NW = Cfg::NW, LPAD = Cfg::LPAD, NT = Cfg::NT;
  constexpr int KROW = Cfg::KROW, VROW = Cfg::VROW, TBL = Cfg::TBL;
  constexpr int CH = HD / 8;   // 16-byte chunks per head row
  constexpr int KS = HD / 16;  // k16 steps of QK^T
  constexpr int DB = HD / 32;  // 32-row blocks of O^T
  static_assert(WS_X % 4 == 0, "groups of 4 consecutive keys must stay inside one window row");
  constexpr float LOG2E = 1.4426950408889634f;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  unsigned char* sK = smem;
  unsigned char* sV = smem + Cfg::K_BYTES;
  unsigned char* sB = smem + Cfg::K_BYTES + Cfg::V_BYTES;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l31 = lane & 31, hi = lane >> 5;

  const int head = blockIdx.x % p.heads;
  const int win = blockIdx.x / p.heads;
  const int wpi = p.nWy * p.nWx;
  const int b = win / wpi;
  const int wrem = win - b * wpi;
  const int wy = wrem / p.nWx, wx = wrem - wy * p.nWx;
  const int H = p.H, W = p.W;
  const int inner = p.heads * HD;
  const int64_t ld_qkv = 3 * (int64_t)inner;
  const int64_t img_base = (int64_t)b * H * W;
  const int y0 = wy * WS_Y + p.sy, x0 = wx * WS_X + p.sx;

  auto token_row = [&](int pos) -> int64_t {
    int Y = y0 + pos / WS_X;
    int X = x0 + pos % WS_X;
    if (Y >= H) Y -= H;
    if (X >= W) X -= W;
    return img_base + (int64_t)Y * W + X;
  };

  // ---- K -> LDS
  const uint16_t* kbase = p.qkv + inner + head * HD;
  for (int idx = tid; idx < LPAD * CH; idx += NT) {
    const int key = idx / CH, c = idx % CH;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (key < L) v = *reinterpret_cast<const u32x4*>(kbase + token_row(key) * ld_qkv + c * 8);
    *reinterpret_cast<u32x4*>(sK + key * KROW + c * 16) = v;
  }
  // ---- V -> registers -> transpose 4 keys x 8 d -> LDS V^T
  const uint16_t* vbase = p.qkv + 2 * inner + head * HD;
  for (int idx = tid; idx < (LPAD / 4) * CH; idx += NT) {
    const int kg = idx / CH, c = idx % CH;
    u32x4 r[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      r[j] = u32x4{0u, 0u, 0u, 0u};
      if (kg * 4 < L) r[j] = *reinterpret_cast<const u32x4*>(vbase + token_row(kg * 4 + j) * ld_qkv + c * 8);
    }
#pragma unroll
    for (int w = 0; w < 4; ++w) {  // word w holds d = 8c + 2w (low half) and 8c + 2w + 1 (high half)
      u32x2 lo, hi2;
      lo.x = (r[0][w] & 0xffffu) | (r[1][w] << 16);
      lo.y = (r[2][w] & 0xffffu) | (r[3][w] << 16);
      hi2.x = (r[0][w] >> 16) | (r[1][w] & 0xffff0000u);
      hi2.y = (r[2][w] >> 16) | (r[3][w] & 0xffff0000u);
      *reinterpret_cast<u32x2*>(sV + (c * 8 + 2 * w) * VROW + kg * 8) = lo;
      *reinterpret_cast<u32x2*>(sV + (c * 8 + 2 * w + 1) * VROW + kg * 8) = hi2;
    }
  }
  // ---- bias column -> LDS 4-vectors
  if (HAS_BIAS) {
    float* sBf = reinterpret_cast<float*>(sB);
    for (int j = tid; j < TBL; j += NT) {
      const float r = bf16_bits_to_f32(p.table[(int64_t)(TBL - 1 - j) * p.heads + head]) * LOG2E;  // R[j]
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (j - e >= 0) sBf[(j - e) * 4 + e] = r;  // R4[j-e][e] = R[j]
    }
    // tail components R4[s][e] with s+e >= TBL are never read by a valid key group
  }

  // ---- Q fragments (B operand): lane = query, 8 consecutive d per k16 step
  int qpos = wave * 32 + l31;
  const bool q_valid = qpos < L;
  if (!q_valid) qpos = L - 1;
  const int64_t q_tok = token_row(qpos);
  bf16x8 qf[KS];
  {
    const uint16_t* qp = p.qkv + q_tok * ld_qkv + head * HD + hi * 8;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const bf16x8*>(qp + s * 16);
  }
  __syncthreads();

  // ---- S^T = K Q^T
  f32x16 acc[NW];
#pragma unroll
  for (int kb = 0; kb < NW; ++kb) {
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[kb][e] = 0.f;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const bf16x8 kf = *reinterpret_cast<const bf16x8*>(sK + (kb * 32 + l31) * KROW + (s * 16 + hi * 8) * 2);
      acc[kb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf[s], acc[kb], 0, 0, 0);
    }
  }
  // acc[kb][4g+i] = <k[key], q[query]>, key = 32kb + 8g + 4hi + i, query = qpos

  // ---- cyclic-shift mask: only windows touching the wrapped border carry more than one region
  const int qiy = qpos / WS_X, qix = qpos % WS_X;
  const bool my = p.use_mask && p.sy > 0 && wy == p.nWy - 1;
  const bool mx = p.use_mask && p.sx > 0 && wx == p.nWx - 1;
  if (my || mx) {
    const float neg = -100.0f / p.scale;  // becomes -100 after the scale multiply below
    const int ry_q = my ? (qiy < WS_Y - p.sy ? 1 : 2) : 0;
    const int rx_q = mx ? (qix < WS_X - p.sx ? 1 : 2) : 0;
#pragma unroll
    for (int kb = 0; kb < NW; ++kb)
#pragma unroll
      for (int g = 0; g < 4; ++g)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb * 32 + g * 8 + hi * 4 + i;
          const int kiy = key / WS_X, kix = key % WS_X;
          const int ry_k = my ? (kiy < WS_Y - p.sy ? 1 : 2) : 0;
          const int rx_k = mx ? (kix < WS_X - p.sx ? 1 : 2) : 0;
          if (ry_k != ry_q || rx_k != rx_q) acc[kb][g * 4 + i] += neg;
        }
  }

  // ---- logits in the exp2 domain, row max
  const float c = p.scale * LOG2E;
  const int sp = (TBL - 1) - (qiy + WS_Y - 1) * (2 * WS_X - 1) - qix - (WS_X - 1);
  float mrow = -INFINITY;
#pragma unroll
  for (int kb = 0; kb < NW; ++kb)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int key0 = kb * 32 + g * 8 + hi * 4;
      const bool valid = (LPAD == L) || key0 < L;
      f32x4 bv = {0.f, 0.f, 0.f, 0.f};
      if (HAS_BIAS) {
        const int kk = valid ? key0 : 0;
        const int qt = (kk / WS_X) * (2 * WS_X - 1) + (kk % WS_X);
        bv = *reinterpret_cast<const f32x4*>(sB + (sp + qt) * 16);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float t = fmaf(acc[kb][g * 4 + i], c, bv[i]);
        if (!valid) t = -INFINITY;
        acc[kb][g * 4 + i] = t;
        mrow = fmaxf(mrow, t);
      }
    }
  mrow = fmaxf(mrow, __shfl_xor(mrow, 32, 64));

  // ---- P = exp2(t - max), row sum, pack to bf16 (B operand of PV)
  float sum = 0.f;
  uint32_t pk[NW][8];
#pragma unroll
  for (int kb = 0; kb < NW; ++kb)
#pragma unroll
    for (int h2 = 0; h2 < 8; ++h2) {
      const float e0 = __builtin_amdgcn_exp2f(acc[kb][2 * h2] - mrow);
      const float e1 = __builtin_amdgcn_exp2f(acc[kb][2 * h2 + 1] - mrow);
      sum += e0 + e1;
      pk[kb][h2] = pack_bf16x2(e0, e1);
    }
  sum += __shfl_xor(sum, 32, 64);
  const float inv = 1.0f / sum;

  // ---- O^T = V^T P^T
  f32x16 o[DB];
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
#pragma unroll
  for (int kb = 0; kb < NW; ++kb)
#pragma unroll
    for (int t2 = 0; t2 < 2; ++t2) {
      // k slots 0-3 <-> keys 32kb+16t2+4hi+(0..3); slots 4-7 <-> keys 32kb+16t2+8+4hi+(0..3)
      u32x4 pw = {pk[kb][4 * t2], pk[kb][4 * t2 + 1], pk[kb][4 * t2 + 2], pk[kb][4 * t2 + 3]};
      const bf16x8 pf = __builtin_bit_cast(bf16x8, pw);
      const int kofs = (kb * 32 + t2 * 16 + hi * 4) * 2;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const unsigned char* vp = sV + (db * 32 + l31) * VROW + kofs;
        const u32x2 v0 = *reinterpret_cast<const u32x2*>(vp);
        const u32x2 v1 = *reinterpret_cast<const u32x2*>(vp + 16);
        u32x4 vw = {v0.x, v0.y, v1.x, v1.y};
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vw), pf, o[db], 0, 0, 0);
      }
    }

  // ---- normalise and store: o[db][4g+i] = O[query][32db + 8g + 4hi + i]
  if (q_valid) {
    uint16_t* op = p.out + q_tok * inner + head * HD + hi * 4;
#pragma unroll
    for (int db = 0; db < DB; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w2;
        w2.x = pack_bf16x2(o[db][g * 4] * inv, o[db][g * 4 + 1] * inv);
        w2.y = pack_bf16x2(o[db][g * 4 + 2] * inv, o[db][g * 4 + 3] * inv);
        *reinterpret_cast<u32x2*>(op + db * 32 + g * 8) = w2;
      }
  }
}

// ---------------------------------------------------------------------------------------------

#define AERIS_ATTN_SHAPES(X) X(8, 8, 32) X(8, 8, 64) X(12, 12, 32) X(12, 12, 64) X(16, 16, 32) X(16, 16, 64)

bool attention_supported(int ws_y, int ws_x, int head_dim) {
#define CHK(Y, Xx, D) if (ws_y == Y && ws_x == Xx && head_dim == D) return true;
  AERIS_ATTN_SHAPES(CHK)
#undef CHK
  return false;
}

hipError_t attention_configure_all() {
  hipError_t e;
#define CFG1(Y, Xx, D, Bi)                                                                                     \
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(window_attention_kernel<Y, Xx, D, Bi>),                 \
                          hipFuncAttributeMaxDynamicSharedMemorySize, AttnCfg<Y, Xx, D, Bi>::SMEM);             \
  if (e != hipSuccess) return e;
#define CFG(Y, Xx, D) CFG1(Y, Xx, D, true) CFG1(Y, Xx, D, false)
  AERIS_ATTN_SHAPES(CFG)
#undef CFG
#undef CFG1
  return hipSuccess;
}

template <int WS_Y, int WS_X, int HD, bool HAS_BIAS>
static hipError_t launch_attn(const AttnParams& p, hipStream_t stream) {
  using Cfg = AttnCfg<WS_Y, WS_X, HD, HAS_BIAS>;
  const int64_t grid = (int64_t)p.B * p.nWy * p.nWx * p.heads;
  hipLaunchKernelGGL((window_attention_kernel<WS_Y, WS_X, HD, HAS_BIAS>), dim3((unsigned)grid), dim3(Cfg::NT),
                     Cfg::SMEM, stream, p);
  return hipGetLastError();
}

hipError_t attention_launch(const void* qkv, void* out, const void* bias_table, int B, int H, int W, int heads,
                            int head_dim, int ws_y, int ws_x, int shift_y, int shift_x, int use_mask, float scale,
                            hipStream_t stream) {
  AttnParams p;
  p.qkv = reinterpret_cast<const uint16_t*>(qkv);
  p.out = reinterpret_cast<uint16_t*>(out);
  p.table = reinterpret_cast<const uint16_t*>(bias_table);
  p.B = B; p.H = H; p.W = W; p.heads = heads;
  p.nWy = H / ws_y; p.nWx = W / ws_x;
  p.sy = shift_y; p.sx = shift_x;
  p.use_mask = use_mask;
  p.scale = scale;
#define DISPATCH(Y, Xx, D)                                                                      \
  if (ws_y == Y && ws_x == Xx && head_dim == D)                                                 \
    return bias_table ? launch_attn<Y, Xx, D, true>(p, stream) : launch_attn<Y, Xx, D, false>(p, stream);
  AERIS_ATTN_SHAPES(DISPATCH)
#undef DISPATCH
  return hipErrorInvalidValue;
}

}  // namespace aeris
