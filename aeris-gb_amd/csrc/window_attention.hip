// Fused windowed multi-head self-attention for gfx950.
//
// One workgroup = one (window, head).  Window partition, window reverse and the cyclic half-window
// shift exist only as address arithmetic: the token at window position p = iy*WS_X + ix of window
// (wy, wx) is row  b*H*W + ((wy*WS_Y + iy + sy) mod H)*W + ((wx*WS_X + ix + sx) mod W)  of the
// natural-order qkv / out matrices, for loads and for stores alike.
//
// Data flow per workgroup (ceil(NQ/2) waves; wave w processes the 32-query groups w and w + NWAVES one after
// the other, so that a workgroup is small enough for two of them to share a CU: while one loads its K / V,
// the other computes):
//   K  [L][HD]   global -> LDS, 16-byte chunks XOR-swizzled (bank-conflict-free ds_read_b128 fragments)
//   V  [L][HD]   global -> registers (4 keys x 8 d per thread) -> 4x8 register transpose ->
//                LDS as V^T [HD][LPAD], key groups permuted so that a PV fragment is one ds_read_b128
//   bias table   column of this head -> LDS as fp32 4-vectors R4[s] = (R[s..s+3]), R reversed and
//                divided by the scale: the biases of 4 consecutive keys are one ds_read_b128
//   Q            global -> registers (MFMA B operand), never in LDS
//   S^T = K Q^T  v_mfma_f32_32x32x16_bf16, accumulators: lane = one query, 16 keys per 32-key block; they start at the
//                bias (read from LDS straight into them), so the bias costs no add and the accumulators no zero-fill
//   softmax      in registers; lane = query so the row max / sum need one cross-lane exchange
//                (lane ^ 32); exp2 with scale*log2(e) folded into one FMA
//   O^T = V^T P^T  P^T taken straight from the S^T accumulator registers as the B operand; the
//                k-slot permutation this implies is mirrored in the V^T fragment reads
//   store        8 consecutive d per lane (16 B, after a lane-half swap) to the folded token row
// LDS reads are software-pipelined by hand (K fragments one key block ahead, bias vectors two, V^T fragments one 16-key
// step ahead of their use); q / k / v are addressed through strides, so they may be the columns of one [tokens, 3*inner]
// matrix or one [tokens, head_dim] plane per part and head.
#include "common.h"
#include "attention_sweep.h"
#include "kernels.h"

namespace aeris {

struct AttnParams {
  const uint16_t* qkv;
  uint16_t* out;
  // where q / k / v of (token, head) start, in elements: part * part_stride + head * head_stride + token * tok_stride
  // ([S, 3 * inner] rows: inner, head_dim, 3 * inner; head planes [3 * heads][S][head_dim]: heads * plane, plane, head_dim)
  int64_t tok_stride, head_stride, part_stride;
  const uint16_t* table;  // [(2WS_Y-1)(2WS_X-1), heads] bf16
  int B, H, W, heads;
  int nWy, nWx;
  int sy, sx;
  int use_mask;
  float scale;
  int q_prescaled;  // q already holds q * scale * log2(e) (the producing GEMM scaled it in fp32 before its only rounding)
};

template <int WS_Y, int WS_X, int HD, bool HAS_BIAS>
struct AttnCfg {
  static constexpr int L = WS_Y * WS_X;
  static constexpr int NQ = (L + 31) / 32;     // 32-query groups (= 32-key blocks)
  static constexpr int LPAD = NQ * 32;
  static constexpr int NWAVES = (NQ + 1) / 2;  // a wave processes query groups w and w + NWAVES in turn
  static constexpr int NT = NWAVES * 64;
  // V^T rows: XOR-swizzled 16-byte chunks when a row holds a multiple of 16 chunks, otherwise padded by 16 B
  static constexpr bool V_SWZ = (LPAD * 2 / 16) % 16 == 0;
  static constexpr int VROW = V_SWZ ? LPAD * 2 : LPAD * 2 + 16;  // bytes
  static constexpr int TBL = (2 * WS_Y - 1) * (2 * WS_X - 1);
  // K rows: 128 B chunk-swizzled (head_dim 64) or 64 B padded to 80 B (head_dim 32)
  static constexpr int K_BYTES = HD == 64 ? LPAD * 128 : LPAD * 80;
  static constexpr int V_BYTES = ((HD * VROW + 15) / 16) * 16;
  static constexpr int B_BYTES = HAS_BIAS ? TBL * 16 : 0;
  static constexpr int SMEM = K_BYTES + V_BYTES + B_BYTES;  // 16x16 x 64 with bias: 80 912 B, two workgroups per CU
};

constexpr int attn_threads(int ws_y, int ws_x) { return (((ws_y * ws_x + 31) / 32 + 1) / 2) * 64; }

// byte offset of 16-byte chunk `chunk` of key row `key` in the K tile
template <int HD>
__device__ __forceinline__ uint32_t k_off(int key, int chunk) {
  if (HD == 64) return (uint32_t)((key >> 1) * 256 + (((((key & 1) << 3) | chunk) ^ ((key >> 1) & 7)) << 4));
  return (uint32_t)(key * 80 + chunk * 16);
}

// XOR pattern of the 16-byte chunks of V^T row d: the fragment reads (16 lanes = 16 consecutive rows, same chunk) are
// conflict-free.  The transposing writes, whose lanes hold rows 8 apart, keep 4-way bank conflicts: also folding
// bits 4-5 of d onto bits 1-2 removes them (LDS conflict cycles -85 % in the counters), but the read addresses then
// no longer share a base: kept in registers they spill (14 % slower), recomputed per step the extra VALU work costs
// 2-3 % - the kernel is bound by its VALU work, not by the LDS.
template <bool SWZ>
__device__ __forceinline__ int v_swz(int d) {
  return SWZ ? (d & 15) : 0;
}

template <int WS_Y, int WS_X, int HD, bool HAS_BIAS>
__global__ void __launch_bounds__(attn_threads(WS_Y, WS_X)) __attribute__((amdgpu_waves_per_eu(2)))
window_attention_kernel(AttnParams p) {  // at least 2 waves per SIMD: two workgroups share a CU
  using Cfg = AttnCfg<WS_Y, WS_X, HD, HAS_BIAS>;
  constexpr int L = Cfg::L, NQ = Cfg::NQ, LPAD = Cfg::LPAD, NT = Cfg::NT, NWAVES = Cfg::NWAVES;
  constexpr int VROW = Cfg::VROW, TBL = Cfg::TBL;
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
  // token rows and the stride between them fit 32 bits (checked by the caller): one 32 x 32 -> 64-bit multiply-add per
  // address instead of a 64 x 64 multiply
  const uint32_t ld_qkv = (uint32_t)p.tok_stride;
  const uint32_t img_base = (uint32_t)b * (uint32_t)(H * W);
  const int y0 = wy * WS_Y + p.sy, x0 = wx * WS_X + p.sx;

  auto token_row = [&](int pos) -> uint32_t {
    int Y = y0 + pos / WS_X;
    int X = x0 + pos % WS_X;
    if (Y >= H) Y -= H;
    if (X >= W) X -= W;
    return img_base + (uint32_t)Y * (uint32_t)W + (uint32_t)X;
  };

  // ---- Q fragments of both query groups of this wave (B operand): lane = query, 8 consecutive d per k16 step.
  // Issued first: they are needed only after the K / V traffic below.
  bf16x8 qf[2][KS];
  uint32_t q_tok[2];
#pragma unroll
  for (int ps = 0; ps < 2; ++ps) {
    int qpos = (wave + ps * NWAVES) * 32 + l31;
    if (qpos >= L) qpos = L - 1;
    q_tok[ps] = token_row(qpos);
    const uint16_t* qp = p.qkv + head * p.head_stride + (uint64_t)q_tok[ps] * ld_qkv + hi * 8;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[ps][s] = *reinterpret_cast<const bf16x8*>(qp + s * 16);
  }

  // ---- all global loads of the workgroup are issued before the first LDS write (one round trip, not one per
  // loop iteration): K chunks, V as 4 keys x 8 d per thread, the head's bias column
  constexpr int K_ITEMS = LPAD * CH, V_ITEMS = (LPAD / 4) * CH;
  constexpr int KIT = (K_ITEMS + NT - 1) / NT, VIT = (V_ITEMS + NT - 1) / NT, BIT = HAS_BIAS ? (TBL + NT - 1) / NT : 1;
  const uint16_t* kbase = p.qkv + p.part_stride + head * p.head_stride;
  const uint16_t* vbase = p.qkv + 2 * p.part_stride + head * p.head_stride;
  u32x4 kreg[KIT], vreg[VIT][4];
  float breg[BIT];
#pragma unroll
  for (int it = 0; it < KIT; ++it) {
    const int idx = tid + it * NT, key = idx / CH, c = idx % CH;
    kreg[it] = u32x4{0u, 0u, 0u, 0u};
    if ((K_ITEMS % NT == 0 || idx < K_ITEMS) && (LPAD == L || key < L))  // both compile-time true for full windows
      kreg[it] = *reinterpret_cast<const u32x4*>(kbase + (uint64_t)token_row(key) * ld_qkv + c * 8);
  }
#pragma unroll
  for (int it = 0; it < VIT; ++it) {
    const int idx = tid + it * NT, kg = idx / CH, c = idx % CH;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      vreg[it][j] = u32x4{0u, 0u, 0u, 0u};
      if ((V_ITEMS % NT == 0 || idx < V_ITEMS) && (LPAD == L || kg * 4 < L))
        vreg[it][j] = *reinterpret_cast<const u32x4*>(vbase + (uint64_t)token_row(kg * 4 + j) * ld_qkv + c * 8);
    }
  }
  if (HAS_BIAS) {
#pragma unroll
    for (int it = 0; it < BIT; ++it) {
      const int j = tid + it * NT;
      breg[it] = j < TBL ? bf16_bits_to_f32(p.table[(int64_t)(TBL - 1 - j) * p.heads + head]) * LOG2E : 0.f;  // R[j]
    }
  }
  // every load above is in flight before the first LDS write below waits for one of them
  __builtin_amdgcn_sched_barrier(0);
  // ---- K -> LDS
#pragma unroll
  for (int it = 0; it < KIT; ++it) {
    const int idx = tid + it * NT, key = idx / CH, c = idx % CH;
    if (K_ITEMS % NT == 0 || idx < K_ITEMS) *reinterpret_cast<u32x4*>(sK + k_off<HD>(key, c)) = kreg[it];
  }
  // ---- V: 4 keys x 8 d register transpose -> LDS as V^T[d][key].  Inside every block of 16 keys the four
  // key groups are stored in the order 0, 2, 1, 3: the 8 keys one lane needs for a k16 step of PV (4hi..4hi+3
  // and 8+4hi..8+4hi+3, the accumulator layout of S^T) are then one aligned 16-byte chunk.  Rows are 2*LPAD
  // bytes, 16-byte chunks XOR-swizzled by the row so that 16 lanes (16 rows, same chunk) hit distinct banks.
#pragma unroll
  for (int it = 0; it < VIT; ++it) {
    const int idx = tid + it * NT, kg = idx / CH, c = idx % CH;
    if (V_ITEMS % NT == 0 || idx < V_ITEMS) {
      const int pos = (kg & ~3) | (((kg & 1) << 1) | ((kg >> 1) & 1));  // swap the two middle groups of a 16-key block
#pragma unroll
      for (int w = 0; w < 4; ++w) {  // word w holds d = 8c + 2w (low half) and 8c + 2w + 1 (high half)
        u32x2 lo, hi2;
        lo.x = (vreg[it][0][w] & 0xffffu) | (vreg[it][1][w] << 16);
        lo.y = (vreg[it][2][w] & 0xffffu) | (vreg[it][3][w] << 16);
        hi2.x = (vreg[it][0][w] >> 16) | (vreg[it][1][w] & 0xffff0000u);
        hi2.y = (vreg[it][2][w] >> 16) | (vreg[it][3][w] & 0xffff0000u);
        const int d0 = c * 8 + 2 * w, d1 = d0 + 1;
        *reinterpret_cast<u32x2*>(sV + d0 * VROW + (((pos >> 1) ^ v_swz<Cfg::V_SWZ>(d0)) << 4) + (pos & 1) * 8) = lo;
        *reinterpret_cast<u32x2*>(sV + d1 * VROW + (((pos >> 1) ^ v_swz<Cfg::V_SWZ>(d1)) << 4) + (pos & 1) * 8) = hi2;
      }
    }
  }
  // ---- bias column -> LDS 4-vectors R4[s] = R[s..s+3]
  if (HAS_BIAS) {
    float* sBf = reinterpret_cast<float*>(sB);
#pragma unroll
    for (int it = 0; it < BIT; ++it) {
      const int j = tid + it * NT;
      if (j < TBL) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (j - e >= 0) sBf[(j - e) * 4 + e] = breg[it];  // R4[j-e][e] = R[j]
      }
    }
    // tail components R4[s][e] with s+e >= TBL are never read by a valid key group
  }
  // ---- q * scale * log2(e), rounded to bf16 once more (unless the producer of q has applied the factor already): the
  // accumulators of K Q^T are then the logits in the exp2 domain and P = exp2(acc) needs no multiply
  if (!p.q_prescaled) {
    const float c = p.scale * LOG2E;
#pragma unroll
    for (int ps = 0; ps < 2; ++ps)
#pragma unroll
      for (int s2 = 0; s2 < KS; ++s2) {
        u32x4 w = __builtin_bit_cast(u32x4, qf[ps][s2]);
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(bf16_lo(w[e]) * c, bf16_hi(w[e]) * c);
        qf[ps][s2] = __builtin_bit_cast(bf16x8, w);
      }
  }
  __syncthreads();

  const bool my = p.use_mask && p.sy > 0 && wy == p.nWy - 1;
  const bool mx = p.use_mask && p.sx > 0 && wx == p.nWx - 1;
  auto load_k = [&](int kb, bf16x8 (&f)[KS]) {
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) f[s2] = *reinterpret_cast<const bf16x8*>(sK + k_off<HD>(kb * 32 + l31, s2 * 2 + hi));
  };
  // V^T fragment of PV step `step` (16 keys): k slots 0-3 <-> keys 16 step + 4hi + (0..3), slots 4-7 <-> keys
  // 16 step + 8 + 4hi + (0..3): one 16-byte chunk per 32-row block of O^T
  auto read_v = [&](int step, bf16x8 (&f)[DB]) {
    const int chunk = step * 2 + hi;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int d = db * 32 + l31;
      f[db] = *reinterpret_cast<const bf16x8*>(sV + d * VROW + ((chunk ^ v_swz<Cfg::V_SWZ>(d)) << 4));
    }
  };
  const LoadVPlain<DB, decltype(read_v)> load_v(read_v);

#pragma unroll
  for (int ps = 0; ps < 2; ++ps) {
    const int qg = wave + ps * NWAVES;
    if (qg >= NQ) break;  // wave-uniform
    int qpos = qg * 32 + l31;
    const bool q_valid = qpos < L;
    if (!q_valid) qpos = L - 1;
    const WindowLogits<WS_Y, WS_X, HAS_BIAS> logits(sB, qpos, hi, my, mx, p.sy, p.sx);
    f32x16 o[DB];
    float sum;
    attention_sweep<NQ, KS, DB, HAS_BIAS>(logits, load_k, load_v, [](int) {}, qf[ps], o, sum);
    store_attention_rows<DB>(p.out + (uint64_t)q_tok[ps] * (uint32_t)inner + head * HD + hi * 8, o, sum, q_valid);
  }
}


// ---------------------------------------------------------------------------------------------
// The same computation for head_dim 64 with K and V brought into LDS by the load unit itself
// (buffer_load ... lds: no staging registers, no ds_write, no VALU work) and V kept row-major: the V^T fragments of
// P V come from ds_read_b64_tr_b16, the LDS read that transposes on the way out.
//   layout   K and V rows of 128 B, 16-byte chunks XOR-swizzled: K by (key >> 1) & 7 (16 consecutive keys of one chunk
//            hit distinct banks for the ds_read_b128 fragments), V by 2 (key & 3) (the 4 keys x 4 column groups that
//            one transposing read gathers per 16 lanes hit distinct banks).  A load instruction of a wave fills 1 KB =
//            8 rows; lane l fetches the chunk that the swizzle keeps at its LDS slot, from the folded token row.
//   tr read  within 16 lanes, source lane 4e + a reads 4 consecutive elements and result lane 4a + b receives element b
//            of the source lanes a, 4 + a, 8 + a, 12 + a: with source lane 4e + a at V[key0 + e][d0 + 4a ..] the result
//            lane owns column d0 + (lane & 15) of the keys key0 .. key0 + 3 - half of an MFMA operand's 8 k slots.
// Requires every byte offset inside a q / k / v plane to fit 32 bits (checked by the caller).
template <int WS_Y, int WS_X, bool HAS_BIAS>
struct AttnDmaCfg {
  static constexpr int L = WS_Y * WS_X;
  static constexpr int NQ = (L + 31) / 32;
  static constexpr int LPAD = NQ * 32;
  static constexpr int NWAVES = (NQ + 1) / 2;
  static constexpr int NT = NWAVES * 64;
  static constexpr int TBL = (2 * WS_Y - 1) * (2 * WS_X - 1);
  static constexpr int KV_BYTES = LPAD * 128;
  static constexpr int SMEM = 2 * KV_BYTES + (HAS_BIAS ? TBL * 16 : 0);
};

template <int WS_Y, int WS_X, bool HAS_BIAS>
__global__ void __launch_bounds__(attn_threads(WS_Y, WS_X)) __attribute__((amdgpu_waves_per_eu(2)))
window_attention_dma_kernel(AttnParams p) {
  using Cfg = AttnDmaCfg<WS_Y, WS_X, HAS_BIAS>;
  constexpr int HD = 64, KS = 4, DB = 2;
  constexpr int L = Cfg::L, NQ = Cfg::NQ, LPAD = Cfg::LPAD, NT = Cfg::NT, NWAVES = Cfg::NWAVES, TBL = Cfg::TBL;
  static_assert(WS_X % 4 == 0, "groups of 4 consecutive keys must stay inside one window row");
  constexpr float LOG2E = 1.4426950408889634f;
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  typedef __attribute__((address_space(3))) bf16x4_t* lds_bf16x4_ptr;

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* sK = smem;
  unsigned char* sV = smem + Cfg::KV_BYTES;
  unsigned char* sB = smem + 2 * Cfg::KV_BYTES;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, hi = lane >> 5;

  const int head = blockIdx.x % p.heads;
  const int win = blockIdx.x / p.heads;
  const int wpi = p.nWy * p.nWx;
  const int b = win / wpi;
  const int wrem = win - b * wpi;
  const int wy = wrem / p.nWx, wx = wrem - wy * p.nWx;
  const int H = p.H, W = p.W;
  const int inner = p.heads * HD;
  const uint32_t ld_qkv = (uint32_t)p.tok_stride;
  const uint32_t img_base = (uint32_t)b * (uint32_t)(H * W);
  const int y0 = wy * WS_Y + p.sy, x0 = wx * WS_X + p.sx;

  auto token_row = [&](int pos) -> uint32_t {
    int Y = y0 + pos / WS_X;
    int X = x0 + pos % WS_X;
    if (Y >= H) Y -= H;
    if (X >= W) X -= W;
    return img_base + (uint32_t)Y * (uint32_t)W + (uint32_t)X;
  };

  // ---- K and V: global -> LDS.  Instruction ii fills rows 8 ii .. 8 ii + 7 of both tiles; the waves share them out.
  {
    const uint16_t* kbase = p.qkv + p.part_stride + head * p.head_stride;
    const uint16_t* vbase = p.qkv + 2 * p.part_stride + head * p.head_stride;
    const uint32_t plane_bytes = (uint32_t)p.B * (uint32_t)(H * W) * ld_qkv * 2u;  // < 2^32, checked by the caller
    const __amdgpu_buffer_rsrc_t rs_k = __builtin_amdgcn_make_buffer_rsrc((void*)kbase, 0, (int)plane_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rs_v = __builtin_amdgcn_make_buffer_rsrc((void*)vbase, 0, (int)plane_bytes, 0x00020000);
    const int rsub = lane >> 3, pc = lane & 7;
#pragma unroll
    for (int j = 0; j < (LPAD / 8 + NWAVES - 1) / NWAVES; ++j) {
      const int ii = wave + j * NWAVES;
      if (ii < LPAD / 8) {  // wave-uniform
        const int key = ii * 8 + rsub;
        uint32_t off_k = 0xFFFFFFF0u, off_v = 0xFFFFFFF0u;  // rows past the window: outside the descriptor, arrive as zeros
        if (LPAD == L || key < L) {
          const uint32_t row_off = token_row(key) * (ld_qkv * 2u);
          off_k = row_off + (uint32_t)((pc ^ ((key >> 1) & 7)) << 4);
          off_v = row_off + (uint32_t)((pc ^ (2 * (key & 3))) << 4);
        }
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_k, (lds_ptr)(sK + ii * 1024), 16, off_k, 0, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_v, (lds_ptr)(sV + ii * 1024), 16, off_v, 0, 0, 0);
      }
    }
  }

  // ---- Q fragments of both query groups of this wave (B operand): lane = query, 8 consecutive d per k16 step
  bf16x8 qf[2][KS];
  uint32_t q_tok[2];
#pragma unroll
  for (int ps = 0; ps < 2; ++ps) {
    int qpos = (wave + ps * NWAVES) * 32 + l31;
    if (qpos >= L) qpos = L - 1;
    q_tok[ps] = token_row(qpos);
    const uint16_t* qp = p.qkv + head * p.head_stride + (uint64_t)q_tok[ps] * ld_qkv + hi * 8;
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) qf[ps][s2] = *reinterpret_cast<const bf16x8*>(qp + s2 * 16);
  }

  // ---- bias column of this head -> LDS as fp32 4-vectors R4[s] = R[s..s+3] (R reversed, times log2 e)
  if (HAS_BIAS) build_bias_lds<TBL>(sB, p.table, p.heads, head, tid, NT);
  // ---- q * scale * log2(e): the accumulators of K Q^T are then the logits in the exp2 domain
  if (!p.q_prescaled) {
    const float c = p.scale * LOG2E;
#pragma unroll
    for (int ps = 0; ps < 2; ++ps)
#pragma unroll
      for (int s2 = 0; s2 < KS; ++s2) {
        u32x4 w = __builtin_bit_cast(u32x4, qf[ps][s2]);
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(bf16_lo(w[e]) * c, bf16_hi(w[e]) * c);
        qf[ps][s2] = __builtin_bit_cast(bf16x8, w);
      }
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): this wave's loads into LDS and its bias writes have landed
  __syncthreads();

  const bool my = p.use_mask && p.sy > 0 && wy == p.nWy - 1;
  const bool mx = p.use_mask && p.sx > 0 && wx == p.nWx - 1;

  auto load_k = [&](int kb, bf16x8 (&f)[KS]) {
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) f[s2] = *reinterpret_cast<const bf16x8*>(sK + k_off<64>(kb * 32 + l31, s2 * 2 + hi));
  };
  const uint32_t v_addr = lds_byte_address(sV);
  auto v_step = [&](int step) { return v_addr + (uint32_t)step * 2048u; };
  const LoadVTransposed<DB, decltype(v_step)> load_v(lane, v_step);

#pragma unroll
  for (int ps = 0; ps < 2; ++ps) {
    const int qg = wave + ps * NWAVES;
    if (qg >= NQ) break;  // wave-uniform
    int qpos = qg * 32 + l31;
    const bool q_valid = qpos < L;
    if (!q_valid) qpos = L - 1;
    const WindowLogits<WS_Y, WS_X, HAS_BIAS> logits(sB, qpos, hi, my, mx, p.sy, p.sx);
    f32x16 o[DB];
    float sum;
    attention_sweep<NQ, KS, DB, HAS_BIAS>(logits, load_k, load_v, [](int) {}, qf[ps], o, sum);
    store_attention_rows<DB>(p.out + (uint64_t)q_tok[ps] * (uint32_t)inner + head * HD + hi * 8, o, sum, q_valid);
  }
}

// ---------------------------------------------------------------------------------------------
// Persistent form of the kernel above: one workgroup per CU walks every gridDim-th (head, window) unit, one wave per
// 32-query group, with two K / V buffer sets in LDS.  While the waves compute unit i from one set, the load unit fills
// the other with the workgroup's next unit (buffer_load ... lds costs the waves 8 instructions each and no
// registers), so the HBM stream and the arithmetic overlap inside one workgroup instead of depending on how two
// independent workgroups on a CU happen to interleave.  One workgroup barrier per unit: a wave passes it when its
// share of the next unit has landed; everyone having passed it means the current unit's buffers are free for the unit
// after the next.  Units are numbered head-major and the stride is far smaller than the windows of one head, so a
// workgroup's consecutive units nearly always share the head: its relative-position bias column in LDS is rebuilt
// only when the head changes.
template <int WS_Y, int WS_X, bool HAS_BIAS>
struct AttnPersistCfg {
  static constexpr int L = WS_Y * WS_X;
  static constexpr int NQ = (L + 31) / 32;
  static constexpr int LPAD = NQ * 32;
  static constexpr int NT = NQ * 64;  // one wave per query group
  static constexpr int TBL = (2 * WS_Y - 1) * (2 * WS_X - 1);
  static constexpr int KV_BYTES = LPAD * 128;
  static constexpr int SMEM = 4 * KV_BYTES + (HAS_BIAS ? TBL * 16 : 0);
};

constexpr int attn_persist_threads(int ws_y, int ws_x) { return ((ws_y * ws_x + 31) / 32) * 64; }

template <int WS_Y, int WS_X, bool HAS_BIAS>
__global__ void __launch_bounds__(attn_persist_threads(WS_Y, WS_X))
window_attention_persist_kernel(AttnParams p, int n_units) {
  using Cfg = AttnPersistCfg<WS_Y, WS_X, HAS_BIAS>;
  constexpr int HD = 64, KS = 4, DB = 2;
  constexpr int L = Cfg::L, NQ = Cfg::NQ, LPAD = Cfg::LPAD, NT = Cfg::NT, TBL = Cfg::TBL, KVB = Cfg::KV_BYTES;
  static_assert(WS_X % 4 == 0, "groups of 4 consecutive keys must stay inside one window row");
  constexpr float LOG2E = 1.4426950408889634f;
  constexpr int DMA_PER_WAVE = (LPAD / 8 + NQ - 1) / NQ;  // instruction pairs (K, V) per wave and unit
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  typedef __attribute__((address_space(3))) bf16x4_t* lds_bf16x4_ptr;

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* sB = smem + 4 * KVB;
  const uint32_t smem_addr = lds_byte_address(smem);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l31 = lane & 31, hi = lane >> 5;
  const int H = p.H, W = p.W;
  const int inner = p.heads * HD;
  const uint32_t ld_qkv = (uint32_t)p.tok_stride;
  const int wpi = p.nWy * p.nWx;
  const int n_win = p.B * wpi;

  const int u_begin = blockIdx.x, u_step = gridDim.x;
  if (u_begin >= n_units) return;

  const uint32_t plane_bytes = (uint32_t)p.B * (uint32_t)(H * W) * ld_qkv * 2u;  // < 2^32, checked by the caller
  const int rsub = lane >> 3, pc = lane & 7;

  // A unit = (head, batch entry, window row, window column), numbered window-fastest; everything about it is
  // workgroup-uniform and lives in scalar registers.  A workgroup takes the units u_begin, u_begin + u_step, ...: the
  // windows on the wrapped border of a shifted grid (a whole window row; their mask arithmetic makes them the slow
  // ones) are then spread over all workgroups instead of filling the ranges of a few.  The successor of a unit
  // follows by adding the digits of u_step with carries, without a division.
  struct Unit { int head, b, wy, wx; };
  auto decode = [&](int u) {
    Unit r;
    r.head = u / n_win;
    const int win = u - r.head * n_win;
    r.b = win / wpi;
    const int wrem = win - r.b * wpi;
    r.wy = wrem / p.nWx;
    r.wx = wrem - r.wy * p.nWx;
    return r;
  };
  const Unit step = decode(u_step);
  auto successor = [&](Unit r) {
    r.wx += step.wx;
    int carry = r.wx >= p.nWx;
    r.wx -= carry ? p.nWx : 0;
    r.wy += step.wy + carry;
    carry = r.wy >= p.nWy;
    r.wy -= carry ? p.nWy : 0;
    r.b += step.b + carry;
    carry = r.b >= p.B;
    r.b -= carry ? p.B : 0;
    r.head += step.head + carry;
    return r;
  };
  // Token row of window position (iy, ix): away from the wrapped border (every window of an un-shifted grid, all but
  // the last window row / column of a shifted one) it is the window's first token plus a per-lane constant; `rel` is
  // that constant, iy * W + ix.  Windows on the border take the two conditional subtractions.
  auto window_wraps = [&](const Unit& un) { return (un.wy + 1) * WS_Y + p.sy > H || (un.wx + 1) * WS_X + p.sx > W; };
  auto window_base = [&](const Unit& un) -> uint32_t {
    return (uint32_t)un.b * (uint32_t)(H * W) + (uint32_t)(un.wy * WS_Y + p.sy) * (uint32_t)W + (uint32_t)(un.wx * WS_X + p.sx);
  };
  auto token_row = [&](const Unit& un, int pos) -> uint32_t {  // general form, used on the border only
    int Y = un.wy * WS_Y + p.sy + pos / WS_X;
    int X = un.wx * WS_X + p.sx + pos % WS_X;
    if (Y >= H) Y -= H;
    if (X >= W) X -= W;
    return (uint32_t)un.b * (uint32_t)(H * W) + (uint32_t)Y * (uint32_t)W + (uint32_t)X;
  };
  // K and V of unit `un` -> buffer set `set`: instruction pair ii fills rows 8 ii .. 8 ii + 7 of both tiles; a wave
  // issues pairs wave, wave + NQ, ...  Per pair and lane: key, and the byte offsets of its K / V chunk relative to
  // the window's first token (un-wrapped windows).
  uint32_t kv_relk[DMA_PER_WAVE], kv_relv[DMA_PER_WAVE];
#pragma unroll
  for (int j = 0; j < DMA_PER_WAVE; ++j) {
    const int key = (wave + j * NQ) * 8 + rsub;
    const uint32_t rel = (uint32_t)((key / WS_X) * W + key % WS_X) * (ld_qkv * 2u);
    kv_relk[j] = rel + (uint32_t)((pc ^ ((key >> 1) & 7)) << 4);
    kv_relv[j] = rel + (uint32_t)((pc ^ (2 * (key & 3))) << 4);
  }
  // The loads of a unit: descriptors and the window's base offset (kv_prepare), then one buffer_load ... lds per
  // call of kv_issue.  They are issued back to back right after the unit barrier.  (Spreading them over the key-block
  // loop, one per block, was measured 8 % slower: a load holds the issuing wave while the CU's one address unit
  // takes its 64 addresses, and inside the loop that wait lands on the arithmetic.)
  constexpr int N_DMA = 2 * DMA_PER_WAVE;
  __amdgpu_buffer_rsrc_t kv_rs_k = __builtin_amdgcn_make_buffer_rsrc((void*)p.qkv, 0, 0, 0x00020000);
  __amdgpu_buffer_rsrc_t kv_rs_v = kv_rs_k;
  bool kv_wraps = false;
  uint32_t kv_base = 0;
  Unit kv_unit = {0, 0, 0, 0};
  auto kv_prepare = [&](const Unit& un) {
    const uint16_t* kbase = p.qkv + p.part_stride + un.head * p.head_stride;
    const uint16_t* vbase = p.qkv + 2 * p.part_stride + un.head * p.head_stride;
    kv_rs_k = __builtin_amdgcn_make_buffer_rsrc((void*)kbase, 0, (int)plane_bytes, 0x00020000);
    kv_rs_v = __builtin_amdgcn_make_buffer_rsrc((void*)vbase, 0, (int)plane_bytes, 0x00020000);
    kv_wraps = window_wraps(un);
    kv_base = window_base(un) * (ld_qkv * 2u);
    kv_unit = un;
  };
  // load number idx of the prepared unit -> buffer set `set`: pair idx / 2 (rows 8 ii .. 8 ii + 7), K for even idx, V for odd
  auto kv_issue = [&](int idx, int set) {
    const int j = idx >> 1, is_v = idx & 1;
    const int ii = wave + j * NQ;  // the pairs divide evenly among the waves for every window built here
    const int key = ii * 8 + rsub;
    uint32_t off = kv_base + (is_v ? kv_relv[j] : kv_relk[j]);
    if (kv_wraps)  // wave-uniform: windows on the wrapped border of a shifted grid
      off = token_row(kv_unit, key < L ? key : 0) * (ld_qkv * 2u) + (uint32_t)((pc ^ (is_v ? 2 * (key & 3) : (key >> 1) & 7)) << 4);
    if (LPAD != L && key >= L) off = 0xFFFFFFF0u;  // outside the descriptor: arrives as zeros
    unsigned char* dst = smem + set * 2 * KVB + is_v * KVB + ii * 1024;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(is_v ? kv_rs_v : kv_rs_k, (lds_ptr)dst, 16, off, 0, 0, 0);
  };
  int qpos = wave * 32 + l31;
  const bool q_valid = qpos < L;
  if (!q_valid) qpos = L - 1;
  const int qiy = qpos / WS_X, qix = qpos % WS_X;
  const uint32_t q_rel = (uint32_t)(qiy * W + qix);
  // Q fragments of this wave's query group (B operand: lane = query, 8 consecutive d per k16 step)
  auto load_q = [&](const Unit& un, bf16x8 (&q)[KS], uint32_t& tok) {
    tok = window_wraps(un) ? token_row(un, qpos) : window_base(un) + q_rel;
    const uint16_t* qp = p.qkv + un.head * p.head_stride + (uint64_t)tok * ld_qkv + hi * 8;
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) q[s2] = *reinterpret_cast<const bf16x8*>(qp + s2 * 16);
  };
  auto build_bias = [&](int head) {
    if (HAS_BIAS) build_bias_lds<TBL>(sB, p.table, p.heads, head, tid, NT);
  };

  const float cq = p.scale * LOG2E;
  constexpr float MASK_NEG = -100.0f * LOG2E;

  // A load instruction holds its wave until the CU's one address unit has taken its 64 addresses, and with all waves
  // issuing their share of the next unit together right after the barrier nothing computes meanwhile.  The upper half
  // of the waves (the SIMD partners of the lower half) therefore issues its share STAGGER_KB key blocks into the unit:
  // while one wave of a SIMD queues loads, the other one computes.
#ifndef AERIS_ATTN_STAGGER
#define AERIS_ATTN_STAGGER (NQ >= 4 ? NQ / 2 : 0)
#endif
  constexpr int STAGGER_KB = AERIS_ATTN_STAGGER;
  const bool late_issuer = STAGGER_KB > 0 && wave >= NQ / 2;
  Unit cur = decode(u_begin);
  int bias_head = cur.head;
  bf16x8 q_cur[KS], q_nxt[KS];
  uint32_t tok_cur, tok_nxt = 0;
  static_assert((LPAD / 8) % NQ == 0, "the load pairs must divide evenly among the waves");
  load_q(cur, q_cur, tok_cur);
  kv_prepare(cur);
#pragma unroll
  for (int i = 0; i < N_DMA; ++i) kv_issue(i, 0);
  build_bias(bias_head);
#pragma unroll
  for (int s2 = 0; s2 < KS; ++s2) q_nxt[s2] = q_cur[s2];

  int set = 1;
  for (int u = u_begin; u < n_units; u += u_step) {
    set ^= 1;
    const bool more = u + u_step < n_units;
    const Unit nxt = successor(cur);
    if (HAS_BIAS && cur.head != bias_head) {  // workgroup-uniform and rare: the walk crosses into the next head
      __syncthreads();
      build_bias(cur.head);
      bias_head = cur.head;
    }
    // this wave's loads of unit u (and its bias writes) have landed; only the 4 output stores of the unit before may
    // still be outstanding (vector memory operations complete in order)
    static_assert(DB * 2 == 4, "the vmcnt(4) below counts the DB * 2 output stores a wave issues per unit");
    if (u == u_begin) __builtin_amdgcn_s_waitcnt(0x0070);
    else __builtin_amdgcn_s_waitcnt(0x0074);  // vmcnt(4) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    if (more) {  // Q first: a later wait for it then does not have to wait for the K / V loads behind it
      load_q(nxt, q_nxt, tok_nxt);
      kv_prepare(nxt);
      if (!late_issuer) {
#pragma unroll
        for (int i = 0; i < N_DMA; ++i) kv_issue(i, set ^ 1);
      }
    }
    __builtin_amdgcn_sched_barrier(0);

    const unsigned char* sK = smem + set * 2 * KVB;
    const unsigned char* sV = sK + KVB;
    const bool my = p.use_mask && p.sy > 0 && cur.wy == p.nWy - 1;
    const bool mx = p.use_mask && p.sx > 0 && cur.wx == p.nWx - 1;
    const WindowLogits<WS_Y, WS_X, HAS_BIAS> logits(sB, qpos, hi, my, mx, p.sy, p.sx);
    bf16x8 qf[KS];
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) qf[s2] = q_cur[s2];
    if (!p.q_prescaled) {
#pragma unroll
      for (int s2 = 0; s2 < KS; ++s2) {
        u32x4 w = __builtin_bit_cast(u32x4, q_cur[s2]);
#pragma unroll
        for (int e = 0; e < 4; ++e) w[e] = pack_bf16x2(bf16_lo(w[e]) * cq, bf16_hi(w[e]) * cq);
        qf[s2] = __builtin_bit_cast(bf16x8, w);
      }
    }
    auto load_k = [&](int kb, bf16x8 (&f)[KS]) {
#pragma unroll
      for (int s2 = 0; s2 < KS; ++s2) f[s2] = *reinterpret_cast<const bf16x8*>(sK + k_off<64>(kb * 32 + l31, s2 * 2 + hi));
    };
    const uint32_t v_addr = smem_addr + (uint32_t)(set * 2 * KVB + KVB);
    auto v_step = [&](int step) { return v_addr + (uint32_t)step * 2048u; };
    const LoadVTransposed<DB, decltype(v_step)> load_v(lane, v_step);
    auto mid = [&](int kb) {  // the late issuers' share of the next unit's loads, STAGGER_KB key blocks into this unit
      if (STAGGER_KB > 0 && kb == STAGGER_KB && late_issuer && more) {
#pragma unroll
        for (int i = 0; i < N_DMA; ++i) kv_issue(i, set ^ 1);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    f32x16 o[DB];
    float sum;
    attention_sweep<NQ, KS, DB, HAS_BIAS>(logits, load_k, load_v, mid, qf, o, sum);
    // Always DB * 2 stores per wave and unit (the wait at the top of the loop counts them); rows past the window store
    // their (recomputed, identical) last row again.  (64 bytes per row and instruction through a further
    // v_permlane16_swap, and the same for the Q loads, measured no faster.)
    store_attention_rows<DB>(p.out + (uint64_t)tok_cur * (uint32_t)inner + cur.head * HD + hi * 8, o, sum, true);
    cur = nxt;
    tok_cur = tok_nxt;
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) q_cur[s2] = q_nxt[s2];
  }
}

// ---------------------------------------------------------------------------------------------

#define AERIS_ATTN_SHAPES(X) X(8, 8, 32) X(8, 8, 64) X(12, 12, 32) X(12, 12, 64) X(16, 16, 32) X(16, 16, 64)

static int g_attn_cus = 256;  // compute units of the device (set by attention_configure_all)

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
#define CFGD(Y, Xx, Bi)                                                                                        \
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(window_attention_dma_kernel<Y, Xx, Bi>),                \
                          hipFuncAttributeMaxDynamicSharedMemorySize, AttnDmaCfg<Y, Xx, Bi>::SMEM);             \
  if (e != hipSuccess) return e;
  CFGD(8, 8, true) CFGD(8, 8, false) CFGD(12, 12, true) CFGD(12, 12, false) CFGD(16, 16, true) CFGD(16, 16, false)
#undef CFGD
#define CFGP(Y, Xx, Bi)                                                                                        \
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(window_attention_persist_kernel<Y, Xx, Bi>),            \
                          hipFuncAttributeMaxDynamicSharedMemorySize, AttnPersistCfg<Y, Xx, Bi>::SMEM);         \
  if (e != hipSuccess) return e;
  CFGP(8, 8, true) CFGP(8, 8, false) CFGP(12, 12, true) CFGP(12, 12, false) CFGP(16, 16, true) CFGP(16, 16, false)
#undef CFGP
  {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
        cus > 0)
      g_attn_cus = cus;
  }
  return hipSuccess;
}

template <int WS_Y, int WS_X, int HD, bool HAS_BIAS>
static hipError_t launch_attn(const AttnParams& p, hipStream_t stream) {
  using Cfg = AttnCfg<WS_Y, WS_X, HD, HAS_BIAS>;
  const int64_t grid = (int64_t)p.B * p.nWy * p.nWx * p.heads;
  // head_dim 64 with every offset inside a q / k / v plane below 2^32 bytes: K and V straight into LDS
  if (HD == 64 && p.head_stride >= (int64_t)p.B * p.H * p.W * p.tok_stride &&
      (int64_t)p.B * p.H * p.W * p.tok_stride * 2 < (int64_t)0xFFFFFFF0u) {
    if (grid >= 2 * (int64_t)g_attn_cus) {  // enough units for every CU to stream a few: the persistent form
      using P = AttnPersistCfg<WS_Y, WS_X, HAS_BIAS>;
      hipLaunchKernelGGL((window_attention_persist_kernel<WS_Y, WS_X, HAS_BIAS>), dim3((unsigned)g_attn_cus), dim3(P::NT), P::SMEM,
                         stream, p, (int)grid);
      return hipGetLastError();
    }
    using D = AttnDmaCfg<WS_Y, WS_X, HAS_BIAS>;
    hipLaunchKernelGGL((window_attention_dma_kernel<WS_Y, WS_X, HAS_BIAS>), dim3((unsigned)grid), dim3(D::NT), D::SMEM,
                       stream, p);
    return hipGetLastError();
  }
  hipLaunchKernelGGL((window_attention_kernel<WS_Y, WS_X, HD, HAS_BIAS>), dim3((unsigned)grid), dim3(Cfg::NT),
                     Cfg::SMEM, stream, p);
  return hipGetLastError();
}

hipError_t attention_launch(const void* qkv, void* out, const void* bias_table, int B, int H, int W, int heads,
                            int head_dim, int ws_y, int ws_x, int shift_y, int shift_x, int use_mask, float scale,
                            int q_prescaled, int64_t tok_stride, int64_t head_stride, int64_t part_stride,
                            hipStream_t stream) {
  AttnParams p;
  p.q_prescaled = q_prescaled;
  p.tok_stride = tok_stride; p.head_stride = head_stride; p.part_stride = part_stride;
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
