// Input embedding in one pass:  tokens = ([x0 / div0 | x1] + ape) W^T + b
// (src/aeris_wp_inference/model.py:346-356: cast to fp32, add the positional encoding, Linear(C -> d) in fp32;
// inference.py:160 for the [x / sigma_d | cond] form).  HBM-bound on its output: the C <= 159 input channels are
// read once, the d-wide token rows are written once, and no [M, K] operand matrix goes through memory in between.
//
// Arithmetic: bf16 MFMA at fp32 accuracy.  Inputs and weights are each split into a bf16 head and a bf16 remainder
// (hi = bf16(v), lo = bf16(v - hi)); hi*hi + lo*hi + hi*lo are accumulated in fp32, only lo*lo (2^-16 relative) is
// dropped.  The bias rides in a spare k column: the input operand holds 1 at k = C and the weight holds b[n] there.
//
// A workgroup of four waves owns 256 token rows; a wave builds the split operand of its 64 rows once, keeps it in
// registers, and then walks over all d output columns in chunks of 64.  The split weight is packed once (when the
// parameter changes) in the order the MFMA operand wants it - 16 bytes per lane, lanes consecutive, 1 KB per
// fragment - so a chunk is one contiguous piece of memory that goes to LDS by DMA (buffer_load ... lds), double
// buffered, and every fragment read is one conflict-free ds_read_b128.  With the weight fragment as first MFMA
// operand a lane ends up with 4 consecutive output columns of one row: results are stored straight from the
// accumulators, 16 bytes per lane.
#include "common.h"
#include "kernels.h"

namespace aeris {

namespace {
constexpr int IS_ROWS = 256, IS_THREADS = 256;
constexpr int IS_RB = 4;    // 16-row blocks per wave
constexpr int IS_NBC = 4;   // 16-column blocks per chunk
constexpr int IS_MAX_KB = 5;

struct InStageParams {
  const float* x0;
  const float* x1;
  const float* ape;
  const unsigned char* wp;  // [d / 16][NKB][hi, lo][64 lanes][8] bf16
  void* out;
  int64_t M, M_ape;
  int C0, C1, d;
  float div0;
};

struct PackParams {
  const float* W;     // [d, C]
  const float* bias;  // [d] or null
  unsigned char* wp;
  int d, C, NKB;
};

// one thread per 16-byte piece of the packed weight
__global__ void __launch_bounds__(256) input_pack_weight_kernel(PackParams p) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int per_nb = p.NKB * 2 * 64;
  if (t >= (int64_t)(p.d / 16) * per_nb) return;
  const int nb = (int)(t / per_nb);
  int r = (int)(t - (int64_t)nb * per_nb);
  const int kb = r / 128;
  r -= kb * 128;
  const int part = r >> 6, lane = r & 63;
  const int n = 16 * nb + (lane & 15), k0 = 32 * kb + 8 * (lane >> 4);
  float v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const int k = k0 + e;
    float w = 0.f;
    if (k < p.C) w = p.W[(int64_t)n * p.C + k];
    else if (k == p.C && p.bias) w = p.bias[n];
    const float hi = bf16_bits_to_f32(f32_to_bf16_bits(w));
    v[e] = part ? w - hi : hi;
  }
  const u32x4 o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]), pack_bf16x2(v[4], v[5]), pack_bf16x2(v[6], v[7])};
  *reinterpret_cast<u32x4*>(p.wp + t * 16) = o;
}

template <int NKB, bool OUT_F32>
__global__ void __launch_bounds__(IS_THREADS, 2) input_stage_kernel(InStageParams p) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  typedef __attribute__((address_space(3))) void* lds_ptr;
  constexpr int NB_BYTES = NKB * 2 * 1024;        // one 16-column block: NKB k-steps x (hi, lo) fragments of 1 KB
  constexpr int CHUNK_BYTES = IS_NBC * NB_BYTES;  // 64 columns
  constexpr int DMA_PER_WAVE = CHUNK_BYTES / 1024 / 4;
  constexpr int ESZ = OUT_F32 ? 4 : 2;

  const int tid = threadIdx.x, lane = tid & 63, l15 = lane & 15, q = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int64_t m0 = (int64_t)blockIdx.x * IS_ROWS + wave * (16 * IS_RB);
  const int d = p.d, NCH = d / (16 * IS_NBC);
  const int C0 = p.C0, C = p.C0 + p.C1;

  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.wp, 0, (int)((int64_t)(d / 16) * NB_BYTES), 0x00020000);
  auto issue_dma = [&](int c, int stage) {
    unsigned char* const dst = smem + stage * CHUNK_BYTES + wave * (DMA_PER_WAVE * 1024);
    const uint32_t src = (uint32_t)c * CHUNK_BYTES + (uint32_t)wave * (DMA_PER_WAVE * 1024);
#pragma unroll
    for (int i = 0; i < DMA_PER_WAVE; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(dst + i * 1024), 16, (uint32_t)lane * 16, src + i * 1024, 0, 0);
  };
  issue_dma(0, 0);

  // ---- the wave's operand: 4 row blocks x NKB k-steps, split into head and remainder, kept in registers.
  // A row block is read column-wise (lane = channel, row pointers wave-uniform: coalesced loads), summed with the
  // positional encoding, and turned into the row-wise fragment order through a wave-private 16 x (32 NKB) f32 tile in
  // the second weight buffer, which is idle until the first chunk has been consumed.  16-byte pieces of a row are
  // XOR-swizzled with the row number so that the fragment reads (16 rows x 16 bytes per quarter wave) do not collide.
  bf16x8 a_hi[IS_RB][NKB], a_lo[IS_RB][NKB];
  unsigned char* orow[IS_RB];
  constexpr int KP = 32 * NKB;             // padded channel count
  constexpr int NG = (KP + 63) / 64;       // column groups of 64 lanes
  float* const tile = reinterpret_cast<float*>(smem + CHUNK_BYTES + wave * (CHUNK_BYTES / 4));
  const int64_t last_row = p.M - 1;
  const int64_t m0c = m0 < last_row ? m0 : last_row;
  const int nvalid = (int)(p.M - m0c < 16 * IS_RB ? p.M - m0c : 16 * IS_RB);  // >= 1
  // the wave's 64 rows wrap around the positional encoding at most once: 64 <= M_ape < 2^31 (checked by the host)
  const int ape_row0 = (int)(m0c % p.M_ape), ape_rows = (int)p.M_ape;
  // null pointers are resolved once, here, into valid bases with strides and masks that make them inert: the
  // per-row code below has no branches, so that the loads of eight rows are in flight together
  const float* const x0b = p.x0 + m0c * C0;
  const float* const x1b = p.x1 ? p.x1 + m0c * p.C1 - C0 : x0b;
  const int x1_stride = p.x1 ? p.C1 : C0;
  const float* const apeb = p.ape ? p.ape : p.x0;
  const int ape_stride = p.ape ? C : 0, ape_kmask = p.ape ? -1 : 0;
  const bool has_ape = p.ape != nullptr;  // wave-uniform
  const float inv_div = 1.0f / p.div0;
#pragma unroll
  for (int rb = 0; rb < IS_RB; ++rb) {
    {
      // Rows below the matrix recompute its last row and store it again (same bits to the same address): every
      // wave then issues the same number of stores per chunk, which the wait at the end of a chunk counts on.
      const int roff = min(rb * 16 + l15, nvalid - 1);
      orow[rb] = reinterpret_cast<unsigned char*>(p.out) + ((m0c + roff) * d + 4 * q) * ESZ;
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {  // eight rows' loads in flight at a time
      float val[8][NG];
#pragma unroll
      for (int rr = 0; rr < 8; ++rr) {
        const int roff = min(rb * 16 + half * 8 + rr, nvalid - 1);  // wave-uniform
        const float* const b0 = x0b + roff * C0;
        const float* const b1 = x1b + roff * x1_stride;
        int arow = ape_row0 + roff;
        arow -= arow >= ape_rows ? ape_rows : 0;
        const float* const ba = apeb + (int64_t)arow * ape_stride;
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const int k = 64 * g + lane;
          const int kc = k < C ? k : C - 1;
          const bool first = kc < C0;
          const float* const src = first ? b0 : b1;
          const float x = src[kc];
          const float a = ba[kc & ape_kmask];
          // x / div0 for the state channels: quotient by reciprocal with one correction step
          float quo = x * inv_div;
          quo = fmaf(fmaf(-quo, p.div0, x), inv_div, quo);
          // without a positional encoding `a` is a stand-in read from the input itself: a select, not a multiply
          // by zero, keeps an Inf or NaN there out of every other token
          const float base = first ? quo : x;
          const float v = has_ape ? a + base : base;
          val[rr][g] = k < C ? v : (k == C ? 1.0f : 0.0f);
        }
      }
#pragma unroll
      for (int rr = 0; rr < 8; ++rr)
#pragma unroll
        for (int g = 0; g < NG; ++g) {
          const int k = 64 * g + lane, r = half * 8 + rr;
          if (k < KP) tile[r * KP + ((((k >> 2) ^ (r & 7)) << 2) | (k & 3))] = val[rr][g];
        }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int kb = 0; kb < NKB; ++kb) {
      const int c4 = 8 * kb + 2 * q;  // 16-byte piece of the lane's 8 channels
      const f32x4 v0 = *reinterpret_cast<const f32x4*>(tile + l15 * KP + ((c4 ^ (l15 & 7)) << 2));
      const f32x4 v1 = *reinterpret_cast<const f32x4*>(tile + l15 * KP + (((c4 + 1) ^ (l15 & 7)) << 2));
      uint32_t hi[4], lo[4];
      hi[0] = pack_bf16x2(v0[0], v0[1]); lo[0] = pack_bf16x2(v0[0] - bf16_lo(hi[0]), v0[1] - bf16_hi(hi[0]));
      hi[1] = pack_bf16x2(v0[2], v0[3]); lo[1] = pack_bf16x2(v0[2] - bf16_lo(hi[1]), v0[3] - bf16_hi(hi[1]));
      hi[2] = pack_bf16x2(v1[0], v1[1]); lo[2] = pack_bf16x2(v1[0] - bf16_lo(hi[2]), v1[1] - bf16_hi(hi[2]));
      hi[3] = pack_bf16x2(v1[2], v1[3]); lo[3] = pack_bf16x2(v1[2] - bf16_lo(hi[3]), v1[3] - bf16_hi(hi[3]));
      a_hi[rb][kb] = __builtin_bit_cast(bf16x8, u32x4{hi[0], hi[1], hi[2], hi[3]});
      a_lo[rb][kb] = __builtin_bit_cast(bf16x8, u32x4{lo[0], lo[1], lo[2], lo[3]});
    }
    __builtin_amdgcn_wave_barrier();
  }
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): chunk 0 has landed
  __syncthreads();

  for (int c = 0; c < NCH; ++c) {
    __builtin_amdgcn_sched_barrier(0);
    if (c + 1 < NCH) issue_dma(c + 1, (c + 1) & 1);
    __builtin_amdgcn_sched_barrier(0);
    const unsigned char* const ws = smem + (c & 1) * CHUNK_BYTES + lane * 16;
#pragma unroll
    for (int nb = 0; nb < IS_NBC; ++nb) {
      f32x4 acc[IS_RB];
#pragma unroll
      for (int rb = 0; rb < IS_RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        const bf16x8 w_hi = *reinterpret_cast<const bf16x8*>(ws + nb * NB_BYTES + (kb * 2 + 0) * 1024);
        const bf16x8 w_lo = *reinterpret_cast<const bf16x8*>(ws + nb * NB_BYTES + (kb * 2 + 1) * 1024);
        // weight fragment first: a lane ends up with 4 consecutive output columns of one row
#pragma unroll
        for (int rb = 0; rb < IS_RB; ++rb) acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_hi, a_hi[rb][kb], acc[rb], 0, 0, 0);
#pragma unroll
        for (int rb = 0; rb < IS_RB; ++rb) acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_hi, a_lo[rb][kb], acc[rb], 0, 0, 0);
#pragma unroll
        for (int rb = 0; rb < IS_RB; ++rb) acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_lo, a_hi[rb][kb], acc[rb], 0, 0, 0);
      }
      const int col_off = (c * (16 * IS_NBC) + nb * 16) * ESZ;
#pragma unroll
      for (int rb = 0; rb < IS_RB; ++rb) {
        if (OUT_F32) {
          *reinterpret_cast<f32x4*>(orow[rb] + col_off) = acc[rb];
        } else {
          const u32x2 o = {pack_bf16x2(acc[rb][0], acc[rb][1]), pack_bf16x2(acc[rb][2], acc[rb][3])};
          *reinterpret_cast<u32x2*>(orow[rb] + col_off) = o;
        }
      }
    }
    // The DMA loads of the next chunk were issued ahead of this chunk's 16 stores and vector memory operations
    // complete in order: "all but the newest 16" is exactly those loads, without waiting for any store.
    static_assert(IS_NBC * IS_RB == 16, "the vmcnt(16) below counts one store per 16-column block and 16-row block");
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_waitcnt(0x4F70);  // vmcnt(16)
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  }
}

template <int NKB>
hipError_t launch_main(const InStageParams& p, bool out_f32, hipStream_t stream) {
  const dim3 grid((unsigned)((p.M + IS_ROWS - 1) / IS_ROWS)), block(IS_THREADS);
  const size_t lds = 2 * (size_t)IS_NBC * NKB * 2 * 1024;
  if (out_f32) hipLaunchKernelGGL((input_stage_kernel<NKB, true>), grid, block, lds, stream, p);
  else hipLaunchKernelGGL((input_stage_kernel<NKB, false>), grid, block, lds, stream, p);
  return hipGetLastError();
}

template <int NKB>
hipError_t configure_one() {
  const int lds = 2 * IS_NBC * NKB * 2 * 1024;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&input_stage_kernel<NKB, true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, lds);
  if (e != hipSuccess) return e;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(&input_stage_kernel<NKB, false>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, lds);
}
}  // namespace

// k-steps of 32 that hold C input channels plus the bias column
static int input_stage_ksteps(int C) { return (C + 1 + 31) / 32; }

bool input_stage_supported(int C, int d) { return C >= 1 && input_stage_ksteps(C) <= IS_MAX_KB && d >= 64 && d % 64 == 0; }

int64_t input_stage_weight_bytes(int C, int d) { return (int64_t)(d / 16) * input_stage_ksteps(C) * 2 * 1024; }

hipError_t input_stage_configure() {
  hipError_t e = configure_one<1>();
  if (e == hipSuccess) e = configure_one<2>();
  if (e == hipSuccess) e = configure_one<3>();
  if (e == hipSuccess) e = configure_one<4>();
  if (e == hipSuccess) e = configure_one<5>();
  return e;
}

hipError_t input_stage_pack_weight_launch(const float* W, const float* bias, void* packed, int C, int d, hipStream_t stream) {
  PackParams p;
  p.W = W; p.bias = bias; p.wp = reinterpret_cast<unsigned char*>(packed); p.d = d; p.C = C; p.NKB = input_stage_ksteps(C);
  const int64_t pieces = (int64_t)(d / 16) * p.NKB * 2 * 64;
  hipLaunchKernelGGL(input_pack_weight_kernel, dim3((unsigned)((pieces + 255) / 256)), dim3(256), 0, stream, p);
  return hipGetLastError();
}

hipError_t input_stage_launch(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape, int64_t M_ape,
                              const void* packed, void* out, int out_dtype, int64_t M, int d, hipStream_t stream) {
  InStageParams p;
  p.x0 = x0; p.x1 = x1; p.ape = ape; p.wp = reinterpret_cast<const unsigned char*>(packed); p.out = out;
  p.M = M; p.M_ape = M_ape > 0 ? M_ape : 1; p.C0 = C0; p.C1 = x1 ? C1 : 0; p.d = d; p.div0 = div0;
  const bool f32 = out_dtype == AERIS_F32;
  switch (input_stage_ksteps(p.C0 + p.C1)) {
    case 1: return launch_main<1>(p, f32, stream);
    case 2: return launch_main<2>(p, f32, stream);
    case 3: return launch_main<3>(p, f32, stream);
    case 4: return launch_main<4>(p, f32, stream);
    default: return launch_main<5>(p, f32, stream);
  }
}

}  // namespace aeris
