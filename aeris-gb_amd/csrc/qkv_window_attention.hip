// to_qkv projection and window attention in ONE kernel for gfx950: q, k and v never exist in HBM.
//
// One unit of work = one (window, head): the 256 token rows of a 16 x 16 window (gathered through the folded
// partition / shift index map: the A operand of a GEMM may come in any row order) times the head's 192 rows of the
// to_qkv weight (64 of q, 64 of k, 64 of v) over all of K - a 256 x 192 x K GEMM with the persistent GEMM's main loop
// (k-tiles of 64, operands straight into LDS by buffer_load ... lds, two stages of A and three of W, the two waves of
// a SIMD alternating memory and compute slots) - and then, in place of a GEMM epilogue, attention on the tile:
// bias added and q multiplied by scale * log2(e) in fp32, q / k / v rounded to bf16 once and written to LDS in the
// layouts of the one-window attention kernels, every wave takes its 32 queries' fragments, and the shared sweep
// (attention_sweep.h) runs from LDS; the output rows go to their folded token rows.  Per output element the GEMM does
// exactly the work of the separate to_qkv GEMM (every (token, head) belongs to one unit), its 128 KB-per-tile epilogue
// and the attention kernel's 96 KB of loads per unit are gone, and so are 9.6 + 9.6 GB of HBM traffic per block at
// the 720 x 1440 x 24 x 64 shape.
//
// LDS (160 KB):   A0 32 K | A1 32 K | W0 24 K | W1 24 K | W2 24 K | bias 16 K | spare 8 K
//   main loop     k-tile j reads A stage j % 2 and W stage j % 3 (j counts k-tiles over the workgroup's whole unit
//                 list: the next unit's first k-tiles are in flight while the current unit is attended to)
//   attention     K / K^T fragments come from the A stage and V from the W stage that the unit's LAST k-tile used (both
//                 are idle until the next unit's second / third k-tile), V's last 64 rows from the spare 8 K; Q passes
//                 through the other A stage, whose refill (the next unit's first k-tile of A) is issued once every
//                 wave has its Q fragments.  K must be even for that (the last k-tile then uses A1).
//   bias          the head's relative-position bias as fp32 4-vectors (WindowLogits), prepared once per parameter value
//                 by qkv_attention_bias_kernel, brought in by the load unit during the main loop
// Units are walked in groups of 4 windows x all heads, so that a window's token rows and a head's weight rows are
// shared in one XCD's L2; the groups are dealt to the 8 XCDs in turn (group g to XCD g % 8) and the units of an XCD's
// groups to its workgroups in turn, which spreads the windows on the wrapped border of a shifted grid - a whole
// window row, slower than the others by their mask arithmetic - evenly over XCDs and workgroups.
#include "common.h"
#include "attention_sweep.h"
#include "gemm_common.h"
#include "kernels.h"
#include <type_traits>

namespace aeris {

namespace {
constexpr int QA_WS = 16, QA_L = 256, QA_HD = 64;
constexpr int QA_BM = 256, QA_BN = 192, QA_BK = 64, QA_WM = 2, QA_WN = 4;
constexpr int QA_NT = QA_WM * QA_WN * 64;            // 512 threads: also one wave per 32-query group
constexpr int QA_FM = QA_BM / QA_WM / 16;            // 8 row fragments per wave
constexpr int QA_FN = QA_BN / QA_WN / 16;            // 3 column fragments per wave
constexpr int QA_A_BYTES = QA_BM * QA_BK * 2;        // 32 KB
constexpr int QA_W_BYTES = QA_BN * QA_BK * 2;        // 24 KB
constexpr int QA_W_OFF = 2 * QA_A_BYTES;
constexpr int QA_BIAS_OFF = QA_W_OFF + 3 * QA_W_BYTES;
constexpr int QA_TBL = (2 * QA_WS - 1) * (2 * QA_WS - 1);
constexpr int QA_BIAS_BYTES = 16384;                 // 961 x 16 B = 15 376, rounded up to whole 1 KB load instructions
constexpr int QA_SPARE_OFF = QA_BIAS_OFF + QA_BIAS_BYTES;
constexpr int QA_SMEM = QA_SPARE_OFF + 8192;         // 160 KB
constexpr int QA_GM = 4;                             // windows per L2 group
static_assert(QA_SMEM == 160 * 1024, "the layout fills the CU's LDS exactly");
static_assert(QA_TBL * 16 <= QA_BIAS_BYTES, "bias table fits its slot");

struct QkvAttnParams {
  const uint16_t* y;      // [B * H * W, K] bf16, natural token order
  const uint16_t* w;      // [3 * heads * 64, K] bf16, rows ordered (c h d)
  const uint16_t* bias;   // [3 * heads * 64] bf16 or null
  const float* bias4;     // [heads][QA_TBL][4] f32 (qkv_attention_bias_kernel) or null
  uint16_t* out;          // [B * H * W, heads * 64] bf16
  int B, H, W, heads, K;
  int nWy, nWx;
  int sy, sx;
  int use_mask;
  float q_scale;          // softmax scale times log2(e)
  int n_win, bpx;         // windows (B * nWy * nWx); workgroups per XCD
  // ceil(2^40 / d) for d = units per group, windows per image, windows per row: n / d = (n * m) >> 40 for n < 2^24.
  // A unit is decoded several times per unit and wave; as true divisions that was 40 % of the kernel's vector ALU work.
  uint64_t m_gsz, m_wpi, m_nwx;
};
__device__ __forceinline__ int div_by_magic(int n, uint64_t m) { return (int)(((uint64_t)(uint32_t)n * m) >> 40); }
}  // namespace

// R4[head][s][e] = table[TBL - 1 - (s + e)][head] * log2(e) for s + e < TBL, else 0: the layout WindowLogits reads
__global__ void qkv_attention_bias_kernel(const uint16_t* table, float* out, int heads) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= heads * QA_TBL * 4) return;
  const int e = idx & 3, s = (idx >> 2) % QA_TBL, head = idx / (4 * QA_TBL);
  const int j = s + e;
  out[idx] = j < QA_TBL ? bf16_bits_to_f32(table[(int64_t)(QA_TBL - 1 - j) * heads + head]) * 1.4426950408889634f : 0.f;
}

template <bool HAS_BIAS>
__global__ void __launch_bounds__(QA_NT) qkv_window_attention_kernel(QkvAttnParams p) {
  constexpr int KS = 4, DB = 2, NQ = 8;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  typedef __attribute__((address_space(3))) bf16x4_t* lds_bf16x4_ptr;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_u = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave_u / QA_WN, wn = wave_u % QA_WN, grp = wm;
  const int l15 = lane & 15, q4 = lane >> 4;
  const int K = p.K, KT = K / QA_BK;
  const int H = p.H, W = p.W;
  const int inner = p.heads * QA_HD;

  // ---- this workgroup's unit list: XCD x (workgroup id & 7: consecutive workgroups go to consecutive XCDs) owns the
  // groups x, x + 8, ...; its workgroup `slot` takes the units slot, slot + bpx, ... of those groups laid end to end.
  // Only the very last group can be short (fewer than QA_GM windows) and it ends its XCD's sequence.
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int gsz = QA_GM * p.heads;
  const int n_groups = (p.n_win + QA_GM - 1) / QA_GM;
  const int my_groups = n_groups > xcd ? (n_groups - xcd + 7) / 8 : 0;
  int seq_len = my_groups * gsz;
  if (my_groups > 0 && (my_groups - 1) * 8 + xcd == n_groups - 1) seq_len -= (n_groups * QA_GM - p.n_win) * p.heads;
  const int n_my = seq_len > slot ? (seq_len - slot + p.bpx - 1) / p.bpx : 0;
  if (n_my == 0) return;
  struct Unit { int head, b, wy, wx; };
  auto decode = [&](int r) {
    const int t = r * p.bpx + slot;
    const int lg = div_by_magic(t, p.m_gsz), within = t - lg * gsz;
    const int g = lg * 8 + xcd;
    int gm = p.n_win - g * QA_GM;
    if (gm > QA_GM) gm = QA_GM;
    Unit u;
    static_assert(QA_GM == 4, "the shift below");
    u.head = gm == QA_GM ? within >> 2 : within / gm;  // only the very last group can be short
    const int win = g * QA_GM + (within - u.head * gm);
    const int wpi = p.nWy * p.nWx;
    u.b = div_by_magic(win, p.m_wpi);
    const int wrem = win - u.b * wpi;
    u.wy = div_by_magic(wrem, p.m_nwx);
    u.wx = wrem - u.wy * p.nWx;
    return u;
  };
  auto window_wraps = [&](const Unit& un) { return (un.wy + 1) * QA_WS + p.sy > H || (un.wx + 1) * QA_WS + p.sx > W; };
  auto window_base = [&](const Unit& un) -> uint32_t {  // first token of the window inside its batch entry
    return (uint32_t)(un.wy * QA_WS + p.sy) * (uint32_t)W + (uint32_t)(un.wx * QA_WS + p.sx);
  };
  auto token_in_image = [&](const Unit& un, int pos) -> uint32_t {  // general form, used on the wrapped border only
    int Y = un.wy * QA_WS + p.sy + pos / QA_WS;
    int X = un.wx * QA_WS + p.sx + pos % QA_WS;
    if (Y >= H) Y -= H;
    if (X >= W) X -= W;
    return (uint32_t)Y * (uint32_t)W + (uint32_t)X;
  };

  // ---- loaders.  One buffer_load ... lds of a wave fills 1 KB = 8 rows of the swizzled tile layout (swz_off); lane l
  // fetches the 16-byte chunk which that layout keeps at LDS byte 16 l.  A: a wave brings in the 32 window positions
  // [32 wave, 32 wave + 32) = two window rows, 4 instructions; the row of a lane is a token row of the folded index
  // map, so its source offset is (token relative to the window's first token) * K * 2 plus the chunk: per-lane
  // constants, except in windows on the wrapped border.  W: a wave brings in 24 of the head's 192 weight rows
  // (tile rows [0, 64) = q, [64, 128) = k, [128, 192) = v of the head), 3 instructions.
  const uint32_t rowb = (uint32_t)K * 2u;
  uint32_t w_voff[2];  // W: lane part of the source offset for even / odd 8-row blocks
  {
    const int dr = lane >> 4, pos = lane & 15;
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      const int logical = pos ^ (par * 4 + dr);
      w_voff[par] = (uint32_t)(dr * 2 + (logical >> 3)) * rowb + (uint32_t)((logical & 7) * 16);
    }
  }
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.w, 0, (int)((int64_t)3 * inner * K * 2), 0x00020000);
  const uint32_t img_bytes = (uint32_t)(H * W) * rowb;  // < 2^32, checked by the caller
  __amdgpu_buffer_rsrc_t rs_a = rs_w;
  int la_r = 0, la_kt = 0, la_stage = 0;  // A stream over (unit, k-tile)
  uint32_t la_base = 0;                   // byte offset of the unit's first token row
  uint32_t la_voff[4];
  auto la_set_unit = [&]() {
    if (la_r >= n_my) return;
    const Unit un = decode(la_r);
    rs_a = __builtin_amdgcn_make_buffer_rsrc((void*)(p.y + (int64_t)un.b * H * W * K), 0, (int)img_bytes, 0x00020000);
    // what a lane's rows are follows from the lane number alone; derived anew per unit from a laundered copy of it, so
    // that none of it occupies registers across the main loop and the attention sweep
    int lane_t = lane;
    asm volatile("" : "+v"(lane_t));
    const int dr = lane_t >> 4, pos = lane_t & 15;
    const bool wraps = window_wraps(un);  // workgroup-uniform
    la_base = wraps ? 0u : window_base(un) * rowb;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int logical = pos ^ ((i & 1) * 4 + dr);
      const int a_pos = wave_u * 32 + i * 8 + dr * 2 + (logical >> 3);  // window position of the lane's row in instruction i
      const uint32_t tok = wraps ? token_in_image(un, a_pos) : (uint32_t)((a_pos / QA_WS) * W + a_pos % QA_WS);
      la_voff[i] = tok * rowb + (uint32_t)((logical & 7) * 16);
    }
  };
  auto issue_a = [&]() {
    if (la_r < n_my) {
      unsigned char* sd = smem + la_stage * QA_A_BYTES + wave_u * 4096;
      const uint32_t so = la_base + (uint32_t)la_kt * (QA_BK * 2);
#pragma unroll
      for (int i = 0; i < 4; ++i) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(sd + i * 1024), 16, la_voff[i], so, 0, 0);
      la_stage ^= 1;
      ++la_kt;
    }
  };
  auto la_next_unit = [&]() {  // the stream has issued all k-tiles of its unit: on to the next one
    la_kt = 0;
    ++la_r;
    la_set_unit();
  };
  // the same inside a unit (k-tiles 1 .. KT - 1 of the unit the stream is in): no end-of-list or end-of-unit decisions
  auto issue_a_same_unit = [&]() {
    unsigned char* sd = smem + la_stage * QA_A_BYTES + wave_u * 4096;
    const uint32_t so = la_base + (uint32_t)la_kt * (QA_BK * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i) __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(sd + i * 1024), 16, la_voff[i], so, 0, 0);
    la_stage ^= 1;
    ++la_kt;
  };
  int lw_r = 0, lw_kt = 0, lw_stage = 0;  // W stream
  uint32_t lw_row[3];                     // W row of the first row of each of this wave's three 8-row blocks
  auto lw_set_unit = [&]() {
    if (lw_r >= n_my) return;
    const Unit un = decode(lw_r);
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      const int t = wave_u * 24 + i * 8;  // tile row; 8-row blocks never straddle the q / k / v parts
      lw_row[i] = (uint32_t)((t >> 6) * inner + un.head * QA_HD + (t & 63));
    }
  };
  auto issue_w = [&]() {
    if (lw_r < n_my) {
      unsigned char* sd = smem + QA_W_OFF + lw_stage * QA_W_BYTES + wave_u * 3072;
      const uint32_t kb = (uint32_t)lw_kt * (QA_BK * 2);
#pragma unroll
      for (int i = 0; i < 3; ++i)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(sd + i * 1024), 16, w_voff[(wave_u * 3 + i) & 1],
                                                 lw_row[i] * rowb + kb, 0, 0);
      lw_stage = lw_stage == 2 ? 0 : lw_stage + 1;
      ++lw_kt;
    }
  };
  auto lw_next_unit = [&]() {
    lw_kt = 0;
    ++lw_r;
    lw_set_unit();
  };
  auto issue_w_same_unit = [&]() {
    unsigned char* sd = smem + QA_W_OFF + lw_stage * QA_W_BYTES + wave_u * 3072;
    const uint32_t kb = (uint32_t)lw_kt * (QA_BK * 2);
#pragma unroll
    for (int i = 0; i < 3; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_w, (lds_ptr)(sd + i * 1024), 16, w_voff[(wave_u * 3 + i) & 1],
                                               lw_row[i] * rowb + kb, 0, 0);
    lw_stage = lw_stage == 2 ? 0 : lw_stage + 1;
    ++lw_kt;
  };
  // the head's bias 4-vectors -> LDS: 16 load instructions of 1 KB, two per wave (the last one ends outside the
  // descriptor: zeros)
  auto issue_bias = [&](int head) {
    if (HAS_BIAS) {
      const __amdgpu_buffer_rsrc_t rs_b = __builtin_amdgcn_make_buffer_rsrc(
          (void*)(p.bias4 + (int64_t)head * QA_TBL * 4), 0, QA_TBL * 16, 0x00020000);
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int blk = wave_u * 2 + i;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_b, (lds_ptr)(smem + QA_BIAS_OFF + blk * 1024), 16, (uint32_t)(lane * 16),
                                                 (uint32_t)(blk * 1024), 0, 0);
      }
    }
  };

  // ---- fragment read offsets of the GEMM (per k-step of 32), relative to a stage
  uint32_t a_roff[2], b_roff[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    a_roff[ks] = swz_off(wm * (QA_BM / QA_WM) + l15, ks * 4 + q4);
    b_roff[ks] = swz_off(wn * (QA_BN / QA_WN) + l15, ks * 4 + q4);
  }

  // ---- accumulators start at the projection's bias.  Column fragment j of wave (wm, wn) holds the tile columns
  // 48 wn + 16 j + 4 q4 + (0..3): part c = column / 64 (q, k, v), d = column % 64
  f32x4 acc[QA_FM][QA_FN];
  auto load_bias = [&](int r, u32x2 (&bq)[QA_FN]) {
    const Unit un = decode(r);
#pragma unroll
    for (int j = 0; j < QA_FN; ++j) {
      const int col = wn * 48 + j * 16 + q4 * 4;
      bq[j] = u32x2{0u, 0u};
      if (p.bias) bq[j] = *reinterpret_cast<const u32x2*>(p.bias + (col >> 6) * inner + un.head * QA_HD + (col & 63));
    }
  };
  auto init_acc = [&](const u32x2 (&bq)[QA_FN]) {
#pragma unroll
    for (int j = 0; j < QA_FN; ++j) {
      const f32x4 b = {bf16_lo(bq[j].x), bf16_hi(bq[j].x), bf16_lo(bq[j].y), bf16_hi(bq[j].y)};
#pragma unroll
      for (int i = 0; i < QA_FM; ++i) acc[i][j] = b;
    }
  };
  {
    u32x2 bq[QA_FN];
    load_bias(0, bq);
    init_acc(bq);
  }

  // s_waitcnt immediates: vmcnt in bits 3:0 (and 15:14), expcnt in 6:4 (7 = no wait), lgkmcnt in 11:8 (15 = no wait)
  constexpr int WAIT_LGKM0 = 0xC07F, WAIT_VM0 = 0x0F70, WAIT_VM3 = 0x0F73, WAIT_VM5 = 0x0F75, WAIT_VM3_LGKM0 = 0x0073,
                WAIT_VM7_LGKM0 = 0x0077, WAIT_VM9_LGKM0 = 0x0079, WAIT_VM4_LGKM0 = 0x0074, WAIT_ALL = 0x0070;

  // ---- attention on the finished tile (in place of a GEMM epilogue)
  auto attend = [&](int r_done, int sw_last) {
    const Unit un = decode(r_done);
    // per-lane constants of this phase, from a laundered copy of the lane number (see la_set_unit).  A wave is a query
    // group: its 32 queries are the window positions 32 wave + l31.
    int lane_t = lane;
    asm volatile("" : "+v"(lane_t));
    const int l15 = lane_t & 15, q4 = lane_t >> 4, l31 = lane_t & 31, hi = lane_t >> 5;
    const int qpos = wave_u * 32 + l31;
    const uint32_t q_rel = (uint32_t)((qpos / QA_WS) * W + qpos % QA_WS);
#if defined(QA_LAB) && QA_LAB == 2
    {  // timing only: the main loop alone (the accumulators are folded into one store so that they stay live)
      f32x4 t = {0.f, 0.f, 0.f, 0.f};
      for (int i = 0; i < QA_FM; ++i) for (int j = 0; j < QA_FN; ++j) t += acc[i][j];
      issue_a();
      *reinterpret_cast<f32x4*>(p.out + ((uint64_t)un.b * (uint32_t)(H * W) + window_base(un) + q_rel) * (uint32_t)inner + un.head * QA_HD + hi * 8) = t;
      u32x2 bq0[QA_FN];
      for (int j = 0; j < QA_FN; ++j) bq0[j] = u32x2{0u, 0u};
      init_acc(bq0);
      __builtin_amdgcn_s_waitcnt(WAIT_ALL);
      __builtin_amdgcn_s_barrier();
      return;
    }
#endif
    unsigned char* const sQ = smem;                                   // A0: idle, its refill is issued below
    unsigned char* const sK = smem + QA_A_BYTES;                      // A1: the last k-tile's stage
    unsigned char* const sV0 = smem + QA_W_OFF + sw_last * QA_W_BYTES;  // the last k-tile's W stage: V rows 0..191
    unsigned char* const sV1 = smem + QA_SPARE_OFF;                   // V rows 192..255
    // 1. q (times scale * log2 e), k, v -> bf16 -> LDS.  A lane holds 4 consecutive d of one token per fragment: half
    // of a 16-byte chunk of the token's row; Q and K rows are chunk-swizzled by (row >> 1) & 7, V rows by 2 (row & 3).
    // The position of row fragment i is that of fragment 0 plus 16 i, which leaves both swizzles as they are: the
    // address of fragment i is the address of fragment 0 plus 2048 i, an immediate offset of the write, so a column
    // fragment needs one address (written out per fragment, the address arithmetic was nine tenths of this phase).
    // V rows 192..255 live in the spare area: for the upper wave group that is the fragments i >= 4.
    {
      const int row0 = wm * (QA_BM / QA_WM) + l15;
      const uint32_t qk_row = (uint32_t)(row0 >> 1) * 256u, qk_hi = (uint32_t)((row0 & 1) << 3), qk_sw = (uint32_t)((row0 >> 1) & 7);
      const uint32_t v_row = (uint32_t)row0 * 128u, v_sw = (uint32_t)(2 * (row0 & 3));
#pragma unroll
      for (int j = 0; j < QA_FN; ++j) {
        const int col = wn * 48 + j * 16;       // wave-uniform: first tile column of the fragment
        const int part = col >> 6, d0 = (col & 63) + q4 * 4;
        const uint32_t chunk = (uint32_t)(d0 >> 3), half8 = (uint32_t)(((d0 >> 2) & 1) * 8);
        const float sc = part == 0 ? p.q_scale : 1.0f;  // a scalar: times 1 is exact, and cheaper than selecting per value
        unsigned char *dst_lo, *dst_hi;  // fragment i goes to (i < 4 ? dst_lo : dst_hi) + 2048 i
        if (part == 2) {
          const uint32_t a = v_row + ((chunk ^ v_sw) << 4) + half8;
          dst_lo = sV0 + a;
          dst_hi = wm == 0 ? dst_lo : sV1 + a - 192 * 128;
        } else {
          dst_lo = dst_hi = (part == 0 ? sQ : sK) + qk_row + (((qk_hi | chunk) ^ qk_sw) << 4) + half8;
        }
#pragma unroll
        for (int i = 0; i < QA_FM; ++i) {
          const f32x4 v = acc[i][j] * sc;
          *reinterpret_cast<u32x2*>((i < QA_FM / 2 ? dst_lo : dst_hi) + i * 2048) = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        }
      }
    }
    __builtin_amdgcn_s_waitcnt(WAIT_LGKM0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
    // 2. this wave's Q fragments (B operand: lane = query, 8 consecutive d per k16 step)
    bf16x8 qf[KS];
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) {
      const int row = wave_u * 32 + l31, chunk = s2 * 2 + hi;
      qf[s2] = *reinterpret_cast<const bf16x8*>(sQ + (row >> 1) * 256 + (((((row & 1) << 3) | chunk) ^ ((row >> 1) & 7)) << 4));
    }
    __builtin_amdgcn_s_waitcnt(WAIT_LGKM0);
    __builtin_amdgcn_sched_barrier(0);
    // This wave has its Q, and the 4 KB of A0 that its own loads fill are exactly the 16 position pairs it has just read
    // (positions 32 wave .. 32 wave + 31, read by no other wave): it refills them with its rows of the next unit's first
    // k-tile (held back in the main loop) without waiting for the other waves.
    la_next_unit();
    issue_a();
    __builtin_amdgcn_sched_barrier(0);
    // 3. the sweep
    // (wave-uniform, and said so: the mask arithmetic must stay behind a scalar branch that all but the border windows skip)
#ifdef QA_LAB_MASK_EVERY  // timing experiment: every QA_LAB_MASK_EVERY-th unit of a workgroup takes the mask path
    const bool my = __builtin_amdgcn_readfirstlane((int)(p.use_mask && (r_done % QA_LAB_MASK_EVERY) == 0)) != 0;
    const bool mx = false;
#else
    const bool my = __builtin_amdgcn_readfirstlane((int)(p.use_mask && p.sy > 0 && un.wy == p.nWy - 1)) != 0;
    const bool mx = __builtin_amdgcn_readfirstlane((int)(p.use_mask && p.sx > 0 && un.wx == p.nWx - 1)) != 0;
#endif
    const WindowLogits<QA_WS, QA_WS, HAS_BIAS> logits(smem + QA_BIAS_OFF, qpos, hi, my, mx, p.sy, p.sx);
    auto load_k = [&](int kb, bf16x8 (&f)[KS]) {
#pragma unroll
      for (int s2 = 0; s2 < KS; ++s2) {
        const int row = kb * 32 + l31, chunk = s2 * 2 + hi;
        f[s2] = *reinterpret_cast<const bf16x8*>(sK + (row >> 1) * 256 + (((((row & 1) << 3) | chunk) ^ ((row >> 1) & 7)) << 4));
      }
    };
    const uint32_t v0_addr = lds_byte_address(sV0), v1_addr = lds_byte_address(sV1);
    auto v_step = [&](int step) {  // step = 16 keys = 2 KB of V rows
      return step < 12 ? v0_addr + (uint32_t)step * 2048u : v1_addr + (uint32_t)(step - 12) * 2048u;
    };
    const LoadVTransposed<DB, decltype(v_step)> load_v(lane_t, v_step);
    f32x16 o[DB];
    float sum;
#if defined(QA_LAB) && QA_LAB >= 1
    sum = 1.f;
    for (int db = 0; db < DB; ++db) for (int e = 0; e < 16; ++e) o[db][e] = __builtin_bit_cast(float, __builtin_bit_cast(u32x4, qf[e & 3])[db]);
#else
    attention_sweep<NQ, KS, DB, HAS_BIAS>(logits, load_k, load_v, [](int) {}, qf, o, sum);
#endif
    const uint32_t tok = (uint32_t)un.b * (uint32_t)(H * W) + (window_wraps(un) ? token_in_image(un, qpos) : window_base(un) + q_rel);
    // the next unit's projection bias: requested ahead of the output stores (vector memory operations complete in order)
    u32x2 bq_next[QA_FN];
#pragma unroll
    for (int j = 0; j < QA_FN; ++j) bq_next[j] = u32x2{0u, 0u};
    if (r_done + 1 < n_my) load_bias(r_done + 1, bq_next);
    store_attention_rows<DB>(p.out + (uint64_t)tok * (uint32_t)inner + un.head * QA_HD + hi * 8, o, sum, true);
    init_acc(bq_next);  // unconditionally: the accumulators are then dead during the sweep on every path
    // 4. K, V and the bias slot are free again once every wave is through; and every wave's rows of the next unit's
    // first k-tile of A (issued above) have landed before any wave reads them.  Nothing that writes a register is
    // pending when the k-loop is entered again (see gemm_persistent.hip).
    // The 4 output stores (the last vector memory operations of this phase; they write no register) drain under the
    // next unit's first slots, whose first counted wait covers them.
    static_assert(DB * 2 == 4, "the wait below counts the output stores");
    __builtin_amdgcn_s_waitcnt(WAIT_VM4_LGKM0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- flat pipeline over (unit, k-tile), ping-pong between the two wave groups: see gemm_persistent.hip.  Per
  // k-tile j the slots M0 | C0 | M1 | C1; a memory slot reads the fragments of half a k-tile (8 + 3 ds_read_b128) and
  // issues loads (M0: the wave's 4 of A[j + 1]; M1: its 3 of W[j + 2]), a compute slot issues 24 MFMAs; group 1 runs
  // one slot behind group 0.  Waits: at the end of M1(j) for W[j + 1] (4 + 3 newer loads), at the end of C1(j) until
  // only the 3 loads of W[j + 2] are outstanding.
  // A compute slot here is 24 MFMAs = 384 cycles, a quarter shorter than the GEMM's: the memory slot of the other
  // group has to fit under it, so the k-tiles of a unit come in four kinds, each compiled as straight-line code of its
  // own without run-time decisions: FIRST also issues the 2 loads of the head's bias 4-vectors behind its A loads
  // (waits: 4 + 2 + 3 newer loads in M1, 2 + 3 outstanding after C1); MIDDLE; NEXT_TO_LAST, whose W loads open the next
  // unit's weight rows; LAST, which issues no A load (the stage it would fill carries Q first: attend() issues it)
  // and whose M1 wait therefore counts 3 newer loads.  In the workgroup's last unit the last two kinds wait for all.
  enum { FIRST = 0, MIDDLE = 1, NEXT_TO_LAST = 2, LAST = 3 };
  la_set_unit();
  lw_set_unit();
  issue_bias(decode(0).head);
  issue_a();
  issue_w();
  issue_w();
  __builtin_amdgcn_s_waitcnt(WAIT_VM0);
  __syncthreads();
  int sa = 0, sw = 0;
  for (int r = 0; r < n_my; ++r) {
    if (grp == 1) __builtin_amdgcn_s_barrier();
    const bool has_next = r + 1 < n_my;
    const bool with_bias = HAS_BIAS && r > 0;  // the first unit's bias came in with the prologue
    const int cur_head = decode(r).head;
    int sw_last = 0;
    auto k_tile = [&](auto kind_c) {
      constexpr int KIND = decltype(kind_c)::value;
      const unsigned char* s_a = smem + sa * QA_A_BYTES;
      const unsigned char* s_w = smem + QA_W_OFF + sw * QA_W_BYTES;
      sw_last = sw;
      sa ^= 1;
      sw = sw == 2 ? 0 : sw + 1;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        bf16x8 af[QA_FM], bfr[QA_FN];
#pragma unroll
        for (int i = 0; i < QA_FM; ++i) af[i] = *reinterpret_cast<const bf16x8*>(s_a + a_roff[half] + i * 16 * 128);
#pragma unroll
        for (int jn = 0; jn < QA_FN; ++jn) bfr[jn] = *reinterpret_cast<const bf16x8*>(s_w + b_roff[half] + jn * 16 * 128);
        __builtin_amdgcn_sched_barrier(0);
        if (half == 0) {
          if (KIND != LAST) issue_a_same_unit();
          if (KIND == FIRST && with_bias) issue_bias(cur_head);
        } else {
          if (KIND == FIRST || KIND == MIDDLE) {
            issue_w_same_unit();
          } else {  // the next unit's first two k-tiles of W (nothing once the list has ended)
            if (KIND == NEXT_TO_LAST) lw_next_unit();
            issue_w();
          }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (half == 0) __builtin_amdgcn_s_waitcnt(WAIT_LGKM0);
        else if (KIND == MIDDLE) __builtin_amdgcn_s_waitcnt(WAIT_VM7_LGKM0);
        else if (KIND == FIRST) {
          if (with_bias) __builtin_amdgcn_s_waitcnt(WAIT_VM9_LGKM0);
          else __builtin_amdgcn_s_waitcnt(WAIT_VM7_LGKM0);
        } else if (!has_next) __builtin_amdgcn_s_waitcnt(WAIT_ALL);
        else if (KIND == NEXT_TO_LAST) __builtin_amdgcn_s_waitcnt(WAIT_VM7_LGKM0);
        else __builtin_amdgcn_s_waitcnt(WAIT_VM3_LGKM0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < QA_FM; ++i)
#pragma unroll
          for (int jn = 0; jn < QA_FN; ++jn)
            acc[i][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[jn], af[i], acc[i][jn], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (half == 1) {
          if (KIND == MIDDLE) __builtin_amdgcn_s_waitcnt(WAIT_VM3);
          else if (KIND == FIRST) {
            if (with_bias) __builtin_amdgcn_s_waitcnt(WAIT_VM5);
            else __builtin_amdgcn_s_waitcnt(WAIT_VM3);
          } else if (!has_next) __builtin_amdgcn_s_waitcnt(WAIT_VM0);
          else __builtin_amdgcn_s_waitcnt(WAIT_VM3);
        }
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    k_tile(std::integral_constant<int, FIRST>{});
    for (int kt = 1; kt < KT - 2; ++kt) k_tile(std::integral_constant<int, MIDDLE>{});
    k_tile(std::integral_constant<int, NEXT_TO_LAST>{});
    k_tile(std::integral_constant<int, LAST>{});
    if (grp == 0) __builtin_amdgcn_s_barrier();
    attend(r, sw_last);
  }
}

bool qkv_attention_supported(int ws_y, int ws_x, int head_dim, int K, int64_t tokens_per_image) {
  return ws_y == QA_WS && ws_x == QA_WS && head_dim == QA_HD && K >= 256 && K % 128 == 0 &&
         tokens_per_image * K * 2 < (int64_t)0xFFFFFFF0u;
}

int64_t qkv_attention_bias_bytes(int heads) { return (int64_t)heads * QA_TBL * 16; }

hipError_t qkv_attention_configure() {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_window_attention_kernel<true>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, QA_SMEM);
  if (e != hipSuccess) return e;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(qkv_window_attention_kernel<false>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, QA_SMEM);
}

hipError_t qkv_attention_bias_launch(const void* table, float* out, int heads, hipStream_t stream) {
  const int n = heads * QA_TBL * 4;
  hipLaunchKernelGGL(qkv_attention_bias_kernel, dim3((n + 255) / 256), dim3(256), 0, stream,
                     reinterpret_cast<const uint16_t*>(table), out, heads);
  return hipGetLastError();
}

hipError_t qkv_attention_launch(const void* y, const void* w, const void* bias, const float* bias4, void* out, int B, int H,
                                int W, int heads, int K, int shift_y, int shift_x, int use_mask, float scale,
                                hipStream_t stream) {
  QkvAttnParams p;
  p.y = reinterpret_cast<const uint16_t*>(y);
  p.w = reinterpret_cast<const uint16_t*>(w);
  p.bias = reinterpret_cast<const uint16_t*>(bias);
  p.bias4 = bias4;
  p.out = reinterpret_cast<uint16_t*>(out);
  p.B = B; p.H = H; p.W = W; p.heads = heads; p.K = K;
  p.nWy = H / QA_WS; p.nWx = W / QA_WS;
  p.sy = shift_y; p.sx = shift_x;
  p.use_mask = use_mask;
  p.q_scale = scale * 1.4426950408889634f;
  p.n_win = B * p.nWy * p.nWx;
  const int max_seq = ((p.n_win + QA_GM - 1) / QA_GM + 7) / 8 * QA_GM * heads;  // units of the XCD with the most groups
  if ((int64_t)p.n_win * heads >= (1 << 24)) return hipErrorInvalidValue;  // the range of div_by_magic
  auto magic = [](int d) { return (((uint64_t)1 << 40) + (uint64_t)d - 1) / (uint64_t)d; };
  p.m_gsz = magic(QA_GM * heads);
  p.m_wpi = magic(p.nWy * p.nWx);
  p.m_nwx = magic(p.nWx);
  p.bpx = max_seq < 32 ? max_seq : 32;
  const dim3 grid(8 * p.bpx), block(QA_NT);
  if (bias4) hipLaunchKernelGGL(qkv_window_attention_kernel<true>, grid, block, QA_SMEM, stream, p);
  else hipLaunchKernelGGL(qkv_window_attention_kernel<false>, grid, block, QA_SMEM, stream, p);
  return hipGetLastError();
}

}  // namespace aeris
