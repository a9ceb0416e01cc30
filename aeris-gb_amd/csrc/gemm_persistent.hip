// Persistent bf16 MFMA GEMM for gfx950, 256x256 output tiles, k-tiles of 64:  C[M,N] = epilogue(A[M,K] * W[N,K]^T)
//
// Same LDS swizzle as the plain tile kernel (gemm.hip), built around what bounds it on MI355X:
//   - v_mfma_f32_16x16x32_bf16, not 32x32x16: same FLOP per cycle and the same LDS bytes per FLOP (a fragment is
//     16 rows x 32 k instead of 32 rows x 16 k), but on operands that change from instruction to instruction the
//     power-managed shader clock holds about 1.9 GHz with it against about 1.7 GHz with the larger shape
//   - global loads go straight into LDS (buffer_load ... lds): no staging registers, no ds_write, and the lane ->
//     address map of the load is the inverse of the LDS swizzle, so the tile lands in the layout the fragment reads
//     want.  A load instruction fetches 8 rows x 128 B: whole cache lines (the CU's address unit takes 64-byte row
//     pieces at 37 B/clk, whole lines at 57 B/clk)
//   - LDS holds two stages of the A tile and three of the W tile (160 KB); the loads of A run one k-tile ahead, those
//     of W two, over the flat sequence (tile, k-tile), so the next tile's first k-tiles are in flight while the
//     epilogue of the current tile runs (one workgroup per CU, persistent)
//   - the two waves of a SIMD alternate memory slots (LDS fragment reads + load issue) and compute slots (32 MFMAs):
//     a load instruction holds the issuing wave until the address unit has taken its 64 addresses, which would stall
//     the MFMA stream if the computing wave issued it
//   - tiles are ordered so that the workgroups resident on one XCD (blockIdx % 8) cover a contiguous chunk, 4 row
//     panels x all column tiles at a time: few distinct A / W k-slices per step compete for that XCD's 4 MB L2
//   - the epilogue stages through the idle A stage (wave-private 4 KB): fragments (4 consecutive n per lane) are
//     written swizzled, read back row-contiguous, and C / residual are accessed as full row segments (8 lanes x 16 B);
//     its loads are issued ahead of its stores because vector memory operations complete in order
#include "common.h"
#include "gemm_common.h"
#include "kernels.h"
#include <type_traits>

namespace aeris {

namespace {
constexpr int BM = 256, BN = 256, BK = 64, WM = 2, WN = 4;
constexpr int NT = WM * WN * 64;          // 512 threads
constexpr int FM = BM / WM / 16;          // 8 fragments of 16 rows
constexpr int FN = BN / WN / 16;          // 4 fragments of 16 columns
constexpr int A_BYTES = BM * BK * 2;      // 32 KB per stage of the A tile
constexpr int B_BYTES = BN * BK * 2;      // 32 KB per stage of the W tile
constexpr int A_STAGES = 2, B_STAGES = 3;
constexpr int B_OFF = A_STAGES * A_BYTES;
constexpr int SMEM = A_STAGES * A_BYTES + B_STAGES * B_BYTES;  // 160 KB: all of the CU's LDS
constexpr int GM = 4;                     // row panels per L2 group
}  // namespace

// PLAIN: no gate and no residual (qkv, fc1): the epilogue is compiled without those paths - about 2 % faster than
// deciding at run time, block by block, that there is nothing to load.  RES_BF16: bf16 C with a bf16 residual (proj,
// fc2 on a bf16 residual stream), compiled as a kernel of its own so that its deeper residual prefetch does not
// share registers with the general path.  RES_F32: the same for f32 C with an f32 residual (proj, fc2 on an f32
// residual stream).
template <int ACT, bool OUT_F32, bool PLAIN, bool RES_BF16 = false, bool RES_F32 = false>
__global__ void __launch_bounds__(NT) gemm_bf16_nt_persistent_kernel(GemmParams p_in) {
  static_assert(!(PLAIN && RES_BF16) && !(OUT_F32 && RES_BF16), "RES_BF16 is a non-plain bf16-output form");
  static_assert(!RES_F32 || (OUT_F32 && !PLAIN && !RES_BF16), "RES_F32 is a non-plain f32-output form");
  GemmParams p = p_in;
  if (RES_F32) p.res_dtype = AERIS_F32;
  if (PLAIN) {
    p.gate = nullptr;
    p.residual = nullptr;
    p.res_dtype = -1;
  }
  if (RES_BF16) p.res_dtype = AERIS_BF16;
  constexpr bool SWIGLU = ACT == AERIS_ACT_SWIGLU;
  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  constexpr int BN_OUT = SWIGLU ? BN / 2 : BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int l15 = lane & 15, q = lane >> 4;
  const int K = p.K, N = p.N;
  const int KT = K / BK;

  // ---- this workgroup's tile list: XCD x owns tiles [x*per_xcd, (x+1)*per_xcd), slot k takes every bpx-th
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int chunk0 = xcd * p.per_xcd;
  int chunk_len = p.total_tiles - chunk0;
  if (chunk_len > p.per_xcd) chunk_len = p.per_xcd;
  const int n_my = chunk_len > slot ? (chunk_len - slot + p.bpx - 1) / p.bpx : 0;
  if (n_my == 0) return;

  auto decode = [&](int r, int& tile_m, int& tile_n) {
    const int t = chunk0 + r * p.bpx + slot;
    const int gsz = GM * p.tiles_n;
    const int grp = (int)(((uint64_t)(uint32_t)t * p.m_gsz) >> 40), within = t - grp * gsz;
    int gm = p.tiles_m - grp * GM;
    if (gm > GM) gm = GM;
    static_assert(GM == 4, "the shift below");
    tile_n = gm == GM ? within >> 2 : within / gm;  // only the last group of row panels can be short
    tile_m = grp * GM + (within - tile_n * gm);
  };

  // ---- loader: global memory -> LDS without passing through registers (buffer_load ... lds, 16 bytes per lane).
  // One instruction of a wave fills 1 KB of LDS, lane l at byte 16 l: four 256-byte double rows = 8 rows of the
  // swizzled tile layout (swz_off), so the lane fetches the chunk which that layout keeps at its LDS slot (eight
  // consecutive lanes fetch the 128 contiguous bytes of one row).  Rows past the end of A or W are outside the
  // buffer descriptor and arrive as zeros; they only feed rows / columns of C that are never stored.
  // Per k-tile a wave brings in 32 rows of A and 32 rows of W, 4 instructions each.  Waves 0-3 (group 0) load the
  // rows of A that only group 0 reads, waves 4-7 those of group 1.  A and W are two independent streams over the
  // flat sequence (tile, k-tile): W runs one k-tile further ahead than A.
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int grp = wave_u / WN;
  uint32_t ld_voff[2];  // lane part of the source offset, for even / odd 8-row blocks
  {
    const int dr = lane >> 4, pos = lane & 15;
#pragma unroll
    for (int par = 0; par < 2; ++par) {
      const int logical = pos ^ (par * 4 + dr);
      ld_voff[par] = (uint32_t)((dr * 2 + (logical >> 3)) * K * 2 + (logical & 7) * 16);
    }
  }
  typedef __attribute__((address_space(3))) void* lds_ptr;
  const __amdgpu_buffer_rsrc_t rs_w =
      __builtin_amdgcn_make_buffer_rsrc((void*)p.W, 0, (int)((SWIGLU ? 2 : 1) * (int64_t)N * K * 2), 0x00020000);
  __amdgpu_buffer_rsrc_t rs_a = rs_w;
  int la_r = 0, la_kt = 0, la_stage = 0;  // A stream
  auto la_set_tile = [&]() {
    if (la_r >= n_my) {  // past the end of the list: a descriptor without records, the loads fetch nothing
      rs_a = __builtin_amdgcn_make_buffer_rsrc((void*)p.A, 0, 0, 0x00020000);
      return;
    }
    int tile_m, tile_n;
    decode(la_r, tile_m, tile_n);
    const int64_t m0 = (int64_t)tile_m * BM;
    int64_t rows = p.M - m0;
    if (rows > BM) rows = BM;
    rs_a = __builtin_amdgcn_make_buffer_rsrc((void*)(p.A + m0 * K), 0, (int)(rows * K * 2), 0x00020000);
  };
  // Always 4 loads, also past the end of the list (into stages nobody reads any more, from a descriptor without
  // records): the number of loads in flight at any point of the k-loop is then the same for every k-tile, and no wait
  // has to be chosen at run time.
  auto issue_a = [&]() {
    unsigned char* sd = smem + la_stage * A_BYTES + wave_u * 4096;
    const uint32_t so = (uint32_t)(wave_u * 32) * (uint32_t)(K * 2) + (uint32_t)la_kt * (BK * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_a, (lds_ptr)(sd + i * 1024), 16, ld_voff[i & 1],
                                               so + (uint32_t)(i * 8) * (uint32_t)(K * 2), 0, 0);
    la_stage ^= 1;
    if (++la_kt == KT) {
      la_kt = 0;
      ++la_r;
      la_set_tile();
    }
  };
  uint32_t lw_row = 0;  // W row of the first of this wave's 32 rows of the tile
  int lw_r = 0, lw_kt = 0, lw_stage = 0;  // W stream
  __amdgpu_buffer_rsrc_t rs_wc = rs_w;  // the W stream's descriptor: rs_w, or one without records past the end of the list
  auto lw_set_tile = [&]() {
    if (lw_r >= n_my) {
      rs_wc = __builtin_amdgcn_make_buffer_rsrc((void*)p.W, 0, 0, 0x00020000);
      lw_row = 0;
      return;
    }
    int tile_m, tile_n;
    decode(lw_r, tile_m, tile_n);
    const int n0 = tile_n * BN_OUT;
    // SwiGLU: tile rows [64 c, 64 c + 64) are the gate rows, then the up rows, of 32 output columns
    if (SWIGLU) lw_row = (uint32_t)((wave_u & 1) * N + n0 + (wave_u >> 1) * 32);
    else lw_row = (uint32_t)(n0 + wave_u * 32);
  };
  auto issue_w = [&]() {
    unsigned char* sd = smem + B_OFF + lw_stage * B_BYTES + wave_u * 4096;
    const uint32_t so = lw_row * (uint32_t)(K * 2) + (uint32_t)lw_kt * (BK * 2);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_wc, (lds_ptr)(sd + i * 1024), 16, ld_voff[i & 1],
                                               so + (uint32_t)(i * 8) * (uint32_t)(K * 2), 0, 0);
    if (++lw_stage == B_STAGES) lw_stage = 0;
    if (++lw_kt == KT) {
      lw_kt = 0;
      ++lw_r;
      lw_set_tile();
    }
  };

  // ---- fragment read offsets (per k-step of 32), relative to the stage of A / of W: lane (l15, q) reads the 8
  // elements k = 32 ks + 8 q .. of row l15 of a 16-row fragment
  uint32_t a_roff[2], b_roff[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) {
    a_roff[ks] = swz_off(wm * (BM / WM) + l15, ks * 4 + q);
    b_roff[ks] = swz_off(wn * (BN / WN) + l15, ks * 4 + q);
  }

  // ---- accumulators.  They start a tile at the bias instead of zero: the bias add costs nothing that way.
  // A lane's fragment columns are 4 consecutive n per column fragment j: n = first column of the wave + 16 j + 4 q
  // (SwiGLU: fragments 0, 1 are the gate columns, 2, 3 the up columns of the same 32 outputs).
  // N % 4 == 0, so a group of 4 is entirely inside or entirely outside the matrix (outside: clamped, computed,
  // never stored).
  constexpr int NJ = SWIGLU ? FN / 2 : FN;  // column fragments of the output
  f32x4 acc[FM][FN];
  auto wave_col0 = [&](int r) {  // first output column of this wave in tile r of the list
    int tile_m, tile_n;
    decode(r, tile_m, tile_n);
    return tile_n * BN_OUT + (wave_u % WN) * (SWIGLU ? 32 : BN / WN);
  };
  auto load_bias = [&](int r, u32x2 (&bq)[FN], int q) {  // q: lane >> 4, from the caller (the epilogue passes its own copy)
    const int n_wave = wave_col0(r);
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      int n = n_wave + (SWIGLU ? (j & 1) : j) * 16 + q * 4;
      if (n >= N) n = N - 4;
      bq[j] = u32x2{0u, 0u};
      if (p.bias) bq[j] = *reinterpret_cast<const u32x2*>(p.bias + (SWIGLU ? (j >> 1) * N : 0) + n);
    }
  };
  auto init_acc = [&](const u32x2 (&bq)[FN]) {
#pragma unroll
    for (int j = 0; j < FN; ++j) {
      const f32x4 b = {bf16_lo(bq[j].x), bf16_hi(bq[j].x), bf16_lo(bq[j].y), bf16_hi(bq[j].y)};
#pragma unroll
      for (int i = 0; i < FM; ++i) acc[i][j] = b;
    }
  };
  {
    u32x2 bq[FN];
    load_bias(0, bq, q);
    init_acc(bq);
  }

  // s_waitcnt immediates: vmcnt in bits 3:0 (and 15:14), expcnt in 6:4 (7 = no wait), lgkmcnt in 11:8 (15 = no wait)
  constexpr int WAIT_LGKM0 = 0xC07F, WAIT_VM0 = 0x0F70, WAIT_VM4 = 0x0F74, WAIT_VM8_LGKM0 = 0x0078;

  // ---- epilogue of the tile whose accumulators are complete.
  // Vector memory operations of a wave complete in order, so a wait for a load also waits for every store issued
  // before it.  The epilogue therefore loads everything it can ahead of its stores: the per-column operands
  // (gate) once per tile, the residual rows of the next 32-row block before the stores of the current one, the
  // bias of the next tile (for its accumulators) at the very start.
  auto epilogue = [&](int r_done) {
    // Everything the epilogue derives from the lane number (staging addresses, column offsets, row offsets) does
    // not depend on the tile; deriving it from a laundered copy of the lane number recomputes it per tile (a few
    // dozen operations) and keeps it out of the registers of the main loop, where the compiler would otherwise
    // park all of it.
    int lane_t = lane;
    asm volatile("" : "+v"(lane_t));
    const int l15 = lane_t & 15, q = lane_t >> 4;
    const int rrow = lane_t >> 3, rch = lane_t & 7;  // read-back mapping: row rrow + 8*it, 16-byte chunk rch
    int tile_m, tile_n;
    decode(r_done, tile_m, tile_n);
    const int64_t m_base = (int64_t)tile_m * BM + grp * (BM / WM);
    // Row addressing: the first row of this wave group in C / the residual is a wave-uniform 64-bit base, a lane adds
    // its row r (0..127, relative) times the row stride as a 24-bit multiply (strides < 2^23, checked at launch)
    // instead of a 64 x 64-bit multiply per access.  rows_left <= 0: a group entirely below the matrix.
    const int64_t rows_left64 = p.M - m_base;
    const int rows_left = rows_left64 < BM / WM ? (int)rows_left64 : BM / WM;
    const int ld24 = (int)p.ldc, rs24 = (int)c_row_stride(p);
    const int rrow_t = rrow;
    const int n_wave = tile_n * BN_OUT + (wave_u % WN) * (SWIGLU ? 32 : BN / WN);  // first output column of this wave
    u32x2 bq_next[FN];  // loaded ahead of the last block's stores, used after them
    // The query part of a qkv projection is multiplied by q_scale here, in fp32, before its only rounding.  Whole
    // 64-column wave blocks lie inside or outside the query columns (q_cols % 64 == 0, checked at launch): a
    // wave-uniform branch that two thirds of the tiles of such a projection skip.
    if (PLAIN && ACT == AERIS_ACT_NONE && !OUT_F32 && n_wave < p.q_cols) {
      const float qs = p.q_scale;
#pragma unroll
      for (int i = 0; i < FM; ++i)
#pragma unroll
        for (int j = 0; j < FN; ++j) acc[i][j] *= qs;
    }
    // Staging area of this wave, 32 rows of 128 B: the A stage that the loader fills next is idle during the
    // epilogue, and the 4 KB of it that this wave's own loads will fill are written by nobody else.
    unsigned char* stg = smem + la_stage * A_BYTES + wave_u * 4096;

    // gate: one row of p.gate per batch.  A tile whose rows are all in one batch (the usual case) loads its gate
    // columns once; otherwise every lane looks up the row of its own fragment row.
    // The per-lane lookup avoids a 64-bit division per row: row r of the group (0..127) is in batch b0 if r < r1
    // (r1 = first row of the next batch), else in batch b0 + 1 + (r - r1) / rows_per_batch, and that quotient of
    // numbers below 128 is a multiply by ceil(2^16 / rows_per_batch) and a shift (0 when a batch has 128 rows or more).
    const float* gate_tile = nullptr;
    bool gate_per_lane = false;
    int gate_b0 = 0, gate_r1 = 0;
    uint32_t gate_magic = 0;
    if (p.gate) {
      if (p.gate_batch_stride == 0) {
        gate_tile = p.gate;
      } else {
        int64_t last = m_base + BM / WM - 1;
        if (last > p.M - 1) last = p.M - 1;
        const int64_t b0 = (int64_t)(((uint64_t)(uint32_t)m_base * p.rpb_magic) >> p.rpb_shift);
        const int64_t b1 = (int64_t)(((uint64_t)(uint32_t)last * p.rpb_magic) >> p.rpb_shift);
        if (b0 == b1) {
          gate_tile = p.gate + b0 * p.gate_batch_stride;
        } else {
          gate_per_lane = true;
          gate_b0 = (int)b0;
          gate_r1 = (int)((b0 + 1) * p.rows_per_batch - m_base);
          if (p.rows_per_batch < BM / WM) gate_magic = (65536u + (uint32_t)p.rows_per_batch - 1u) / (uint32_t)p.rows_per_batch;
        }
      }
    }
    // stage 1: activation on the 16 x 16 fragment of row fragment i, output column fragment j (the bias is in the
    // accumulators already).  The gate is applied after the staging, where a lane holds consecutive columns of
    // one row and needs far fewer gate registers.
    auto fragment = [&](int i, int j, float (&v)[4]) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float x = acc[i][j][e];
        if (SWIGLU) x = silu_f(x) * acc[i][j + 2][e];
        else if (ACT == AERIS_ACT_GELU) x = OUT_F32 ? gelu_erf_f(x) : gelu_bf16_f(x);
        v[e] = x;
      }
    };
    auto gate_row_of = [&](int r) {  // slow path: the group's rows straddle a batch boundary; r = row in the group
      if (r > rows_left - 1) r = rows_left - 1;
      const int d = r - gate_r1;
      const int b = gate_b0 + (d < 0 ? 0 : 1 + (int)(((uint32_t)d * gate_magic) >> 16));
      return p.gate + (int64_t)b * (int64_t)(int)p.gate_batch_stride;
    };

    // bf16 C: block i of 32 rows (two row fragments) goes to the staging area as rows of 128 B, chunk-swizzled.
    // A row's 16-byte chunk (8 columns) of column fragment j is split between the lanes q = 0 / 1 (columns 0-3 /
    // 4-7 of the fragment) or q = 2 / 3 (8-11 / 12-15).  v_permlane16_swap on the registers of fragments 2m and
    // 2m+1 gives the lanes q = 0, 2 the two whole chunks of fragment 2m and the lanes q = 1, 3 those of fragment
    // 2m+1: one ds_write_b128 per lane and fragment pair instead of two conflicting ds_write_b64.
    auto stage_block_bf16 = [&](int i) {
#pragma unroll
      for (int ii = 0; ii < 2; ++ii) {
        u32x2 w2[NJ];
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          float v[4];
          fragment(2 * i + ii, j, v);
          w2[j] = u32x2{pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
        }
#pragma unroll
        for (int mm = 0; mm < NJ / 2; ++mm) {
          const auto rx = __builtin_amdgcn_permlane16_swap(w2[2 * mm].x, w2[2 * mm + 1].x, false, false);
          const auto ry = __builtin_amdgcn_permlane16_swap(w2[2 * mm].y, w2[2 * mm + 1].y, false, false);
          *reinterpret_cast<u32x4*>(stg + swz_off(ii * 16 + l15, 4 * mm + 2 * (q & 1) + (q >> 1))) =
              u32x4{rx[0], ry[0], rx[1], ry[1]};
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    // Interior tiles of the two forms that gain from it (bf16 residual with an optional per-tile gate: +5 % on
    // K = 1536; plain GELU: +1 %; plain without activation measured 2 % slower this way and stays on the general
    // path) take a path without any per-lane condition: every row and column of the group's 128 x 64 block is
    // inside the matrix.  Straight-line code lets the compiler wait for exactly the loads a block needs (with the
    // branches of the general path it waited for the next block's residual rows right after the stores), and the
    // residual rows are requested two blocks ahead: block 0 at the start, block 1 once block 0's accumulators
    // are staged and their registers free, blocks 2 and 3 after blocks 0 and 1 have been combined.
    const bool interior = (RES_BF16 || (PLAIN && ACT == AERIS_ACT_GELU)) && !OUT_F32 && !SWIGLU &&
                          rows_left == BM / WM && n_wave + BN / WN <= N && !gate_per_lane;
    // Interior plain SwiGLU tiles skip the staging (in the read-back of the general path half of the lanes idle on
    // its 64-byte rows; +2 %).  For the other forms this was slower (qkv -4 %, proj -5 %: 64-byte row pieces), although
    // gate and residual are then applied in fp32 before the only rounding.
    const bool interior_direct = SWIGLU && PLAIN && !OUT_F32 && rows_left == BM / WM && n_wave + 32 <= N;
    // Every path ends in a wait of its own.  Nothing that writes a register may be pending when the k-loop is entered:
    // the compiler would guard the fragment registers with a wait for all vector memory operations inside the loop,
    // on every k-tile, which cuts the lead of the W loads to one slot.  The first k-tile needs the oldest loads at once
    // anyway.  Stores write no register: the straight-line paths end with 4 of them behind their last load (the next
    // tile's bias) and leave those to drain under the first slots of the next tile, whose first counted wait (end of
    // M1(0)) covers them.  The wait has to stand inside the path: behind the join the compiler no longer knows that the
    // operations left outstanding are stores, and puts a wait for all of them into the k-loop.
    if (interior_direct) {
      // No staging: after a swap between lane rows (v_permlane16_swap on the registers of column fragments 2m and
      // 2m + 1) lane (l15, q) owns 8 consecutive columns, 32 m + 16 (q & 1) + 8 (q >> 1) .., of row 16 i + l15: four
      // lanes cover 64 contiguous bytes of a row of C, a store instruction 16 rows.
      constexpr int NP = NJ / 2;
      unsigned char* c_lane[NP];
#pragma unroll
      for (int m = 0; m < NP; ++m) {
        const int n = n_wave + 32 * m + 16 * (q & 1) + 8 * (q >> 1);
        c_lane[m] = reinterpret_cast<unsigned char*>(p.C) + (m_base * c_row_stride(p) + c_col_off(p, n)) * 2;
      }
#pragma unroll
      for (int i = 0; i < FM; ++i) {
        if (i + 1 == FM && r_done + 1 < n_my) load_bias(r_done + 1, bq_next, q);
#pragma unroll
        for (int m = 0; m < NP; ++m) {
          float a[4], b[4];
          fragment(i, 2 * m, a);
          fragment(i, 2 * m + 1, b);
          const auto rx = __builtin_amdgcn_permlane16_swap(pack_bf16x2(a[0], a[1]), pack_bf16x2(b[0], b[1]), false, false);
          const auto ry = __builtin_amdgcn_permlane16_swap(pack_bf16x2(a[2], a[3]), pack_bf16x2(b[2], b[3]), false, false);
          *reinterpret_cast<u32x4*>(c_lane[m] + (int64_t)__mul24(i * 16 + l15, rs24) * 2) = u32x4{rx[0], ry[0], rx[1], ry[1]};
        }
      }
      __builtin_amdgcn_s_waitcnt(WAIT_VM0);
    } else if (interior) {
      const int n = n_wave + rch * 8;
      unsigned char* const c_lane =
          reinterpret_cast<unsigned char*>(p.C) + (m_base * c_row_stride(p) + c_col_off(p, n)) * 2;
      f32x4 gt0 = {1.f, 1.f, 1.f, 1.f}, gt1 = {1.f, 1.f, 1.f, 1.f};
      if (gate_tile) {
        gt0 = *reinterpret_cast<const f32x4*>(gate_tile + n);
        gt1 = *reinterpret_cast<const f32x4*>(gate_tile + n + 4);
      }
      const unsigned char* const res_lane =
          reinterpret_cast<const unsigned char*>(p.residual) + (m_base * p.ldc + n) * 2;
      u32x4 rq[FM / 2][4];
      auto load_res = [&](int b) {
#pragma unroll
        for (int it = 0; it < 4; ++it)
          rq[b][it] = *reinterpret_cast<const u32x4*>(res_lane + (int64_t)__mul24(b * 32 + rrow + 8 * it, ld24) * 2);
      };
      if (RES_BF16) load_res(0);
#pragma unroll
      for (int i = 0; i < FM / 2; ++i) {
        stage_block_bf16(i);
        if (RES_BF16 && i == 0) load_res(1);
        u32x4 out[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          u32x4 w4 = *reinterpret_cast<const u32x4*>(stg + swz_off(rrow + 8 * it, rch));
          if (RES_BF16) {
            float o[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) { o[2 * e] = bf16_lo(w4[e]); o[2 * e + 1] = bf16_hi(w4[e]); }
#pragma unroll
            for (int e = 0; e < 4; ++e) { o[e] *= gt0[e]; o[4 + e] *= gt1[e]; }
            const u32x4 r4 = rq[i][it];
#pragma unroll
            for (int e = 0; e < 4; ++e) { o[2 * e] += bf16_lo(r4[e]); o[2 * e + 1] += bf16_hi(r4[e]); }
            w4 = u32x4{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7])};
          }
          out[it] = w4;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        // the next loads go ahead of the stores below
        if (RES_BF16 && i + 2 < FM / 2) load_res(i + 2);
        if (i + 1 == FM / 2 && r_done + 1 < n_my) load_bias(r_done + 1, bq_next, q);
#pragma unroll
        for (int it = 0; it < 4; ++it)
          *reinterpret_cast<u32x4*>(c_lane + (int64_t)__mul24(i * 32 + rrow + 8 * it, rs24) * 2) = out[it];
      }
      __builtin_amdgcn_s_waitcnt(WAIT_VM4);  // the 4 stores of the last block may still be on their way
    } else if (!OUT_F32) {
      // stage 2 (bf16 C): a whole 32 x 64 (SwiGLU: 32 x 32) block through LDS, rows of 128 B, chunk-swizzled; it
      // is read back as 16-byte chunks, 8 lanes per row, and C / residual are accessed as full row segments
      constexpr int CHUNKS = SWIGLU ? 4 : 8;  // 16-byte chunks (8 columns) per staged row
      const int n = n_wave + rch * 8;
      const bool col_ok = rch < CHUNKS && n < N;
      const bool full = n + 8 <= N;  // N % 4 == 0: a chunk is whole or exactly its first half is inside
      // residual: 16 bytes (bf16) or 2 x 16 bytes (f32) per lane and row, from an address that is always valid:
      // rows are clamped to M - 1, a half chunk reads the 4 columns before it as well (bf16) or its first half
      // twice (f32)
      int n_ld = n;
      if (!col_ok) n_ld = n_wave;
      else if (!full && (RES_BF16 || p.res_dtype == AERIS_BF16)) n_ld = n - 4;
      const bool upper = col_ok && !full;  // bf16: the wanted 4 columns are the upper half of what was loaded
      const int n_g = col_ok ? n : n_wave;
      // where this lane's chunk of row 0 goes in C / comes from in the residual
      unsigned char* const c_lane =
          reinterpret_cast<unsigned char*>(p.C) + (m_base * c_row_stride(p) + c_col_off(p, col_ok ? n : n_wave)) * 2;
      f32x4 gt0 = {1.f, 1.f, 1.f, 1.f}, gt1 = {1.f, 1.f, 1.f, 1.f};
      if (gate_tile) {
        gt0 = *reinterpret_cast<const f32x4*>(gate_tile + n_g);
        gt1 = *reinterpret_cast<const f32x4*>(gate_tile + n_g + (full ? 4 : 0));
      }
      const unsigned char* const res_lane = reinterpret_cast<const unsigned char*>(p.residual) +
                                            (m_base * p.ldc + n_ld) * ((RES_BF16 || p.res_dtype == AERIS_BF16) ? 2 : 4);
      const int res_dtype = RES_BF16 ? (int)AERIS_BF16 : p.res_dtype;
      u32x4 rq[4][2];
      auto load_res = [&](int i) {
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          int r = i * 32 + rrow_t + 8 * it;
          if (r > rows_left - 1) r = rows_left - 1;  // rows below the matrix read its last row (may be negative: M >= 1)
          const int64_t off = (int64_t)__mul24(r, ld24);
          if (res_dtype == AERIS_BF16) {
            rq[it][0] = *reinterpret_cast<const u32x4*>(res_lane + off * 2);
          } else {
            const float* rp = reinterpret_cast<const float*>(res_lane + off * 4);
            rq[it][0] = *reinterpret_cast<const u32x4*>(rp);
            rq[it][1] = *reinterpret_cast<const u32x4*>(rp + (full ? 4 : 0));
          }
        }
      };
      if (res_dtype >= 0) load_res(0);
#pragma unroll
      for (int i = 0; i < FM / 2; ++i) {  // blocks of 32 rows = two row fragments
        stage_block_bf16(i);
        u32x4 out[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int row = rrow + 8 * it;
          u32x4 w4 = *reinterpret_cast<const u32x4*>(stg + swz_off(row, rch));
          if (p.gate || res_dtype >= 0) {
            float o[8];
#pragma unroll
            for (int e = 0; e < 4; ++e) { o[2 * e] = bf16_lo(w4[e]); o[2 * e + 1] = bf16_hi(w4[e]); }
            if (gate_per_lane) {
              const float* gr = gate_row_of(i * 32 + row);
              gt0 = *reinterpret_cast<const f32x4*>(gr + n_g);
              gt1 = *reinterpret_cast<const f32x4*>(gr + n_g + (full ? 4 : 0));
            }
            if (p.gate) {
#pragma unroll
              for (int e = 0; e < 4; ++e) { o[e] *= gt0[e]; o[4 + e] *= gt1[e]; }
            }
            if (res_dtype == AERIS_BF16) {
              u32x4 r4 = rq[it][0];
              if (upper) { r4.x = r4.z; r4.y = r4.w; }
#pragma unroll
              for (int e = 0; e < 4; ++e) { o[2 * e] += bf16_lo(r4[e]); o[2 * e + 1] += bf16_hi(r4[e]); }
            } else if (res_dtype == AERIS_F32) {
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                o[e] += __uint_as_float(rq[it][0][e]);
                o[4 + e] += __uint_as_float(rq[it][1][e]);
              }
            }
            w4 = u32x4{pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7])};
          }
          out[it] = w4;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (i + 1 < FM / 2) {
          if (res_dtype >= 0) load_res(i + 1);  // ahead of the stores below
        } else if (r_done + 1 < n_my) {
          load_bias(r_done + 1, bq_next, q);
        }
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int r = i * 32 + rrow_t + 8 * it;
          if (col_ok && r < rows_left) {
            unsigned char* cp = c_lane + (int64_t)__mul24(r, rs24) * 2;
            if (full) *reinterpret_cast<u32x4*>(cp) = out[it];
            else *reinterpret_cast<u32x2*>(cp) = u32x2{out[it].x, out[it].y};
          }
        }
      }
      __builtin_amdgcn_s_waitcnt(WAIT_VM0);
    } else if (RES_F32 && ACT != AERIS_ACT_SWIGLU && rows_left == BM / WM && n_wave + BN / WN <= N && !gate_per_lane) {
      // Interior tiles with f32 C and an f32 residual: the staging of the general f32 path below (units of 32 rows x
      // 32 columns through the wave's 4 KB), as straight-line code without per-lane conditions, the residual rows
      // requested two units ahead of their use and always ahead of the stores of the unit before.
      constexpr int NU = FN / 2, UNITS = FM / 2 * NU;
      const int n_lane = n_wave + rch * 4;
      f32x4 gt[NU];
#pragma unroll
      for (int j = 0; j < NU; ++j) {
        gt[j] = f32x4{1.f, 1.f, 1.f, 1.f};
        if (gate_tile) gt[j] = *reinterpret_cast<const f32x4*>(gate_tile + n_lane + 32 * j);
      }
      const unsigned char* const res_lane = reinterpret_cast<const unsigned char*>(p.residual) + (m_base * p.ldc + n_lane) * 4;
      unsigned char* const c_lane = reinterpret_cast<unsigned char*>(p.C) + (m_base * p.ldc + n_lane) * 4;
      u32x4 rq[3][4];
      auto load_res = [&](int u) {
#pragma unroll
        for (int it = 0; it < 4; ++it)
          rq[u % 3][it] = *reinterpret_cast<const u32x4*>(
              res_lane + ((int64_t)__mul24((u / NU) * 32 + rrow + 8 * it, ld24) + (u % NU) * 32) * 4);
      };
      load_res(0);
#pragma unroll
      for (int u = 0; u < UNITS; ++u) {
        const int i = u / NU, j = u % NU;
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            float v[4];
            fragment(2 * i + ii, 2 * j + jj, v);
            *reinterpret_cast<f32x4*>(stg + swz_off(ii * 16 + l15, jj * 4 + q)) = f32x4{v[0], v[1], v[2], v[3]};
          }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if (u == 0) load_res(1);  // once the first unit's accumulators are staged and their registers free
        f32x4 out[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          f32x4 o = *reinterpret_cast<const f32x4*>(stg + swz_off(rrow + 8 * it, rch));
          o *= gt[j];
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] += __uint_as_float(rq[u % 3][it][e]);
          out[it] = o;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (u + 2 < UNITS) load_res(u + 2);  // ahead of the stores below
        if (u + 1 == UNITS && r_done + 1 < n_my) load_bias(r_done + 1, bq_next, q);
#pragma unroll
        for (int it = 0; it < 4; ++it)
          *reinterpret_cast<f32x4*>(c_lane + ((int64_t)__mul24(i * 32 + rrow + 8 * it, ld24) + j * 32) * 4) = out[it];
      }
      __builtin_amdgcn_s_waitcnt(WAIT_VM4);  // the 4 stores of the last unit may still be on their way
    } else {
      // stage 2 (f32 C): units of 32 rows x 32 columns (2 x 2 fragments), rows of 128 B (32 floats), 4 floats per
      // lane and row
      constexpr int NU = NJ / 2;  // units per block of 32 rows
      constexpr int UNITS = FM / 2 * NU;
      u32x4 rq[4];
      auto unit_col = [&](int u) { return n_wave + (u % NU) * 32 + rch * 4; };
      f32x4 gt[NU];
#pragma unroll
      for (int j = 0; j < NU; ++j) {
        int n = unit_col(j);
        if (n >= N) n = N - 4;
        gt[j] = f32x4{1.f, 1.f, 1.f, 1.f};
        if (gate_tile) gt[j] = *reinterpret_cast<const f32x4*>(gate_tile + n);
      }
      auto load_res = [&](int u) {
        const int i = u / NU;
        int n = unit_col(u);
        if (n >= N) n = N - 4;
        const unsigned char* const res_lane = reinterpret_cast<const unsigned char*>(p.residual) +
                                              (m_base * p.ldc + n) * (p.res_dtype == AERIS_BF16 ? 2 : 4);
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          int r = i * 32 + rrow_t + 8 * it;
          if (r > rows_left - 1) r = rows_left - 1;
          const int64_t off = (int64_t)__mul24(r, ld24);
          if (p.res_dtype == AERIS_BF16) {
            const u32x2 r2 = *reinterpret_cast<const u32x2*>(res_lane + off * 2);
            rq[it] = u32x4{r2.x, r2.y, 0u, 0u};
          } else {
            rq[it] = *reinterpret_cast<const u32x4*>(res_lane + off * 4);
          }
        }
      };
      if (p.res_dtype >= 0) load_res(0);
#pragma unroll
      for (int u = 0; u < UNITS; ++u) {
        const int i = u / NU, j = u % NU;
#pragma unroll
        for (int ii = 0; ii < 2; ++ii)
#pragma unroll
          for (int jj = 0; jj < 2; ++jj) {
            float v[4];
            fragment(2 * i + ii, 2 * j + jj, v);
            *reinterpret_cast<f32x4*>(stg + swz_off(ii * 16 + l15, jj * 4 + q)) = f32x4{v[0], v[1], v[2], v[3]};
          }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        f32x4 out[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int row = rrow + 8 * it;
          f32x4 o = *reinterpret_cast<const f32x4*>(stg + swz_off(row, rch));
          if (gate_per_lane) {
            int n = unit_col(u);
            if (n >= N) n = N - 4;
            gt[j] = *reinterpret_cast<const f32x4*>(gate_row_of(i * 32 + row) + n);
          }
          if (p.gate) o *= gt[j];
          if (p.res_dtype == AERIS_BF16) {
            o.x += bf16_lo(rq[it].x); o.y += bf16_hi(rq[it].x); o.z += bf16_lo(rq[it].y); o.w += bf16_hi(rq[it].y);
          } else if (p.res_dtype == AERIS_F32) {
#pragma unroll
            for (int e = 0; e < 4; ++e) o[e] += __uint_as_float(rq[it][e]);
          }
          out[it] = o;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        if (u + 1 < UNITS) {
          if (p.res_dtype >= 0) load_res(u + 1);  // ahead of the stores below
        } else if (r_done + 1 < n_my) {
          load_bias(r_done + 1, bq_next, q);
        }
        const int n = unit_col(u);
        unsigned char* const c_lane =
            reinterpret_cast<unsigned char*>(p.C) + (m_base * c_row_stride(p) + c_col_off(p, n < N ? n : 0)) * 4;
#pragma unroll
        for (int it = 0; it < 4; ++it) {
          const int r = i * 32 + rrow_t + 8 * it;
          if (r < rows_left && n < N) *reinterpret_cast<f32x4*>(c_lane + (int64_t)__mul24(r, rs24) * 4) = out[it];
        }
      }
      __builtin_amdgcn_s_waitcnt(WAIT_VM0);
    }
    if (r_done + 1 < n_my) init_acc(bq_next);
  };

  // ---- flat pipeline over (tile, k-tile), ping-pong between the two wave groups.
  // Group 0 (wm = 0, one wave per SIMD) and group 1 (wm = 1, the other wave of each SIMD) run, per k-tile j, the
  // slots  M0 | C0 | M1 | C1 : a memory slot reads the fragments of half a k-tile (12 ds_read_b128) and issues 4
  // loads, a compute slot issues the 32 MFMAs on those fragments.  Group 1 runs one slot behind group 0 and every
  // slot ends in a workgroup barrier: while one wave of a SIMD computes, the other one does its memory work.
  // Slots are numbered globally: group 0 runs k-tile j in slots 4j .. 4j+3, group 1 in 4j+1 .. 4j+4.
  //   A, two stages: the rows of A[j-1] that a group reads are last read in its M1(j-1); the group's own waves
  //     reload them with A[j+1] in their M0(j), three slots before that group's M0(j+1) reads them.
  //   W, three stages: W[j-1] is last read in slot 4j-1; every wave loads its rows of W[j+2] into that stage in
  //     its M1(j) (slots 4j+2, 4j+3), five slots before slot 4j+8 reads them.
  // Waits (vector memory operations complete in order, so a count of the loads issued since is enough, and
  // anything the epilogue has issued in between only makes a wait more conservative): group 0 reads A[j+1] and
  // W[j+1] in slot 4j+4.  Each wave of group 0 waits at the end of its C1(j) until only its 4 loads of W[j+2] are
  // outstanding; each wave of group 1 waits for its rows of W[j+1] at the end of its M1(j) (slot 4j+3; 8 newer
  // loads) and for its rows of A[j+1] at the end of its C1(j).  Both groups take both waits (for group 0 the first
  // one is early, for loads a k-tile old), and the streams keep issuing past the end of the list, so the waits are
  // the same constants in every k-tile: nothing is decided at run time between a barrier and the next MFMAs.
  // A slot ends in a bare s_barrier: the fences of __syncthreads() would make every wave wait for all of its
  // outstanding loads into LDS.  What a barrier has to order is stated explicitly with s_waitcnt.
  la_set_tile();
  lw_set_tile();
  issue_a();
  issue_w();
  issue_w();
  __builtin_amdgcn_s_waitcnt(WAIT_VM0);
  __syncthreads();
  int sa = 0, sw = 0;  // the A and W stages of the k-tile at hand
  for (int r = 0; r < n_my; ++r) {
    // Group 1 runs one slot behind group 0.  The offset is set up anew for every tile (group 1 waits one slot
    // here, group 0 one slot before its epilogue), so that both groups run their epilogues at the same time:
    // with the epilogues one slot apart, each would hold up the other group at a barrier.
    if (grp == 1) __builtin_amdgcn_s_barrier();
    for (int kt = 0; kt < KT; ++kt) {
      const unsigned char* s_a = smem + sa * A_BYTES;
      const unsigned char* s_w = smem + B_OFF + sw * B_BYTES;
      sa ^= 1;
      if (++sw == B_STAGES) sw = 0;
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        // ---- memory slot: LDS reads first (queued, non-blocking), then the loads
        bf16x8 af[FM], bfr[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) af[i] = *reinterpret_cast<const bf16x8*>(s_a + a_roff[half] + i * 16 * 128);
#pragma unroll
        for (int jn = 0; jn < FN; ++jn) bfr[jn] = *reinterpret_cast<const bf16x8*>(s_w + b_roff[half] + jn * 16 * 128);
        __builtin_amdgcn_sched_barrier(0);
        if (half == 0) issue_a();
        else issue_w();
        __builtin_amdgcn_sched_barrier(0);
        // (group 0 needs its rows of W[j+1] only one slot later and could do without the vmcnt part here; waiting in both
        // groups costs nothing - those loads are a k-tile old - and spares a decision per slot)
        if (half == 0) __builtin_amdgcn_s_waitcnt(WAIT_LGKM0);
        else __builtin_amdgcn_s_waitcnt(WAIT_VM8_LGKM0);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // ---- compute slot
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
          for (int jn = 0; jn < FN; ++jn)
            acc[i][jn] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bfr[jn], af[i], acc[i][jn], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
        if (half == 1) __builtin_amdgcn_s_waitcnt(WAIT_VM4);
        __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (grp == 0) __builtin_amdgcn_s_barrier();
    epilogue(r);  // leaves the accumulators at the bias of the next tile
  }
}

hipError_t gemm_persistent_configure() {
  hipError_t e;
#define CFG1(A, F32, PL)                                                                                   \
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_nt_persistent_kernel<A, F32, PL>),         \
                          hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);                                 \
  if (e != hipSuccess) return e;
#define CFG(A, F32) CFG1(A, F32, false) CFG1(A, F32, true)
  CFG(AERIS_ACT_NONE, false) CFG(AERIS_ACT_NONE, true) CFG(AERIS_ACT_GELU, false) CFG(AERIS_ACT_GELU, true)
  CFG(AERIS_ACT_SWIGLU, false) CFG(AERIS_ACT_SWIGLU, true)
#undef CFG
#undef CFG1
#define CFGR(A)                                                                                            \
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_nt_persistent_kernel<A, false, false, true>), \
                          hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);                                 \
  if (e != hipSuccess) return e;
  CFGR(AERIS_ACT_NONE) CFGR(AERIS_ACT_GELU) CFGR(AERIS_ACT_SWIGLU)
#undef CFGR
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_nt_persistent_kernel<AERIS_ACT_NONE, true, false, false, true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, SMEM);
  if (e != hipSuccess) return e;
  return hipSuccess;
}

// p.act must be NONE, GELU or SWIGLU; N % 4 == 0 and ldc % 4 == 0; bias / gate rows 8- / 16-byte aligned
hipError_t gemm_persistent_launch(const GemmParams& p0, hipStream_t stream) {
  GemmParams p = p0;
  const bool swiglu = p.act == AERIS_ACT_SWIGLU;
  const int bn_out = swiglu ? BN / 2 : BN;
  p.tiles_m = (int)((p.M + BM - 1) / BM);
  p.tiles_n = (p.N + bn_out - 1) / bn_out;
  p.total_tiles = p.tiles_m * p.tiles_n;
  p.per_xcd = (p.total_tiles + 7) / 8;
  p.bpx = p.per_xcd < 32 ? p.per_xcd : 32;  // 32 CUs per XCD, one workgroup each
  if (p.total_tiles >= (1 << 24)) return hipErrorInvalidValue;  // the range of the multiply-shift division
  p.m_gsz = (((uint64_t)1 << 40) + (uint64_t)(GM * p.tiles_n) - 1) / (uint64_t)(GM * p.tiles_n);
  // rows of a tile (first row of a wave group, at most tiles_m * 256 + 128) and rows_per_batch below 2^31
  if ((int64_t)p.tiles_m * BM + BM >= (int64_t(1) << 31) || p.rows_per_batch <= 0 || p.rows_per_batch >= (int64_t(1) << 31))
    return hipErrorInvalidValue;
  {
    int lg = 0;
    while (((int64_t)1 << lg) < p.rows_per_batch) ++lg;
    p.rpb_shift = 31 + lg;
    p.rpb_magic = (uint32_t)((((uint64_t)1 << p.rpb_shift) + (uint64_t)p.rows_per_batch - 1) / (uint64_t)p.rows_per_batch);
  }
  dim3 grid(8 * p.bpx), block(NT);
  const bool f32 = p.c_dtype == AERIS_F32;
  const bool plain = !p.gate && p.res_dtype < 0;
  const bool res_bf16 = !f32 && p.res_dtype == AERIS_BF16;
  if (f32 && p.res_dtype == AERIS_F32 && p.act == AERIS_ACT_NONE && !p.split) {
    hipLaunchKernelGGL((gemm_bf16_nt_persistent_kernel<AERIS_ACT_NONE, true, false, false, true>), grid, block, SMEM, stream, p);
    return hipGetLastError();
  }
#define GO1(A, F32)                                                                                        \
  do {                                                                                                     \
    if (plain) hipLaunchKernelGGL((gemm_bf16_nt_persistent_kernel<A, F32, true>), grid, block, SMEM, stream, p);  \
    else hipLaunchKernelGGL((gemm_bf16_nt_persistent_kernel<A, F32, false>), grid, block, SMEM, stream, p);       \
  } while (0)
#define GO(A)                                                                                              \
  do {                                                                                                     \
    if (res_bf16)                                                                                            \
      hipLaunchKernelGGL((gemm_bf16_nt_persistent_kernel<A, false, false, true>), grid, block, SMEM, stream, p);  \
    else if (f32) GO1(A, true);                                                                              \
    else GO1(A, false);                                                                                      \
  } while (0)
  if (swiglu) GO(AERIS_ACT_SWIGLU);
  else if (p.act == AERIS_ACT_GELU) GO(AERIS_ACT_GELU);
  else GO(AERIS_ACT_NONE);
#undef GO
#undef GO1
  return hipGetLastError();
}

}  // namespace aeris
