// Windowed multi-head self-attention for gfx950, streaming variant: windows of any size up to 4096 tokens
// (the reference's 60 x 60) and head_dim 64 or 128, no relative-position bias, no shift mask (model.py:289-293).
//
// One workgroup = 256 queries of one (window, head): 8 waves x 32 queries, one workgroup per CU (with 128 queries per
// workgroup and two workgroups per CU every K / V chunk was loaded, transposed and stored twice as often per query:
// 6-7 % slower).  The keys of the window are streamed
// through LDS in chunks of 64 (four buffers: the global loads of chunk j+2 are in flight while chunk j is
// being consumed, and are written to LDS at its end) with an online softmax (running row max m and row sum l, output rescaled only when a max
// moves).  Window partition, window reverse and the cyclic shift are address arithmetic exactly as in the
// one-window-per-workgroup kernel (window_attention.hip); the token row of every window position is computed once
// per workgroup into an LDS table, so the streaming loop needs no integer division.
//
//   K chunk [64][HD]   global -> registers -> LDS, 16-byte chunks XOR-swizzled (conflict-free ds_read_b128)
//   V chunk [64][HD]   global -> registers (4 keys x 8 d per thread) -> 4x8 register transpose -> LDS as
//                      V^T [HD][64], key groups permuted so that a PV fragment is one ds_read_b128
//   Q                  global -> registers (MFMA B operand), once
//   S^T = K Q^T        v_mfma_f32_32x32x16_bf16; lane = one query, registers = keys
//   O^T += V^T P^T     P^T straight from the S^T accumulator registers
// The query blocks of one (window, head) are placed on the same XCD (blockIdx % 8), so its K / V rows are fetched
// into that XCD's L2 once and re-read from there by the other query blocks.
#include "common.h"
#include "kernels.h"
#include <type_traits>

namespace aeris {

namespace {

struct StreamParams {
  const uint16_t* qkv;
  uint16_t* out;
  int64_t tok_stride, head_stride, part_stride;  // q / k / v addressing, as in the one-window kernel
  int B, H, W, heads;
  int nWy, nWx, ws_y, ws_x;
  int sy, sx;
  int n_units, qblks;
  float scale;
  int q_prescaled;  // q already holds q * scale * log2(e)
  uint32_t span_bytes;  // DMA form: bytes of one image's k (or v) plane that a token offset can reach, < 2^32
};

constexpr int KC = 64;    // keys per chunk
constexpr int NWAVE = 8;         // waves per workgroup (two per SIMD, one workgroup per CU)
constexpr int QB = 32 * NWAVE;   // queries per workgroup
constexpr int MAX_L = 4096;
// K / V chunk buffers in LDS.  With four, chunk j + 2 is written while chunk j is consumed and the workgroup needs a
// barrier only after every second chunk (2 buffers, one barrier per chunk: 2.5 % slower).
constexpr int NBUF = 4;

// byte offset of 16-byte chunk `chunk` of row `row` in a tile with 128-byte rows (8 chunks), swizzled over double rows
__device__ __forceinline__ uint32_t off128(int row, int chunk) {
  return (uint32_t)((row >> 1) * 256 + (((((row & 1) << 3) | chunk) ^ ((row >> 1) & 7)) << 4));
}
// V^T tile (rows = d, 128 bytes = 64 keys each): the chunk XOR also takes bits 4-6 of the row.  With the thread -> (key
// group, d piece) map of the V staging below, both the transposing 8-byte writes (16 lanes = 8 pieces 8 rows apart x 2
// key groups in the two halves of a chunk) and the fragment reads (16 lanes = 16 consecutive rows) are free of bank
// conflicts (LDS counters: 3.9 cycles per instruction each); with off128() and consecutive threads on the pieces of
// one key group the writes were 8-way conflicts, 31 cycles per instruction, and took most of the kernel's LDS time.
// (head_dim 64, where half of the threads stage V and the writes are 4-way conflicts, is faster with the plain
// layout and thread order: measured, -8 % with this one.)
template <int HD>
__device__ __forceinline__ uint32_t vt_off(int d, int chunk) {
  return (uint32_t)((d >> 1) * 256 + ((((d & 1) << 3) | (chunk ^ ((d >> 1) & 7) ^ (HD == 128 ? (d >> 4) & 7 : 0))) << 4));
}
// the same for 256-byte rows (16 chunks)
__device__ __forceinline__ uint32_t off256(int row, int chunk) { return (uint32_t)(row * 256 + ((chunk ^ (row & 15)) << 4)); }

template <int HD>
struct StreamCfg {
  static constexpr int K_BYTES = KC * HD * 2;
  static constexpr int V_BYTES = HD * KC * 2;
  static constexpr int BUF = K_BYTES + V_BYTES;
  // the K chunks of all buffers first, then the V^T chunks: with head_dim 128 every K fragment of every buffer is
  // then within the 64 KB that the offset field of an LDS read reaches from one per-lane base
  static constexpr int V_BASE = NBUF * K_BYTES;
  static constexpr int TBL_OFF = NBUF * BUF;
};

}  // namespace

// DMA (head_dim 128): K and V chunks go into LDS by the load unit itself (buffer_load ... lds: no staging registers,
// no ds_write, no transposing VALU work) and V stays row-major; the V^T fragments of P V then come from
// ds_read_b64_tr_b16, the LDS read that transposes on the way out (within 16 lanes, source lane 4e + a reads 4
// consecutive elements and result lane 4a + b receives element b of source lanes a, 4 + a, 8 + a, 12 + a).  Rows of
// 256 B, 16-byte chunks XOR-swizzled: K by row & 15 (conflict-free ds_read_b128 fragments), V by 4 (row & 3) (the 4
// keys x 4 column groups that the two 16-lane halves of a transposing read's 32-lane pass gather - 16 pieces of 16
// bytes - land on the 16 distinct slots of a 256-byte bank period; with 2 (row & 3) the two halves shared eight).  Needs every byte offset
// inside an image's k / v plane to fit 32 bits (span_bytes; checked by the launcher).
template <int HD, bool DMA>
__global__ void __launch_bounds__(64 * NWAVE) __attribute__((amdgpu_waves_per_eu(2)))
window_attention_stream_kernel(StreamParams p) {
  static_assert(!DMA || HD == 128, "the DMA form is built for head_dim 128");
  using Cfg = StreamCfg<HD>;
  constexpr int CH = HD / 8;   // 16-byte chunks per head row
  constexpr int KS = HD / 16;  // k16 steps of QK^T
  constexpr int DB = HD / 32;  // 32-row blocks of O^T
  constexpr int NT = 64 * NWAVE;
  constexpr int KIT = KC * CH / NT;                     // 16-byte K pieces per thread and chunk (1 or 2)
  constexpr int V_ITEMS = (KC / 4) * CH;                // (4 keys x 8 d) V pieces per chunk: 128 or 256
  constexpr float LOG2E = 1.4426950408889634f;

  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const uint32_t smem_addr = lds_byte_address(smem);
  int* tok = reinterpret_cast<int*>(smem + Cfg::TBL_OFF);  // token row (inside the image) of every window position
  int* const redo = tok + ((p.ws_y * p.ws_x + 3) & ~3);    // set by a wave whose sums left the range of the fast sweep

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l31 = lane & 31, hi = lane >> 5;

  // all query blocks of one (window, head) on one XCD
  const int xcd = blockIdx.x & 7, s_idx = blockIdx.x >> 3;
  const int unit = xcd + 8 * (s_idx / p.qblks);
  const int qb = s_idx % p.qblks;
  if (unit >= p.n_units) return;
  const int head = unit % p.heads;
  const int win = unit / p.heads;
  const int wpi = p.nWy * p.nWx;
  const int b = win / wpi;
  const int wrem = win - b * wpi;
  const int wy = wrem / p.nWx, wx = wrem - wy * p.nWx;
  const int H = p.H, W = p.W;
  const int L = p.ws_y * p.ws_x;
  const int inner = p.heads * HD;
  const uint32_t ld_qkv = (uint32_t)p.tok_stride;  // token rows and their stride fit 32 bits: one 32 x 32 -> 64-bit multiply-add per address
  const int64_t img_base = (int64_t)b * H * W;
  const int y0 = wy * p.ws_y + p.sy, x0 = wx * p.ws_x + p.sx;

  for (int pos = tid; pos < L; pos += NT) {
    int Y = y0 + pos / p.ws_x;
    int X = x0 + pos % p.ws_x;
    if (Y >= H) Y -= H;
    if (X >= W) X -= W;
    tok[pos] = Y * W + X;
  }
  if (tid == 0) *redo = 0;
  __syncthreads();

  // ---- Q fragments (B operand): lane = query, 8 consecutive d per k16 step
  int qpos = qb * QB + wave * 32 + l31;
  const bool q_valid = qpos < L;
  if (!q_valid) qpos = L - 1;
  const int64_t q_row = img_base + tok[qpos];
  bf16x8 qf[KS];
  {
    const uint16_t* qp = p.qkv + head * p.head_stride + (uint64_t)(uint32_t)q_row * ld_qkv + hi * 8;
#pragma unroll
    for (int s = 0; s < KS; ++s) qf[s] = *reinterpret_cast<const bf16x8*>(qp + s * 16);
  }
  {
    // q is multiplied by scale * log2(e) once, here (the reference scales q in bf16 too, model.py:290): the
    // accumulators of K Q^T are then the logits in the exp2 domain and no score needs a multiply.  q_prescaled: the
    // producer of q has applied the factor in fp32 before its only rounding, and this is a multiplication by one
    const float c = p.q_prescaled ? 1.0f : p.scale * LOG2E;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      const u32x4 w = __builtin_bit_cast(u32x4, qf[s]);
      u32x4 r;
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = pack_bf16x2(bf16_lo(w[e]) * c, bf16_hi(w[e]) * c);
      qf[s] = __builtin_bit_cast(bf16x8, r);
    }
  }

  const uint16_t* kbase = p.qkv + img_base * (int64_t)ld_qkv + p.part_stride + head * p.head_stride;
  const uint16_t* vbase = p.qkv + img_base * (int64_t)ld_qkv + 2 * p.part_stride + head * p.head_stride;
  const int nch = (L + KC - 1) / KC;

  u32x4 kreg[KIT], vreg[4];
  const bool v_item = (V_ITEMS >= NT) || tid < V_ITEMS;  // waves 0-3 (head_dim 64: waves 0-1) carry a V piece
  // V piece of this thread: 4 keys (key group v_kg of the chunk) x 8 d (piece v_c).  Lane bits 0-2 (and 4 for head_dim
  // 128) select the piece - the lanes of a key group still cover whole rows of V - bit 3 the key group within a pair
  // that shares a 16-byte chunk of V^T: see vt_off().
  const int v_b3 = (tid >> 3) & 1, v_b4 = (tid >> 4) & 1, v_b5 = (tid >> 5) & 1;
  const int v_c = HD == 128 ? 8 * v_b4 + (tid & 7) : tid % CH;
  const int v_kg = HD == 128 ? 4 * (tid >> 6) + 2 * v_b3 + v_b5 : tid / CH;
  auto load_chunk = [&](int j) {
    const int key0 = j * KC;
#pragma unroll
    for (int it = 0; it < KIT; ++it) {
      const int idx = tid + it * NT, key = idx / CH, c = idx % CH;
      int kp = key0 + key;
      if (kp > L - 1) kp = L - 1;  // rows past the window: any valid row, their scores are masked
      kreg[it] = *reinterpret_cast<const u32x4*>(kbase + (uint64_t)(uint32_t)tok[kp] * ld_qkv + c * 8);
    }
    if (v_item) {
      const int kg = v_kg, c = v_c;
#pragma unroll
      for (int jj = 0; jj < 4; ++jj) {
        int kp = key0 + kg * 4 + jj;
        if (kp > L - 1) kp = L - 1;
        vreg[jj] = *reinterpret_cast<const u32x4*>(vbase + (uint64_t)(uint32_t)tok[kp] * ld_qkv + c * 8);
      }
    }
  };
  auto store_chunk = [&](int buf) {
    unsigned char* sK = smem + buf * Cfg::K_BYTES;
    unsigned char* sV = smem + Cfg::V_BASE + buf * Cfg::V_BYTES;
#pragma unroll
    for (int it = 0; it < KIT; ++it) {
      const int idx = tid + it * NT, key = idx / CH, c = idx % CH;
      *reinterpret_cast<u32x4*>(sK + (HD == 64 ? off128(key, c) : off256(key, c))) = kreg[it];
    }
    // V: 4 keys x 8 d register transpose -> V^T[d][key].  Inside every block of 16 keys the four key groups are
    // stored in the order 0, 2, 1, 3: the 8 keys one lane needs for a k16 step of PV (4hi..4hi+3 and
    // 8+4hi..8+4hi+3, the accumulator layout of S^T) are then one aligned 16-byte chunk.
    if (v_item) {
      const int kg = v_kg, c = v_c;
      const int pos = (kg & ~3) | (((kg & 1) << 1) | ((kg >> 1) & 1));
#pragma unroll
      for (int w = 0; w < 4; ++w) {  // word w holds d = 8c + 2w (low half) and 8c + 2w + 1 (high half)
        u32x2 lo, hi2;
        lo.x = (vreg[0][w] & 0xffffu) | (vreg[1][w] << 16);
        lo.y = (vreg[2][w] & 0xffffu) | (vreg[3][w] << 16);
        hi2.x = (vreg[0][w] >> 16) | (vreg[1][w] & 0xffff0000u);
        hi2.y = (vreg[2][w] >> 16) | (vreg[3][w] & 0xffff0000u);
        const int d0 = c * 8 + 2 * w, d1 = d0 + 1;
        *reinterpret_cast<u32x2*>(sV + vt_off<HD>(d0, pos >> 1) + (pos & 1) * 8) = lo;
        *reinterpret_cast<u32x2*>(sV + vt_off<HD>(d1, pos >> 1) + (pos & 1) * 8) = hi2;
      }
    }
  };

  // DMA form: one instruction of a wave fills 1 KB = 4 rows of a chunk; wave w issues rows 4w.. and 32 + 4w.. of K and
  // of V.  Lane = (row within the four, LDS chunk slot); it fetches the global chunk that the swizzle keeps there.
  // Keys past the window get an offset outside the descriptor and arrive as zeros (their scores are masked).
  typedef __attribute__((address_space(3))) void* lds_vptr;
  const __amdgpu_buffer_rsrc_t rs_k = __builtin_amdgcn_make_buffer_rsrc((void*)kbase, 0, (int)p.span_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t rs_v = __builtin_amdgcn_make_buffer_rsrc((void*)vbase, 0, (int)p.span_bytes, 0x00020000);
  auto issue_chunk = [&](int j, int buf) {
    const int rsub = lane >> 4, pc = lane & 15;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int ii = wave + NWAVE * i;  // 0..15
      const int row = 4 * ii + rsub, key = j * KC + row;
      const uint32_t rowoff = key < L ? (uint32_t)tok[key < L ? key : 0] * (ld_qkv * 2u) : 0xFFFFF000u;
      const uint32_t ok = rowoff + (uint32_t)((pc ^ (row & 15)) << 4), ov = rowoff + (uint32_t)((pc ^ (4 * rsub)) << 4);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_k, (lds_vptr)(smem + buf * Cfg::K_BYTES + ii * 1024), 16, ok, 0, 0, 0);
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rs_v, (lds_vptr)(smem + Cfg::V_BASE + buf * Cfg::V_BYTES + ii * 1024), 16, ov, 0, 0, 0);
    }
  };
  // per-lane part of the transposing V reads: block of 16 lanes jb = lane >> 4 (d half jb & 1, key half jb >> 1),
  // source lane 4e + a inside it reads V[key0 + 4 (jb >> 1) + e][32 db + 16 (jb & 1) + 4a ..]
  typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
  typedef __attribute__((address_space(3))) bf16x4_t* lds_bf16x4_ptr;
  uint32_t v_tr[DB];
  if (DMA) {
    const int jb = lane >> 4, e = (lane >> 2) & 3, a = lane & 3;
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = (4 * db + 2 * (jb & 1) + (a >> 1)) ^ (4 * e);
      v_tr[db] = (uint32_t)(Cfg::V_BASE + (4 * (jb >> 1) + e) * (HD * 2) + (chunk << 4) + (a & 1) * 8);
      asm volatile("" : "+v"(v_tr[db]));
    }
  }

  // Fragment addresses = per-lane part (below, loop-invariant) + compile-time part (buffer, key block / row block):
  //   K fragment of k16 step s, key block kb:  k_lane[s] + buf * K_BYTES + kb * 32 rows
  //   V^T fragment of step, row block db:      v_lane[head_dim 128: step ^ db, else step] + V_BASE + buf * V_BYTES + db * 4096
  // (the swizzles depend on the row only through bits that the block offsets leave alone)
  // (kept as opaque 32-bit LDS addresses: left to itself the compiler splits them again into a common and a per-step
  // part and adds the two in front of every read)
  typedef __attribute__((address_space(3))) const unsigned char* lds_cptr;
  lds_cptr k_lane[KS], v_lane[4];
#pragma unroll
  for (int sq = 0; sq < KS; ++sq) {
    k_lane[sq] = (lds_cptr)(smem + (HD == 64 ? off128(l31, 2 * sq + hi) : off256(l31, 2 * sq + hi)));
    asm volatile("" : "+v"(k_lane[sq]));
  }
#pragma unroll
  for (int sx = 0; sx < 4; ++sx) {
    v_lane[sx] = (lds_cptr)(smem + Cfg::V_BASE +
                 (HD == 128 ? (uint32_t)((l31 >> 1) * 256 + (l31 & 1) * 128) + (uint32_t)(((2 * sx) ^ hi ^ ((l31 >> 1) & 7) ^ (l31 >> 4)) << 4)
                            : vt_off<HD>(l31, 2 * sx + hi)));
    asm volatile("" : "+v"(v_lane[sx]));
  }
  float m = -INFINITY, l = 0.f;
  f32x16 o[DB];
  // A wave whose 32 queries all lie past the window (last query block of a window whose size is not a multiple of 256)
  // only stages K / V and keeps the barriers; its MFMA and softmax work would be thrown away.
  const bool wave_active = qb * QB + wave * 32 < L;  // wave-uniform

  // One pass over the window's keys.  FAST: P = exp2(logit) without a row maximum - softmax does not depend on the
  // subtracted constant, the maximum only guards the range, and the range is checked afterwards.  Otherwise the
  // online form: running maximum m, accumulated output and sum rescaled whenever a maximum moves.
  auto sweep = [&](auto fast_tag) {
  constexpr bool FAST = decltype(fast_tag)::value;
  m = -INFINITY;
  l = 0.f;
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[db][e] = 0.f;

  if (DMA) {
    issue_chunk(0, 0);
    if (nch > 1) issue_chunk(1, 1);
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): this wave's loads into LDS have landed
  } else {
    load_chunk(0);
    store_chunk(0);
    if (NBUF == 4 && nch > 1) {
      load_chunk(1);
      store_chunk(1);
    }
  }
  __syncthreads();

  // the chunk loop is unrolled over the buffers, so that the buffer a chunk sits in is a compile-time constant
  for (int j0 = 0; j0 < nch; j0 += NBUF) {
#pragma unroll
  for (int u = 0; u < NBUF; ++u) {
    const int j = j0 + u;
    if (j >= nch) break;
    constexpr int LEAD = NBUF / 2;  // chunk j + LEAD is loaded and written to LDS while chunk j is consumed
    if (DMA) {
      // both chunks of the next pair are requested at the start of this pair (the buffers were last read before the
      // barrier that ended the pair before), and awaited at the barrier that ends this pair
      if ((u & 1) == 0) {
        if (j + LEAD < nch) issue_chunk(j + LEAD, (u + LEAD) & (NBUF - 1));
        if (j + LEAD + 1 < nch) issue_chunk(j + LEAD + 1, (u + LEAD + 1) & (NBUF - 1));
      }
    } else if (j + LEAD < nch) {
      load_chunk(j + LEAD);
    }
    f32x16 acc[2];
    if (wave_active) {

    // ---- S^T = K Q^T for the 64 keys of the chunk: acc[kb][4g+i] = <k[key], q>, key = 64j + 32kb + 8g + 4hi + i
    // The K fragments are read PF MFMAs ahead of their use (left to itself the compiler reads each one right before
    // its MFMA and exposes the LDS latency every time).
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[kb][e] = 0.f;
    {
      constexpr int PF = 2, NS = 2 * KS;
      bf16x8 kfr[PF + 1];
      auto read_k = [&](int t) {  // rows 32 (t / KS) + l31, 16-byte chunk 2 (t % KS) + hi
        typedef __attribute__((address_space(3))) const bf16x8* frag_ptr;
        return *(frag_ptr)(k_lane[t % KS] + u * Cfg::K_BYTES + (t / KS) * 32 * (HD * 2));
      };
#pragma unroll
      for (int t = 0; t < PF; ++t) kfr[t] = read_k(t);
#pragma unroll
      for (int t = 0; t < NS; ++t) {
        if (t + PF < NS) kfr[(t + PF) % (PF + 1)] = read_k(t + PF);
        __builtin_amdgcn_sched_barrier(0);
        acc[t / KS] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[t % (PF + 1)], qf[t % KS], acc[t / KS], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if (j * KC + KC > L) {  // last, partial chunk (uniform): keys past the window do not take part
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = j * KC + kb * 32 + (e >> 2) * 8 + hi * 4 + (e & 3);
          if (key >= L) acc[kb][e] = -INFINITY;
        }
    }

    // PV step (kb, t2): k slots 0-3 <-> keys 32kb+16t2+4hi+(0..3); slots 4-7 <-> keys 32kb+16t2+8+4hi+(0..3): one V^T
    // chunk per 32-row block of O^T.  The fragments of a step are read one step ahead of its MFMAs.
    // DMA form: the transposing reads are inline assembly (the builtin form would make the compiler wait for the load
    // unit's pending loads of the next chunks in front of every one of them, see lds_read_tr16_b64); what they return
    // becomes usable in v_ready().
    bf16x8 vfb[2][DB];
    TrFrag vtr[2][DMA ? DB : 1];
    auto load_v = [&](int step, int slot) {  // V^T rows 32 db + l31, chunk step * 2 + hi: vt_off(), taken apart
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        if (DMA) {  // keys 16 step + 4 hi + (0..3) and 16 step + 8 + 4 hi + (0..3) of row-major V, transposed by the read
          const uint32_t a0 = smem_addr + v_tr[db] + u * Cfg::V_BYTES + step * 16 * (HD * 2);
          vtr[slot][DMA ? db : 0].lo = lds_read_tr16_b64<0>(a0);
          vtr[slot][DMA ? db : 0].hi = lds_read_tr16_b64<8 * (HD * 2)>(a0);
        } else {
          vfb[slot][db] = *(__attribute__((address_space(3))) const bf16x8*)(v_lane[HD == 128 ? step ^ db : step] + u * Cfg::V_BYTES + db * 4096);
        }
      }
    };
    auto v_ready = [&](int slot) {
      if (DMA) {
        static_assert(!DMA || DB == 4, "the DMA form is built for head_dim 128");
        lds_tr_wait(vtr[slot][0], vtr[slot][DMA ? 1 : 0], vtr[slot][DMA ? 2 : 0], vtr[slot][DMA ? 3 : 0]);
#pragma unroll
        for (int db = 0; db < DB; ++db) vfb[slot][db] = tr_frag_value(vtr[slot][DMA ? db : 0]);
      }
    };
    load_v(0, 0);  // in flight during the softmax arithmetic below

    // ---- online softmax (exp2 domain): new row max, rescale what has been accumulated if any max moved
    if (!FAST) {
      float cm = acc[0][0];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; e += 2) cm = fmaxf(fmaxf(cm, acc[kb][e]), acc[kb][e + 1]);
      cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
      const float m_new = fmaxf(m, cm);
      if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {
        const float alpha = __builtin_amdgcn_exp2f(m - m_new);  // 0 for the first chunk (m = -inf)
        l *= alpha;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int e = 0; e < 16; ++e) o[db][e] *= alpha;
        m = m_new;
      }
    }

    // ---- P = exp2(s) or exp2(s - m) for 16 keys at a time and O^T += V^T P^T: while the MFMAs of a step run, the P of the next
    // step is formed (the VALU work hides the MFMAs) and its V^T fragments are read
    uint32_t pkb[2][4];
    auto exp_step = [&](int step, uint32_t (&pk)[4]) {
      const int kb = step >> 1, t2 = step & 1;
#pragma unroll
      for (int h = 0; h < 4; ++h) {
        const int h2 = 4 * t2 + h;
        const float e0 = __builtin_amdgcn_exp2f(FAST ? acc[kb][2 * h2] : acc[kb][2 * h2] - m);
        const float e1 = __builtin_amdgcn_exp2f(FAST ? acc[kb][2 * h2 + 1] : acc[kb][2 * h2 + 1] - m);
        pk[h] = pack_bf16x2(e0, e1);
        l = dot2_ones(pk[h], l);  // the row sum of what PV multiplies: the rounded values, one instruction per pair
      }
    };
    exp_step(0, pkb[0]);
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      __builtin_amdgcn_sched_barrier(0);
      v_ready(step & 1);  // ahead of the next step's reads: the wait then covers reads issued a whole step ago only
      if (step + 1 < 4) {
        load_v(step + 1, (step + 1) & 1);
        exp_step(step + 1, pkb[(step + 1) & 1]);
      }
      const uint32_t* pk = pkb[step & 1];
      const u32x4 pw = {pk[0], pk[1], pk[2], pk[3]};
      const bf16x8 pf = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
      for (int db = 0; db < DB; ++db) o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfb[step & 1][db], pf, o[db], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    }  // wave_active

    if (!DMA && j + LEAD < nch) store_chunk((u + LEAD) & (NBUF - 1));
    if (NBUF == 2 || (u & 1)) {
      if (DMA) __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the next pair's chunks, requested two chunks ago
      __syncthreads();
    }
  }
  }
  };  // sweep

  sweep(std::true_type{});
  // Range check of the sweep without maximum: a row sum that left [2^-40, 2^100] (or is not a number) means logits
  // beyond what exp2 holds without the maximum; the workgroup then repeats the window's keys in the online form.
  {
    const float lt = l + __shfl_xor(l, 32, 64);
    const bool bad = wave_active && !(lt >= 0x1p-40f && lt <= 0x1p100f);
    if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0) *redo = 1;
    __syncthreads();
    if (*redo != 0) sweep(std::false_type{});
  }

  // ---- normalise and store: o[db][4g+i] = O[query][32db + 8g + 4hi + i]
  l += __shfl_xor(l, 32, 64);
  const float inv = __builtin_amdgcn_rcpf(l);
  if (q_valid) {
    uint16_t* op = p.out + q_row * inner + head * HD + hi * 4;
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

static int stream_smem(int head_dim, int L) { return NBUF * (KC * head_dim * 2 + head_dim * KC * 2) + ((L * 4 + 15) / 16) * 16 + 16; }

bool attention_stream_supported(int ws_y, int ws_x, int head_dim, bool has_bias, bool use_mask) {
  const int64_t L = (int64_t)ws_y * ws_x;
  return (head_dim == 64 || head_dim == 128) && L >= 1 && L <= MAX_L && !has_bias && !use_mask;
}

hipError_t attention_stream_configure_all() {
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(window_attention_stream_kernel<64, false>),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, stream_smem(64, MAX_L));
  if (e != hipSuccess) return e;
  e = hipFuncSetAttribute(reinterpret_cast<const void*>(window_attention_stream_kernel<128, false>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, stream_smem(128, MAX_L));
  if (e != hipSuccess) return e;
  return hipFuncSetAttribute(reinterpret_cast<const void*>(window_attention_stream_kernel<128, true>),
                             hipFuncAttributeMaxDynamicSharedMemorySize, stream_smem(128, MAX_L));
}

hipError_t attention_stream_launch(const void* qkv, void* out, int B, int H, int W, int heads, int head_dim, int ws_y,
                                   int ws_x, int shift_y, int shift_x, float scale, int q_prescaled, int64_t tok_stride,
                                   int64_t head_stride, int64_t part_stride, hipStream_t stream) {
  StreamParams p;
  p.q_prescaled = q_prescaled;
  p.tok_stride = tok_stride; p.head_stride = head_stride; p.part_stride = part_stride;
  p.qkv = reinterpret_cast<const uint16_t*>(qkv);
  p.out = reinterpret_cast<uint16_t*>(out);
  p.B = B; p.H = H; p.W = W; p.heads = heads;
  p.nWy = H / ws_y; p.nWx = W / ws_x; p.ws_y = ws_y; p.ws_x = ws_x;
  p.sy = shift_y; p.sx = shift_x;
  p.scale = scale;
  const int L = ws_y * ws_x;
  p.n_units = B * p.nWy * p.nWx * heads;
  p.qblks = (L + QB - 1) / QB;
  const int64_t grid = (int64_t)((p.n_units + 7) / 8) * 8 * p.qblks;
  const int smem = stream_smem(head_dim, L);
  // bytes of an image's k (or v) plane that a token offset can reach; the DMA form addresses them with 32 bits
  const int64_t span = ((int64_t)H * W - 1) * tok_stride * 2 + (int64_t)head_dim * 2;
  p.span_bytes = span < ((int64_t)1 << 32) - 4096 ? (uint32_t)span : 0u;
  if (head_dim == 64)
    hipLaunchKernelGGL((window_attention_stream_kernel<64, false>), dim3((unsigned)grid), dim3(64 * NWAVE), smem, stream, p);
  else if (p.span_bytes != 0 && tok_stride > 0)
    hipLaunchKernelGGL((window_attention_stream_kernel<128, true>), dim3((unsigned)grid), dim3(64 * NWAVE), smem, stream, p);
  else
    hipLaunchKernelGGL((window_attention_stream_kernel<128, false>), dim3((unsigned)grid), dim3(64 * NWAVE), smem, stream, p);
  return hipGetLastError();
}

}  // namespace aeris
