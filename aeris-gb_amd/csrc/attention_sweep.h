// The arithmetic of one 32-query group against the keys of one window, shared by every one-window attention kernel:
// logits' start values (relative-position bias) and shift mask, the sweep over the key blocks, the two-pass form for
// rows whose logits leave the range of the sweep, and the normalised store of the output rows.
//
// Operand layout (v_mfma_f32_32x32x16_bf16, lane = l31 + 32 hi):
//   S^T block kb = K[32 kb ..][:] Q^T: a[4g + i] is the logit (times log2 e) of key 32 kb + 8 g + 4 hi + i and the lane's
//   query l31.  P^T = exp2(S^T) packed to bf16 pairs is, register for register, the B operand of O^T = V^T P^T: k slots
//   0-3 of PV step 2 kb + t2 are the keys 32 kb + 16 t2 + 4 hi + (0..3), slots 4-7 the keys 32 kb + 16 t2 + 8 + 4 hi + (0..3).
//   o[db][4g + i] = O[query][32 db + 8 g + 4 hi + i].
// A kernel supplies how its K and V^T fragments are read from LDS: `load_k(kb, f)`, and for V^T one of the two
// loaders below (`load_v(step, raw)` issues the reads of one 16-key step, `load_v.ready(...)` turns what was read into
// MFMA operands once it is needed).
#pragma once
#include "common.h"

namespace aeris {

// V^T fragments from a row-major V tile by the transposing LDS read.  Within every 16 lanes, source lane 4 e + a reads 4
// consecutive elements and result lane 4 a + b receives element b of the source lanes a, 4 + a, 8 + a, 12 + a: with
// source lane 4 e + a at V[key0 + e][d0 + 4 a ..] the result lane owns column d0 + (lane & 15) of the keys
// key0 .. key0 + 3, half of an MFMA operand's 8 k slots.  V rows are 128 B with 16-byte chunks XOR-swizzled by
// 2 (key & 3).  `step_base(step)` is the LDS byte address of V row 16 step.  The reads are issued as inline assembly
// (see lds_read_tr16_b64): ready() is the s_waitcnt that makes their results usable.
template <int DB, class StepBase>
struct LoadVTransposed {
  using Raw = TrFrag;
  uint32_t v_lane[DB];
  StepBase step_base;
  __device__ __forceinline__ LoadVTransposed(int lane, StepBase sb) : step_base(sb) {
    const int jb = lane >> 4, e = (lane >> 2) & 3, a = lane & 3;  // 16-lane block (column half jb & 1, key half jb >> 1), source lane 4 e + a
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      const int chunk = (4 * db + 2 * (jb & 1) + (a >> 1)) ^ (2 * e);
      v_lane[db] = (uint32_t)((4 * (jb >> 1) + e) * 128 + (chunk << 4) + (a & 1) * 8);
    }
  }
  __device__ __forceinline__ void operator()(int step, Raw (&f)[DB]) const {
    const uint32_t b = step_base(step);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      f[db].lo = lds_read_tr16_b64<0>(b + v_lane[db]);
      f[db].hi = lds_read_tr16_b64<1024>(b + v_lane[db]);
    }
  }
  __device__ __forceinline__ void ready(Raw (&a)[DB], Raw (&b)[DB], bf16x8 (&va)[DB], bf16x8 (&vb)[DB]) const {
    static_assert(DB == 2, "head_dim 64");
    lds_tr_wait(a[0], a[1], b[0], b[1]);
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      va[db] = tr_frag_value(a[db]);
      vb[db] = tr_frag_value(b[db]);
    }
  }
  __device__ __forceinline__ void ready(Raw (&a)[DB], bf16x8 (&va)[DB]) const {
    static_assert(DB == 2, "head_dim 64");
    lds_tr_wait(a[0], a[1]);
#pragma unroll
    for (int db = 0; db < DB; ++db) va[db] = tr_frag_value(a[db]);
  }
};

// V^T fragments by ordinary reads (`read(step, f)`: a tile that was transposed when it was written): nothing to wait for.
template <int DB, class Read>
struct LoadVPlain {
  using Raw = bf16x8;
  Read read;
  __device__ __forceinline__ explicit LoadVPlain(Read r) : read(r) {}
  __device__ __forceinline__ void operator()(int step, Raw (&f)[DB]) const { read(step, f); }
  __device__ __forceinline__ void ready(Raw (&a)[DB], Raw (&b)[DB], bf16x8 (&va)[DB], bf16x8 (&vb)[DB]) const {
#pragma unroll
    for (int db = 0; db < DB; ++db) {
      va[db] = a[db];
      vb[db] = b[db];
    }
  }
  __device__ __forceinline__ void ready(Raw (&a)[DB], bf16x8 (&va)[DB]) const {
#pragma unroll
    for (int db = 0; db < DB; ++db) va[db] = a[db];
  }
};

// Start values and mask of the logits of one query group.  The bias table lies in LDS as fp32 4-vectors
// R4[s] = (R[s..s+3]), R reversed and multiplied by log2 e, so that the biases of 4 consecutive keys are one
// ds_read_b128 at index sp(query) + qt(first key), read straight into the accumulators of K Q^T before its MFMAs:
// the bias costs neither an add nor a zero-fill.  The cyclic-shift mask is computed from the window position (only
// windows on the wrapped border of a shifted grid carry more than one region; -100 across regions); keys past the
// window (windows whose token count is not a multiple of 32) get -inf.
template <int WS_Y, int WS_X, bool HAS_BIAS>
struct WindowLogits {
  static constexpr int L = WS_Y * WS_X, LPAD = (L + 31) / 32 * 32, TBL = (2 * WS_Y - 1) * (2 * WS_X - 1);
  static constexpr float MASK_NEG = -100.0f * 1.4426950408889634f;  // the additive -100, in the exp2 domain
  const unsigned char* sB;
  const unsigned char* sB_lane;  // sB + (sp + 4 hi) * 16: the lane's part of every bias vector address
  int sp, hi;
  bool my, mx;
  int ry_q, rx_q, sy, sx;

  // qpos: the lane's query position in the window (already clamped to L - 1); my / mx: the window lies on the wrapped
  // border in y / x and the mask is on
  __device__ __forceinline__ WindowLogits(const unsigned char* bias_lds, int qpos, int hi_, bool my_, bool mx_, int sy_, int sx_)
      : sB(bias_lds), hi(hi_), my(my_), mx(mx_), sy(sy_), sx(sx_) {
    const int qiy = qpos / WS_X, qix = qpos % WS_X;
    sp = (TBL - 1) - (qiy + WS_Y - 1) * (2 * WS_X - 1) - qix - (WS_X - 1);
    sB_lane = sB + (sp + 4 * hi) * 16;
    ry_q = my ? (qiy < WS_Y - sy ? 1 : 2) : 0;
    rx_q = mx ? (qix < WS_X - sx ? 1 : 2) : 0;
  }
  __device__ __forceinline__ void init_acc(int kb, f32x16& a) const {
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      f32x4 bv = {0.f, 0.f, 0.f, 0.f};
      if (HAS_BIAS) {
        if (WS_X % 8 == 0 && LPAD == L) {
          // the lane's 4 keys start at column (8-aligned part) + 4 hi of their window row and never cross into the next
          // row: the index is the lane's own part, sp + 4 hi, plus a part that is a constant once kb is one (the
          // unrolled sweep): a per-lane base address and an immediate offset, no arithmetic per key group
          const int base = kb * 32 + g * 8;
          const int qt0 = (base / WS_X) * (2 * WS_X - 1) + (base % WS_X);
          bv = *reinterpret_cast<const f32x4*>(sB_lane + qt0 * 16);
        } else {
          const int key0 = kb * 32 + g * 8 + hi * 4;
          const int kk = ((LPAD == L) || key0 < L) ? key0 : 0;
          const int qt = (kk / WS_X) * (2 * WS_X - 1) + (kk % WS_X);
          bv = *reinterpret_cast<const f32x4*>(sB + (sp + qt) * 16);
        }
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) a[g * 4 + i] = bv[i];
    }
  }
  __device__ __forceinline__ void mask_block(int kb, f32x16& a) const {
    if (my || mx) {
      if (WS_X % 8 == 0 && LPAD == L) {
        // as in init_acc: the lane's 4 keys of a group lie in one window row, whose number is a constant once kb is; what
        // depends on the lane is whether column (8-aligned part) + 4 hi + i has wrapped around, one compare per key
        const int h4 = 4 * hi;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int base = kb * 32 + g * 8;
          const int kiy = base / WS_X, cx0 = base % WS_X;
          const bool ydiff = my && ((kiy < WS_Y - sy) != (ry_q == 1));
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool xdiff = mx && ((h4 < WS_X - sx - i - cx0) != (rx_q == 1));
            if (ydiff || xdiff) a[g * 4 + i] += MASK_NEG;
          }
        }
      } else {
#pragma unroll
        for (int g = 0; g < 4; ++g)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = kb * 32 + g * 8 + hi * 4 + i;
            const int kiy = key / WS_X, kix = key % WS_X;
            const int ry_k = my ? (kiy < WS_Y - sy ? 1 : 2) : 0;
            const int rx_k = mx ? (kix < WS_X - sx ? 1 : 2) : 0;
            if (ry_k != ry_q || rx_k != rx_q) a[g * 4 + i] += MASK_NEG;
          }
      }
    }
    if (LPAD != L) {
#pragma unroll
      for (int g = 0; g < 4; ++g)
        if (kb * 32 + g * 8 + hi * 4 >= L) {
#pragma unroll
          for (int i = 0; i < 4; ++i) a[g * 4 + i] = -INFINITY;
        }
    }
  }
};

// Build the head's bias column in LDS (see WindowLogits): R4[j - e][e] = R[j] = table[TBL - 1 - j][head] * log2 e.
// Tail components R4[s][e] with s + e >= TBL are never read by a valid key group.
template <int TBL>
__device__ __forceinline__ void build_bias_lds(unsigned char* sB, const uint16_t* table, int heads, int head, int tid, int nt) {
  float* sBf = reinterpret_cast<float*>(sB);
  for (int j = tid; j < TBL; j += nt) {
    const float r = bf16_bits_to_f32(table[(int64_t)(TBL - 1 - j) * heads + head]) * 1.4426950408889634f;
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (j - e >= 0) sBf[(j - e) * 4 + e] = r;
  }
}

// o = sum over the window's keys of P V and `sum` = the row sum of P, for the lane's query, P = softmax numerator.
// Fast path: ONE sweep over the key blocks with P = exp2(logit) and no row maximum (q carries scale * log2 e, the bias
// table log2 e, so the accumulators of K Q^T are the logits in the exp2 domain).  softmax does not depend on the
// subtracted constant; it only guards the range, and the range is checked afterwards: a row sum outside
// [2^-40, 2^100] (or not finite) in any lane sends the wave through the two-pass form with the row maximum (S^T
// recomputed block by block).  Per key block the MFMAs of S^T for block kb + 1 are issued ahead of the exp2 of block
// kb and those of P V for block kb after it, so that the matrix pipe runs while the VALU forms P; K fragments are read
// from LDS two blocks ahead, V^T fragments one block ahead.  Without a bias the first MFMA of an S^T block takes a
// literal zero as its C operand, and so does the first one of O^T: no accumulator is zero-filled by the VALU.
// `mid(kb)` is called at the start of key block kb (a hook for work a kernel wants issued inside the sweep).
template <int NQ, int KS, int DB, bool HAS_BIAS, class Logits, class LoadK, class LoadV, class Mid>
__device__ __forceinline__ void attention_sweep(const Logits& lg, const LoadK& load_k, const LoadV& load_v, const Mid& mid,
                                                const bf16x8 (&qf)[KS], f32x16 (&o)[DB], float& sum) {
  {
    const f32x16 zero16 = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    f32x16 acc2[2];
    bf16x8 kf[2][KS], vf[2][DB];
    typename LoadV::Raw vraw[2][DB];
    uint32_t pk[8];
    sum = 0.f;
    auto qk_block = [&](f32x16& acc, const bf16x8 (&kfr)[KS]) {
#pragma unroll
      for (int s2 = 0; s2 < KS; ++s2)
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kfr[s2], qf[s2], (!HAS_BIAS && s2 == 0) ? zero16 : acc, 0, 0, 0);
    };
    load_k(0, kf[0]);
    if (HAS_BIAS) lg.init_acc(0, acc2[0]);
    if (NQ > 1) {
      load_k(1, kf[1]);
      if (HAS_BIAS) lg.init_acc(1, acc2[1]);
    }
    __builtin_amdgcn_sched_barrier(0);
    qk_block(acc2[0], kf[0]);
#pragma unroll
    for (int kb = 0; kb < NQ; ++kb) {
      f32x16& a = acc2[kb & 1];
      __builtin_amdgcn_sched_barrier(0);
      mid(kb);
      // S^T of the next block first, the V^T reads of this block behind it: the compiler's wait for the bias vectors
      // and K fragments that those MFMAs consume (it does not know of the assembly reads and waits for "all") then
      // falls where only reads issued a block ago are outstanding, not on top of the V^T reads just issued
      if (kb + 1 < NQ) qk_block(acc2[(kb + 1) & 1], kf[(kb + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      load_v(2 * kb, vraw[0]);
      load_v(2 * kb + 1, vraw[1]);
      // Keep every accumulator of the S^T block just issued live across these reads.  Where the compiler can prove part
      // of it unused (keys past the window become -inf whatever the MFMA wrote) it would hand those registers to the
      // V^T reads, and it places no wait between an MFMA still writing a register and an assembly read returning into
      // it: the MFMA's late write would replace the V^T fragment.
      if (kb + 1 < NQ) asm volatile("" : "+v"(acc2[(kb + 1) & 1]));
      __builtin_amdgcn_sched_barrier(0);
      if (kb + 2 < NQ) load_k(kb + 2, kf[kb & 1]);
      lg.mask_block(kb, a);
#pragma unroll
      for (int h = 0; h < 8; ++h) {
        const float e0 = __builtin_amdgcn_exp2f(a[2 * h]);
        const float e1 = __builtin_amdgcn_exp2f(a[2 * h + 1]);
        pk[h] = pack_bf16x2(e0, e1);
        sum = dot2_ones(pk[h], sum);  // the row sum of what PV multiplies: the rounded values
      }
      __builtin_amdgcn_sched_barrier(0);
      load_v.ready(vraw[0], vraw[1], vf[0], vf[1]);
      // the accumulators of block kb are consumed: the bias of block kb + 2 goes straight into them
      if (HAS_BIAS && kb + 2 < NQ) lg.init_acc(kb + 2, a);
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2) {
        const u32x4 pw = {pk[4 * t2], pk[4 * t2 + 1], pk[4 * t2 + 2], pk[4 * t2 + 3]};
        const bf16x8 pf = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
        for (int db = 0; db < DB; ++db)
          o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[t2][db], pf, (kb == 0 && t2 == 0) ? zero16 : o[db], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    sum += __shfl_xor(sum, 32, 64);
  }
  const bool in_range = sum >= 0x1p-40f && sum <= 0x1p100f;  // false for NaN as well
  if (__builtin_amdgcn_ballot_w64(!in_range) != 0) {
    float mrow = -INFINITY;
#pragma unroll 1
    for (int pass = 0; pass < 2; ++pass) {
      if (pass == 1) {
        mrow = fmaxf(mrow, __shfl_xor(mrow, 32, 64));
        sum = 0.f;
#pragma unroll
        for (int db = 0; db < DB; ++db)
#pragma unroll
          for (int e = 0; e < 16; ++e) o[db][e] = 0.f;
      }
#pragma unroll 1
      for (int kb = 0; kb < NQ; ++kb) {
        f32x16 a;
        bf16x8 kf[KS];
        load_k(kb, kf);
        lg.init_acc(kb, a);
#pragma unroll
        for (int s2 = 0; s2 < KS; ++s2) a = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[s2], qf[s2], a, 0, 0, 0);
        lg.mask_block(kb, a);
        if (pass == 0) {
#pragma unroll
          for (int e = 0; e < 16; e += 2) mrow = fmaxf(fmaxf(mrow, a[e]), a[e + 1]);
        } else {
#pragma unroll
          for (int t2 = 0; t2 < 2; ++t2) {
            bf16x8 vf[DB];
            typename LoadV::Raw vraw[DB];
            load_v(2 * kb + t2, vraw);
            load_v.ready(vraw, vf);
            uint32_t pk[4];
#pragma unroll
            for (int h = 0; h < 4; ++h) {
              const int h2 = 4 * t2 + h;
              pk[h] = pack_bf16x2(__builtin_amdgcn_exp2f(a[2 * h2] - mrow), __builtin_amdgcn_exp2f(a[2 * h2 + 1] - mrow));
              sum = dot2_ones(pk[h], sum);
            }
            const u32x4 pw = {pk[0], pk[1], pk[2], pk[3]};
            const bf16x8 pf = __builtin_bit_cast(bf16x8, pw);
#pragma unroll
            for (int db = 0; db < DB; ++db) o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[db], pf, o[db], 0, 0, 0);
          }
        }
      }
    }
    sum += __shfl_xor(sum, 32, 64);
  }
}

// Normalise and store the lane's output row: o[db][4g + i] = O[query][32 db + 8 g + 4 hi + i].  The two lanes of a
// query (l31 and l31 + 32) each hold half of every 16-byte piece of the row; v_permlane32_swap on the pieces 2m and
// 2m + 1 gives the lower lane all of piece 2m and the upper lane all of piece 2m + 1: 32 contiguous bytes per row and
// instruction.  `op` points at element hi * 8 of the row's head slice.  DB * 2 store instructions, issued by every
// lane for which `valid` holds.
template <int DB>
__device__ __forceinline__ void store_attention_rows(uint16_t* op, const f32x16 (&o)[DB], float sum, bool valid) {
  const float inv = __builtin_amdgcn_rcpf(sum);
#pragma unroll
  for (int db = 0; db < DB; ++db)
#pragma unroll
    for (int m = 0; m < 2; ++m) {
      const int g0 = 2 * m, g1 = 2 * m + 1;
      const uint32_t x0 = pack_bf16x2(o[db][g0 * 4] * inv, o[db][g0 * 4 + 1] * inv);
      const uint32_t x1 = pack_bf16x2(o[db][g0 * 4 + 2] * inv, o[db][g0 * 4 + 3] * inv);
      const uint32_t y0 = pack_bf16x2(o[db][g1 * 4] * inv, o[db][g1 * 4 + 1] * inv);
      const uint32_t y1 = pack_bf16x2(o[db][g1 * 4 + 2] * inv, o[db][g1 * 4 + 3] * inv);
      const auto rx = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
      const auto ry = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
      if (valid) *reinterpret_cast<u32x4*>(op + db * 32 + m * 16) = u32x4{rx[0], ry[0], rx[1], ry[1]};
    }
}

}  // namespace aeris
