// Parameter block and LDS swizzle shared by the GEMM kernels.
#pragma once
#include "common.h"

namespace aeris {

struct GemmParams {
  const uint16_t* A;
  const uint16_t* W;
  void* C;
  const uint16_t* bias;
  const float* gate;
  const void* residual;
  int64_t M;
  int N;  // logical output columns
  int K;
  int64_t ldc;
  // output as column blocks ("head planes"): element (m, n) at (n / split) * plane_stride + m * split + n % split
  // instead of m * ldc + n; split = 0: plain row-major C.  split % 8 == 0, no residual in this mode.
  int split;
  int64_t plane_stride;
  int64_t gate_batch_stride;
  int64_t rows_per_batch;
  int tiles_n;
  // persistent kernel only: tile schedule
  int tiles_m;
  int total_tiles;
  int per_xcd;  // tiles in one XCD's contiguous chunk
  int bpx;      // workgroups per XCD
  // ceil(2^40 / (tiles per L2 group)): t / group size = (t * m_gsz) >> 40 for t < 2^24 (a tile is decoded several
  // times per tile and wave; a true division is some 25 vector ALU operations each time)
  uint64_t m_gsz;
  // row / rows_per_batch = (row * rpb_magic) >> rpb_shift, exact for row, rows_per_batch < 2^31 (magic = ceil(2^shift /
  // rows_per_batch), shift = 31 + ceil(log2 rows_per_batch)): the batch entry of a tile's rows, for the per-batch gate.
  // As 64-bit divisions these were some 400 scalar instructions per tile and wave, through the CU's one scalar unit.
  uint32_t rpb_magic;
  int rpb_shift;
  int act;
  int res_dtype;  // -1 none, AERIS_BF16, AERIS_F32
  int c_dtype;
  // output columns n < q_cols are multiplied by q_scale in fp32, after the bias and before the only rounding (the
  // query part of a qkv projection: softmax scale times log2(e)); q_cols = 0: none.  bf16 C without activation,
  // gate and residual only.
  float q_scale;
  int q_cols;
};

// offset of the group of columns starting at n (a group never straddles a column block) within its row, and the
// stride between rows, for either output layout
__device__ __forceinline__ int64_t c_col_off(const GemmParams& p, int n) {
  return p.split ? (int64_t)(n / p.split) * p.plane_stride + n % p.split : (int64_t)n;
}
__device__ __forceinline__ int64_t c_row_stride(const GemmParams& p) { return p.split ? (int64_t)p.split : p.ldc; }

__device__ __forceinline__ uint32_t swz_off(int row, int chunk) {
  // byte offset of 16-byte chunk `chunk` (0..7) of tile row `row` in a [rows][64] bf16 tile
  return (uint32_t)((row >> 1) * 256 + (((((row & 1) << 3) | chunk) ^ ((row >> 1) & 7)) << 4));
}

// 256x256 persistent kernel (gemm_persistent.hip); needs N % 4 == 0 and ldc % 4 == 0
hipError_t gemm_persistent_configure();
hipError_t gemm_persistent_launch(const GemmParams& p, hipStream_t stream);

}  // namespace aeris
