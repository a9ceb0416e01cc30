// Internal launch interface between the C-ABI layer (api.hip) and the kernel translation units.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "../../include/aeris_hip.h"

namespace aeris {

// one-time hipFuncSetAttribute(MaxDynamicSharedMemorySize) for every kernel that needs > 64 KB LDS
hipError_t gemm_configure_all();
hipError_t attention_configure_all();

hipError_t gemm_launch(const void* A, const void* W, void* C, const void* bias, const float* gate,
                       const void* residual, int64_t M, int N, int K, int64_t ldc, int act, int res_dtype,
                       int c_dtype, int64_t gate_batch_stride, int64_t rows_per_batch, int split, int64_t plane_stride,
                       float q_scale, int q_cols, hipStream_t stream);

// returns hipErrorInvalidValue when (ws_y, ws_x, head_dim) has no instantiation.  q / k / v of (token, head) start at
// part * part_stride + head * head_stride + token * tok_stride (elements) for part = 0, 1, 2
bool attention_supported(int ws_y, int ws_x, int head_dim);
// streaming kernel (window_attention_stream.hip): any window of up to 4096 tokens, head_dim 64 / 128, no bias, no mask
bool attention_stream_supported(int ws_y, int ws_x, int head_dim, bool has_bias, bool use_mask);
hipError_t attention_stream_configure_all();
hipError_t attention_stream_launch(const void* qkv, void* out, int B, int H, int W, int heads, int head_dim, int ws_y,
                                   int ws_x, int shift_y, int shift_x, float scale, int q_prescaled, int64_t tok_stride,
                                   int64_t head_stride, int64_t part_stride, hipStream_t stream);
hipError_t attention_launch(const void* qkv, void* out, const void* bias_table, int B, int H, int W, int heads,
                            int head_dim, int ws_y, int ws_x, int shift_y, int shift_x, int use_mask, float scale,
                            int q_prescaled, int64_t tok_stride, int64_t head_stride, int64_t part_stride,
                            hipStream_t stream);

// to_qkv projection fused with window attention (qkv_window_attention.hip): 16x16 windows, head_dim 64, K % 128 == 0
bool qkv_attention_supported(int ws_y, int ws_x, int head_dim, int K, int64_t tokens_per_image);
int64_t qkv_attention_bias_bytes(int heads);
hipError_t qkv_attention_configure();
hipError_t qkv_attention_bias_launch(const void* table, float* out, int heads, hipStream_t stream);
hipError_t qkv_attention_launch(const void* y, const void* w, const void* bias, const float* bias4, void* out, int B, int H,
                                int W, int heads, int K, int shift_y, int shift_x, int use_mask, float scale,
                                hipStream_t stream);

bool norm_supported(int d);
hipError_t norm_modulate_launch(const void* x, int x_dtype, void* y, int y_dtype, const void* gamma, const void* beta,
                                int param_dtype, const float* shift, const float* scale, int64_t mod_batch_stride, int64_t B,
                                int64_t rows_per_batch, int d, int kind, int order, float eps, hipStream_t stream);

// fused output stage (output_stage.hip): norm -> modulate -> head in one pass; N <= 80, d % 64 == 0
bool output_stage_supported(int N, int d);
int64_t output_stage_workspace_bytes(int N, int d, int B_mod);
// the library's own scratch array for the entry point that allocates nothing: capacity in bytes, and its device
// address on the current device (hipErrorNotReady when it has not been looked up yet and lookup_allowed is false)
int64_t output_stage_scratch_capacity();
hipError_t output_stage_scratch(void** ptr, bool lookup_allowed);
hipError_t output_stage_launch(const void* x, int x_dtype, const void* gamma, const void* beta, int param_dtype,
                               const float* shift, const float* scale, int64_t mod_batch_stride, const float* head_w,
                               float* out, int64_t B, int64_t rows_per_batch, int N, int d, int kind, float eps,
                               void* workspace, hipStream_t stream);

hipError_t modulation_linear_launch(const float* x, const void* W, const void* bias, float* y, int B, int N, int K,
                                    int w_dtype, int act, hipStream_t stream);
hipError_t timestep_embedding_launch(const float* t, float* emb, int B, int dim, float max_period, hipStream_t stream);
hipError_t embed_prepare_launch(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape, void* out,
                                int64_t M, int64_t M_ape, int K_pad, int split, hipStream_t stream);


// Fused input embedding (input_stage.hip): tokens = ([x0 / div0 | x1] + ape) W^T + b at fp32 accuracy
bool input_stage_supported(int C, int d);
int64_t input_stage_weight_bytes(int C, int d);
hipError_t input_stage_configure();
hipError_t input_stage_pack_weight_launch(const float* W, const float* bias, void* packed, int C, int d, hipStream_t stream);
hipError_t input_stage_launch(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape, int64_t M_ape,
                              const void* packed, void* out, int out_dtype, int64_t M, int d, hipStream_t stream);

}  // namespace aeris
