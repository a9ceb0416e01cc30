/*
 * aeris_hip.h - C ABI of libaeris_hip.so: gfx950 (MI355X) kernels for the shifted-window Swin
 * denoiser block of AERIS window-partitioned inference.
 *
 * The reference has no native code and no FFI: its boundary for this path is the torch.nn.Module
 * API of src/aeris_wp_inference/model.py.  Each entry point below replaces a sequence of
 * ATen / einops calls of that file (cited per function).  The Python modules of the package
 * keep the reference's class names, constructor arguments and state_dict keys and call these
 * functions through ctypes.
 *
 * Conventions
 *   - Every function returns 0 on success and a negative AERIS_E* code on failure;
 *     aeris_last_error() returns a thread-local description of the last failure.
 *   - Argument validation runs on the host before anything touches the GPU, so it is testable
 *     without a device.
 *   - All device pointers are borrowed for the duration of the enqueue.  The library allocates
 *     nothing, frees nothing and keeps no pointer.  Every launch is asynchronous on `stream`
 *     (a hipStream_t passed as void*; NULL = default stream).  No hidden synchronisation,
 *     so calls may be captured into a HIP graph.
 *   - "bf16" = bfloat16 bits in a uint16_t; row-major everywhere; token rows are the natural
 *     row-major lat x lon order n = Y*W + X (model.py:302).
 */
#ifndef AERIS_HIP_H
#define AERIS_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AERIS_OK 0
#define AERIS_EINVAL (-1)       /* bad argument (null pointer, non-positive size, misalignment) */
#define AERIS_EUNSUPPORTED (-2) /* shape outside what the kernels cover */
#define AERIS_ELAUNCH (-3)      /* HIP runtime reported an error */

/* element types of the tensors whose type may vary */
#define AERIS_BF16 0
#define AERIS_F32 1

/* norm kinds / modulation order (aeris_norm_modulate_fwd) */
#define AERIS_NORM_LAYER 0 /* (x-mean)*rsqrt(var+eps)*gamma+beta */
#define AERIS_NORM_RMS 1   /* x*rsqrt(mean(x^2)+eps)*gamma       */
#define AERIS_NORM_THEN_MOD 0 /* modulate(norm(x))  - model.py:426 */
#define AERIS_MOD_THEN_NORM 1 /* norm(modulate(x))  - model.py:400-401 */

/* GEMM epilogue activations (aeris_gemm_fwd) */
#define AERIS_ACT_NONE 0
#define AERIS_ACT_GELU 1   /* erf GELU 0.5 x (1 + erf(x / sqrt 2)), see the note at aeris_gemm_fwd */
#define AERIS_ACT_SWIGLU 2 /* W has 2*N rows [gate | up]; C = silu(gate)*up  (model.py:156-158) */
#define AERIS_ACT_SILU 3

int aeris_version(void);
const char* aeris_last_error(void);

/* One-time per-process set-up on the current device (kernel attribute configuration).
 * Optional: every launch entry point performs it lazily; call it before graph capture. */
int aeris_init(void);

/* ---- host-only index maps (test hooks; no GPU needed) ---------------------------------- */

/* Folded partition + cyclic-roll address table.  out[(b*nWy*nWx + wy*nWx + wx)*L + iy*ws_x + ix]
 * = b*H*W + ((wy*ws_y+iy+shift_y) mod H)*W + ((wx*ws_x+ix+shift_x) mod W).
 * Replaces: rearrange at model.py:302/307 composed with torch.roll at model.py:111-114.
 * This is the exact map the attention kernel uses for its loads and stores. */
int aeris_window_index_map(int B, int H, int W, int ws_y, int ws_x, int shift_y, int shift_x,
                           int64_t* out);

/* Swin-v1 relative-position index, out[p*L+q] (no reference counterpart; textbook definition). */
int aeris_relative_position_index(int ws_y, int ws_x, int32_t* out);

/* Region id (0..8) of position (iy,ix) of window (wy,wx) on the rolled grid, out[nW*L]
 * (the quantity the in-kernel shift mask compares; textbook Swin-v1 img_mask). */
int aeris_shift_region_ids(int H, int W, int ws_y, int ws_x, int shift_y, int shift_x,
                           int32_t* out);

/* ---- device entry points --------------------------------------------------------------- */

/* Fused windowed multi-head self-attention.
 *   qkv  bf16 [B*H*W, 3*heads*head_dim], columns ordered (c h d): q | k | v, head-major (model.py:300)
 *   out  bf16 [B*H*W, heads*head_dim], columns (h d) (model.py:307)
 *   bias_table bf16 [(2ws_y-1)(2ws_x-1), heads] or NULL
 *   use_mask != 0 adds the Swin-v1 cyclic-shift mask (-100 across regions) when a shift is non-zero
 * Window partition / reverse and the cyclic shift are folded into the load / store addresses.
 * Replaces model.py:300-307 (+ the swin_shift calls at model.py:471-475 on one device).
 * Supported: windows 8x8, 12x12, 16x16 with head_dim 32 or 64 (bias table and mask optional); without bias table and
 * mask any window of up to 4096 tokens with head_dim 64 or 128, which includes the reference's 60x60 windows and
 * head_dim 128 (model.py:22-27).  Anything else: AERIS_EUNSUPPORTED. */
int aeris_window_attention_fwd(const void* qkv, void* out, const void* bias_table, int B, int H, int W,
                               int heads, int head_dim, int ws_y, int ws_x, int shift_y, int shift_x,
                               int use_mask, float scale, void* stream);

/* The same with q, k, v as head planes: plane (c*heads + h) holds part c (q, k, v) of head h as bf16 [B*H*W, head_dim],
 * the planes plane_stride elements apart (what aeris_gemm_heads_fwd writes).  A window's keys are then runs of
 * ws_x * head_dim contiguous elements instead of head_dim-element pieces a whole qkv row apart: about 13 % faster at
 * 16x16 windows on the 720x1440 grid.  Same arithmetic, bit-identical output.  The layout is internal to this library: it
 * replaces the intermediate of model.py:299-302, which the reference never exposes.
 * q_prescaled != 0: the q planes already hold q * scale * log2(e), as aeris_gemm_heads_fwd writes them when it is given
 * q_scale = scale * log2(e): the factor of model.py:290 is then applied once, in fp32, before q's only rounding to bf16,
 * and the kernel uses q as it is (`scale` is ignored apart from its validity check). */
int aeris_window_attention_heads_fwd(const void* qkv_planes, void* out, const void* bias_table, int B, int H, int W,
                                     int heads, int head_dim, int ws_y, int ws_x, int shift_y, int shift_x,
                                     int use_mask, float scale, int q_prescaled, int64_t plane_stride, void* stream);

/* to_qkv projection and window attention in one kernel: q, k and v never leave the chip.
 *   y    bf16 [B*H*W, K]      the normalised tokens, natural (row-major lat x lon) order
 *   w    bf16 [3*heads*head_dim, K], rows ordered (c h d) like to_qkv.weight (model.py:284,300); qkv_bias bf16
 *        [3*heads*head_dim] or NULL
 *   bias4  the relative-position bias table in the form aeris_qkv_attention_prepare_bias writes
 *        (aeris_qkv_attention_bias_bytes(heads, ws_y, ws_x) bytes, to be refreshed when the table changes), or NULL
 *   out  bf16 [B*H*W, heads*head_dim]
 * One (window, head) at a time: the window's rows of y (gathered through the folded partition / shift index map) times
 * the head's 3*head_dim weight rows, bias added and q multiplied by scale * log2(e) in fp32, one rounding to bf16, then
 * the same softmax(q k^T + bias + mask) v as aeris_window_attention_heads_fwd from on-chip memory.  Replaces
 * model.py:299-307 (+ the swin_shift calls at model.py:471-475 on one device): the same result as aeris_gemm_heads_fwd
 * (with q_scale) followed by aeris_window_attention_heads_fwd (q_prescaled), bit for bit.
 * Built for 16x16 windows, head_dim 64, K % 128 == 0, K >= 256, H*W*K*2 < 2^32; anything else: AERIS_EUNSUPPORTED. */
int64_t aeris_qkv_attention_bias_bytes(int heads, int ws_y, int ws_x);
int aeris_qkv_attention_prepare_bias(const void* bias_table, int heads, int ws_y, int ws_x, void* out, void* stream);
int aeris_qkv_window_attention_fwd(const void* y, const void* w, const void* qkv_bias, const void* bias4, void* out,
                                   int B, int H, int W, int heads, int head_dim, int K, int ws_y, int ws_x,
                                   int shift_y, int shift_x, int use_mask, float scale, void* stream);

/* Row norm fused with noise-level modulation.
 *   x  [B*rows_per_batch, d] (x_dtype bf16|f32)  ->  y [B*rows_per_batch, d] (y_dtype bf16|f32)
 *   gamma [d]; beta [d] or NULL (both param_dtype bf16|f32); shift, scale f32 [B_mod, d] or NULL
 *   (gamma, beta, shift, scale 16-byte aligned and mod_batch_stride a multiple of 4: they are read 16 bytes at a time)
 *   (B_mod = 1 or B, given by mod_batch_stride: 0 = one row broadcast over the batch, otherwise the
 *   distance in elements between the rows of consecutive batch entries)
 * Replaces torch.nn.RMSNorm + modulate (model.py:121-125,400-401,426) / LayerNorm + modulate. */
int aeris_norm_modulate_fwd(const void* x, int x_dtype, void* y, int y_dtype, const void* gamma, const void* beta,
                            int param_dtype, const float* shift, const float* scale, int64_t mod_batch_stride,
                            int64_t B, int64_t rows_per_batch, int d, int kind, int order, float eps,
                            void* stream);

/* Output stage in one pass: out f32 [B*rows_per_batch, N] = head_w * modulate(norm(x), shift, scale)
 *   x [B*rows_per_batch, d] (x_dtype bf16|f32); gamma [d], beta [d] or NULL (param_dtype); shift, scale f32
 *   [B_mod, d] or NULL (mod_batch_stride as for aeris_norm_modulate_fwd); head_w f32 [N, d] (nn.Linear layout, no bias)
 *   kind: AERIS_NORM_LAYER | AERIS_NORM_RMS; the order is norm then modulate.
 * Replaces x.to(float32) -> norm -> modulate -> head of OutputStage.forward (model.py:421-429) at its fp32 accuracy
 * (bf16 MFMA on operands split into a bf16 head and remainder, fp32 accumulation) without writing the normalised
 * tokens anywhere.  workspace: device memory of at least aeris_output_stage_workspace_bytes(N, d, B_mod) bytes, 16-byte
 * aligned, borrowed for the call (the per-call fold of gamma, beta, shift, scale into the head weight lives there);
 * B_mod = B when shift / scale carry one row per batch entry (mod_batch_stride != 0 and B > 1), otherwise 1.
 * Supported: N <= 80, d % 64 == 0, and rows_per_batch % 64 == 0 when B_mod > 1; otherwise AERIS_EUNSUPPORTED (use
 * aeris_norm_modulate_fwd + aeris_gemm_fwd). */
int64_t aeris_output_stage_workspace_bytes(int N, int d, int B_mod);
int aeris_output_stage_fwd(const void* x, int x_dtype, const void* gamma, const void* beta, int param_dtype,
                           const float* shift, const float* scale, int64_t mod_batch_stride, const float* head_w,
                           float* out, int64_t B, int64_t rows_per_batch, int N, int d, int kind, float eps,
                           void* workspace, int64_t workspace_bytes, void* stream);

/* aeris_output_stage_fwd without the workspace argument, for callers that cannot allocate device memory (code under
 * HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  The
 * per-call fold lives in an array of 2 MiB inside the library (one copy per GPU, held until the process ends); the
 * call allocates and frees nothing.  Limit: aeris_output_stage_workspace_bytes(N, d, B_mod) <= 2 MiB (at N <= 80,
 * d = 1536: up to 4 modulation rows), otherwise AERIS_EUNSUPPORTED.  Same kernels and results as
 * aeris_output_stage_fwd.  Every call on a GPU uses that GPU's one array: calls that overlap in time on one GPU
 * (two streams, two threads) race; order them on one stream.  The array's address is looked up on aeris_init() or
 * on the first call per device, which must happen outside any stream capture. */
int aeris_output_stage_noalloc_fwd(const void* x, int x_dtype, const void* gamma, const void* beta, int param_dtype,
                                   const float* shift, const float* scale, int64_t mod_batch_stride,
                                   const float* head_w, float* out, int64_t B, int64_t rows_per_batch, int N, int d,
                                   int kind, float eps, void* stream);

/* C[M,N] = epilogue(A[M,K] * W[N,K]^T).
 *   A bf16 [M,K] (lda = K); W bf16 [N,K] ([2N,K] for SWIGLU); bias bf16 [N] ([2N] for SWIGLU) or NULL
 *   epilogue: v = acc + bias; v = act(v); if gate: v *= gate[b, n]; if residual: v += residual[m, n]
 *   gate f32 [B_mod, N] or NULL (gate_batch_stride as above, rows_per_batch rows of C per batch entry)
 *   residual [M, N] (res_dtype) or NULL, may alias C;  C [M, ldc] (c_dtype), ldc >= N
 * Replaces nn.Linear at model.py:153-154,284-285,342,418 and the gate/residual elementwise passes
 * at model.py:400-401.  Requires K % 64 == 0.
 * AERIS_ACT_GELU is the erf form in both tile kernels, evaluated to the accuracy of the output type.  bf16 C from
 * the 256x256-tile kernel (M >= 256 and at least 256 tiles, N a multiple of 256 or >= 1024): a polynomial on the
 * clamp [-3.5, 3.5], |error| <= 2.0e-4 |x| for x >= -3.5 (a tenth of half a bf16 ulp) and the constant -8.1e-4 below
 * -3.5, where the exact value lies between -8.1e-4 and 0.  Every other case (f32 C, or the 128x128-tile kernel that
 * takes small and ragged problems): erf to 1.5e-7 absolute.  The two agree to within one bf16 ulp of the result for
 * x >= -1; which one runs depends on the shape only, never on the data. */
int aeris_gemm_fwd(const void* A, const void* W, void* C, const void* bias, const float* gate,
                   const void* residual, int64_t M, int N, int K, int64_t ldc, int act, int res_dtype,
                   int c_dtype, int64_t gate_batch_stride, int64_t rows_per_batch, void* stream);

/* C = A[M,K] * W[N,K]^T + bias written as N / head_dim planes of bf16 [M, head_dim], plane j = columns
 * [j*head_dim, (j+1)*head_dim), the planes plane_stride elements apart (>= M * head_dim, multiple of 8).
 * The to_qkv Linear (model.py:284,299) writing the layout aeris_window_attention_heads_fwd reads; the rearrange at
 * model.py:300 ("(c h d) -> c h d") is this split.  Requires K % 64 == 0, head_dim % 8 == 0, N % head_dim == 0.
 * The first q_planes planes (the query part; 0 = none) are multiplied by q_scale in fp32 after the bias and before the
 * rounding to bf16: with q_scale = head_dim^-0.5 * log2(e) this is the `q * self.scale` of model.py:290 in the exp2
 * domain, and aeris_window_attention_heads_fwd takes such planes with q_prescaled = 1. */
int aeris_gemm_heads_fwd(const void* A, const void* W, void* C, const void* bias, int64_t M, int N, int K,
                         int head_dim, int64_t plane_stride, float q_scale, int q_planes, void* stream);

/* y[b, n] = act(sum_k x[b,k] * W[n,k] + bias[n]);  x f32 [B,K], W bf16|f32 [N,K], bias same type or NULL,
 * y f32 [B,N].  The two Linear layers of ModulationLinear (model.py:311-325) with SiLU in between. */
int aeris_modulation_linear_fwd(const float* x, const void* W, const void* bias, float* y, int B, int N,
                                int K, int w_dtype, int act, void* stream);

/* Sinusoidal noise-level embedding [sin | cos], t f32 [B] (device) -> emb f32 [B, dim]  (model.py:127-143). */
int aeris_timestep_embedding_fwd(const float* t, float* emb, int B, int dim, float max_period, void* stream);

/* A-operand preparation for the input embedding: out bf16 [M, K_pad] = (x f32 [M, C] + ape f32 [M_ape, C] or NULL),
 * zero padded from C to K_pad columns; ape row = m % M_ape.  (model.py:350-352)
 * split != 0: the C values v are written as [hi | lo | hi | 1 | 1], hi = bf16(v), lo = bf16(v - hi), zero padded from
 * 3 C + 2 to K_pad columns.  With the weight laid out [W_hi | W_hi | W_lo | b_hi | b_lo] along K the bf16 GEMM returns
 * v W^T + b to about 2^-16 relative: the reference computes this Linear in fp32 (model.py:352). */
int aeris_embed_prepare_fwd(const float* x, const float* ape, void* out, int64_t M, int64_t M_ape, int C,
                            int K_pad, int split, void* stream);

/* The same with the sampler's channel concatenation folded in: out bf16 [M, K_pad] =
 * ([x0 f32 [M, C0] / div0 | x1 f32 [M, C1]] + ape f32 [M_ape, C0 + C1] or NULL), zero padded.  x0 is the noised state
 * (divided by sigma_data), x1 the conditioning channels: torch.cat([x_t / sigma_d, conditioning], dim=2) of
 * inference.py:160 followed by model.py:350-352, without materialising the concatenated tensor. */
int aeris_embed_concat_fwd(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape, void* out,
                           int64_t M, int64_t M_ape, int K_pad, int split, void* stream);

/* Input embedding in one pass (model.py:346-356; inference.py:160 for the two-part input):
 *   out [M, d] = ([x0 f32 [M, C0] / div0 | x1 f32 [M, C1]] + ape f32 [M_ape, C0 + C1] or NULL) W^T + b
 * at the accuracy of the reference's fp32 Linear (inputs and weight each split into bf16 head + remainder, three bf16
 * MFMA products summed in fp32; about 2^-16 relative), without an [M, K] operand matrix in memory.  x1 may be NULL
 * with C1 = 0; ape row = m % M_ape; out is f32 or bf16 (out_dtype).  C0 + C1 <= 159, d a multiple of 64, and
 * M_ape >= 64 when ape is given; other shapes return AERIS_EUNSUPPORTED (use aeris_embed_prepare_fwd / aeris_embed_concat_fwd + aeris_gemm_fwd).
 * The weight is packed once per parameter value: aeris_input_stage_weight_bytes(C, d) bytes (0 if the shape is not
 * supported), filled by aeris_input_stage_pack_weight from W f32 [d, C] and b f32 [d] (or NULL). */
int64_t aeris_input_stage_weight_bytes(int C, int d);
int aeris_input_stage_pack_weight(const float* W, const float* bias, void* packed, int C, int d, void* stream);
int aeris_input_stage_fwd(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape,
                          int64_t M_ape, const void* packed_w, void* out, int out_dtype, int64_t M, int d,
                          void* stream);

#ifdef __cplusplus
}
#endif
#endif /* AERIS_HIP_H */
