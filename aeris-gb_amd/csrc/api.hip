// C ABI of libaeris_hip.so: argument validation (host only, before any GPU call), error reporting,
// one-time kernel attribute set-up, and the host-side index-map test hooks.
#include <hip/hip_runtime.h>
#include <cstdarg>
#include <cstdio>
#include <atomic>
#include <mutex>

#include "kernels.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int hip_fail(hipError_t e, const char* what) {
  return fail(AERIS_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
}

std::once_flag g_init_once;
std::atomic<bool> g_init_done{false};
hipError_t g_init_status = hipSuccess;

// One-time kernel attribute set-up.  A launch entry point performs it lazily, but never inside a stream capture:
// hipFuncSetAttribute is not a stream operation and must not run while `stream` is being recorded into a graph.
int ensure_init(void* stream = nullptr, bool from_launch = false) {
  if (from_launch && !g_init_done.load(std::memory_order_acquire)) {
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(reinterpret_cast<hipStream_t>(stream), &st) == hipSuccess && st != hipStreamCaptureStatusNone)
      return fail(AERIS_EINVAL, "the library is not initialised and the stream is being captured: call aeris_init() "
                                "before the capture begins");
  }
  std::call_once(g_init_once, [] {
    g_init_status = aeris::gemm_configure_all();
    if (g_init_status == hipSuccess) g_init_status = aeris::attention_configure_all();
    if (g_init_status == hipSuccess) g_init_status = aeris::attention_stream_configure_all();
    if (g_init_status == hipSuccess) g_init_status = aeris::input_stage_configure();
    if (g_init_status == hipSuccess) g_init_status = aeris::qkv_attention_configure();
    g_init_done.store(true, std::memory_order_release);
  });
  if (g_init_status == hipSuccess && !from_launch) {
    // aeris_init() itself: also resolve, for the device that is current now, the address of the scratch array
    // that aeris_output_stage_noalloc_fwd uses (once per device; a later device gets it on its own aeris_init
    // or on its first call of that entry point)
    void* p = nullptr;
    hipError_t e = aeris::output_stage_scratch(&p, true);
    if (e != hipSuccess) return hip_fail(e, "aeris_init (hipGetSymbolAddress of the scratch array)");
  }
  if (g_init_status != hipSuccess) return hip_fail(g_init_status, "aeris_init (hipFuncSetAttribute)");
  return AERIS_OK;
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

int check_window_geometry(int B, int H, int W, int ws_y, int ws_x, int shift_y, int shift_x) {
  if (B <= 0 || H <= 0 || W <= 0 || ws_y <= 0 || ws_x <= 0)
    return fail(AERIS_EINVAL, "window geometry: B, H, W, ws_y, ws_x must be positive (got %d %d %d %d %d)", B, H, W, ws_y, ws_x);
  if (H % ws_y || W % ws_x)
    return fail(AERIS_EINVAL, "window geometry: grid %dx%d is not a multiple of window %dx%d", H, W, ws_y, ws_x);
  if (shift_y < 0 || shift_x < 0 || shift_y >= ws_y || shift_x >= ws_x)
    return fail(AERIS_EINVAL, "window geometry: shift (%d,%d) must lie in [0, window)", shift_y, shift_x);
  return AERIS_OK;
}

}  // namespace

extern "C" {

int aeris_version(void) { return 1; }

const char* aeris_last_error(void) { return g_err; }

int aeris_init(void) { return ensure_init(); }

int aeris_window_index_map(int B, int H, int W, int ws_y, int ws_x, int shift_y, int shift_x, int64_t* out) {
  if (!out) return fail(AERIS_EINVAL, "aeris_window_index_map: out is NULL");
  if (int rc = check_window_geometry(B, H, W, ws_y, ws_x, shift_y, shift_x)) return rc;
  const int nWy = H / ws_y, nWx = W / ws_x;
  int64_t o = 0;
  for (int b = 0; b < B; ++b)
    for (int wy = 0; wy < nWy; ++wy)
      for (int wx = 0; wx < nWx; ++wx) {
        // same arithmetic as token_row() of the attention kernel
        const int y0 = wy * ws_y + shift_y, x0 = wx * ws_x + shift_x;
        for (int pos = 0; pos < ws_y * ws_x; ++pos) {
          int Y = y0 + pos / ws_x, X = x0 + pos % ws_x;
          if (Y >= H) Y -= H;
          if (X >= W) X -= W;
          out[o++] = (int64_t)b * H * W + (int64_t)Y * W + X;
        }
      }
  return AERIS_OK;
}

int aeris_relative_position_index(int ws_y, int ws_x, int32_t* out) {
  if (!out) return fail(AERIS_EINVAL, "aeris_relative_position_index: out is NULL");
  if (ws_y <= 0 || ws_x <= 0) return fail(AERIS_EINVAL, "aeris_relative_position_index: window must be positive");
  const int L = ws_y * ws_x;
  for (int p = 0; p < L; ++p)
    for (int q = 0; q < L; ++q) {
      // same closed form as the kernel: (iy_p - iy_q + ws_y - 1) * (2 ws_x - 1) + (ix_p - ix_q + ws_x - 1)
      const int dy = p / ws_x - q / ws_x + ws_y - 1;
      const int dx = p % ws_x - q % ws_x + ws_x - 1;
      out[p * L + q] = dy * (2 * ws_x - 1) + dx;
    }
  return AERIS_OK;
}

int aeris_shift_region_ids(int H, int W, int ws_y, int ws_x, int shift_y, int shift_x, int32_t* out) {
  if (!out) return fail(AERIS_EINVAL, "aeris_shift_region_ids: out is NULL");
  if (int rc = check_window_geometry(1, H, W, ws_y, ws_x, shift_y, shift_x)) return rc;
  const int nWy = H / ws_y, nWx = W / ws_x;
  int64_t o = 0;
  for (int wy = 0; wy < nWy; ++wy)
    for (int wx = 0; wx < nWx; ++wx) {
      const bool my = shift_y > 0 && wy == nWy - 1;
      const bool mx = shift_x > 0 && wx == nWx - 1;
      for (int iy = 0; iy < ws_y; ++iy)
        for (int ix = 0; ix < ws_x; ++ix) {
          // same predicate as the kernel's mask pass
          const int ry = my ? (iy < ws_y - shift_y ? 1 : 2) : 0;
          const int rx = mx ? (ix < ws_x - shift_x ? 1 : 2) : 0;
          out[o++] = 3 * ry + rx;
        }
    }
  return AERIS_OK;
}

static int window_attention_impl(const char* who, const void* qkv, void* out, const void* bias_table, int B, int H, int W,
                                 int heads, int head_dim, int ws_y, int ws_x, int shift_y, int shift_x, int use_mask,
                                 float scale, int q_prescaled, int64_t tok_stride, int64_t head_stride, int64_t part_stride,
                                 void* stream) {
  if (!qkv || !out) return fail(AERIS_EINVAL, "%s: qkv/out is NULL", who);
  if (!aligned16(qkv) || !aligned16(out)) return fail(AERIS_EINVAL, "%s: qkv/out must be 16-byte aligned", who);
  if (heads <= 0 || head_dim <= 0) return fail(AERIS_EINVAL, "%s: heads/head_dim must be positive", who);
  if (int rc = check_window_geometry(B, H, W, ws_y, ws_x, shift_y, shift_x)) return rc;
  if (!(scale > 0.f)) return fail(AERIS_EINVAL, "%s: scale must be positive", who);
  if ((int64_t)B * H * W > 0x7fffffffLL || tok_stride > 0x7fffffffLL)
    return fail(AERIS_EUNSUPPORTED, "%s: more than 2^31-1 tokens or elements per token row", who);
  const bool small = aeris::attention_supported(ws_y, ws_x, head_dim);
  const bool masked = use_mask && (shift_y > 0 || shift_x > 0);
  if (!small && !aeris::attention_stream_supported(ws_y, ws_x, head_dim, bias_table != nullptr, masked))
    return fail(AERIS_EUNSUPPORTED,
                "%s: no kernel for window %dx%d head_dim %d%s (built: 8x8, 12x12, 16x16 with head_dim "
                "32 or 64, bias and mask optional; any window of up to 4096 tokens with head_dim 64 or 128 without bias and mask)",
                who, ws_y, ws_x, head_dim, bias_table ? " with a bias table" : (masked ? " with the shift mask" : ""));
  const int64_t units = (int64_t)B * (H / ws_y) * (W / ws_x) * heads;
  if (units > 0x7fffffffLL || (!small && (units + 8) * (((int64_t)ws_y * ws_x + 127) / 128) > 0x7fffffffLL))
    return fail(AERIS_EUNSUPPORTED, "%s: more than 2^31-1 workgroups", who);
  if (int rc = ensure_init(stream, true)) return rc;
  if (!small) {
    hipError_t e = aeris::attention_stream_launch(qkv, out, B, H, W, heads, head_dim, ws_y, ws_x, shift_y, shift_x, scale,
                                                  q_prescaled, tok_stride, head_stride, part_stride,
                                                  reinterpret_cast<hipStream_t>(stream));
    if (e != hipSuccess) return hip_fail(e, "window attention launch (streaming kernel)");
    return AERIS_OK;
  }
  hipError_t e = aeris::attention_launch(qkv, out, bias_table, B, H, W, heads, head_dim, ws_y, ws_x, shift_y, shift_x,
                                         use_mask, scale, q_prescaled, tok_stride, head_stride, part_stride,
                                         reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "window attention launch");
  return AERIS_OK;
}

int aeris_window_attention_fwd(const void* qkv, void* out, const void* bias_table, int B, int H, int W, int heads,
                               int head_dim, int ws_y, int ws_x, int shift_y, int shift_x, int use_mask, float scale,
                               void* stream) {
  const int64_t inner = (int64_t)heads * head_dim;
  return window_attention_impl("aeris_window_attention_fwd", qkv, out, bias_table, B, H, W, heads, head_dim, ws_y, ws_x,
                               shift_y, shift_x, use_mask, scale, 0, 3 * inner, head_dim, inner, stream);
}

int aeris_window_attention_heads_fwd(const void* qkv_planes, void* out, const void* bias_table, int B, int H, int W, int heads,
                                     int head_dim, int ws_y, int ws_x, int shift_y, int shift_x, int use_mask, float scale,
                                     int q_prescaled, int64_t plane_stride, void* stream) {
  if (head_dim > 0 && B > 0 && H > 0 && W > 0 && (plane_stride < (int64_t)B * H * W * head_dim || plane_stride % 8))
    return fail(AERIS_EINVAL, "aeris_window_attention_heads_fwd: plane_stride must be a multiple of 8 and at least B*H*W*head_dim");
  return window_attention_impl("aeris_window_attention_heads_fwd", qkv_planes, out, bias_table, B, H, W, heads, head_dim, ws_y,
                               ws_x, shift_y, shift_x, use_mask, scale, q_prescaled ? 1 : 0, head_dim, plane_stride,
                               (int64_t)heads * plane_stride, stream);
}

int64_t aeris_qkv_attention_bias_bytes(int heads, int ws_y, int ws_x) {
  if (heads <= 0 || !aeris::qkv_attention_supported(ws_y, ws_x, 64, 256, 1)) return 0;
  return aeris::qkv_attention_bias_bytes(heads);
}

int aeris_qkv_attention_prepare_bias(const void* bias_table, int heads, int ws_y, int ws_x, void* out, void* stream) {
  if (!bias_table || !out) return fail(AERIS_EINVAL, "aeris_qkv_attention_prepare_bias: bias_table/out is NULL");
  if (heads <= 0) return fail(AERIS_EINVAL, "aeris_qkv_attention_prepare_bias: heads must be positive");
  if (!aeris::qkv_attention_supported(ws_y, ws_x, 64, 256, 1))
    return fail(AERIS_EUNSUPPORTED, "aeris_qkv_attention_prepare_bias: only 16x16 windows are built (got %dx%d)", ws_y, ws_x);
  if (!aligned16(out)) return fail(AERIS_EINVAL, "aeris_qkv_attention_prepare_bias: out must be 16-byte aligned");
  hipError_t e = aeris::qkv_attention_bias_launch(bias_table, reinterpret_cast<float*>(out), heads, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_qkv_attention_prepare_bias launch");
  return AERIS_OK;
}

int aeris_qkv_window_attention_fwd(const void* y, const void* w, const void* qkv_bias, const void* bias4, void* out, int B,
                                   int H, int W, int heads, int head_dim, int K, int ws_y, int ws_x, int shift_y, int shift_x,
                                   int use_mask, float scale, void* stream) {
  const char* who = "aeris_qkv_window_attention_fwd";
  if (!y || !w || !out) return fail(AERIS_EINVAL, "%s: y/w/out is NULL", who);
  if (!aligned16(y) || !aligned16(w) || !aligned16(out) || (bias4 && !aligned16(bias4)))
    return fail(AERIS_EINVAL, "%s: y/w/out/bias4 must be 16-byte aligned", who);
  if (qkv_bias && (reinterpret_cast<uintptr_t>(qkv_bias) & 7u)) return fail(AERIS_EINVAL, "%s: qkv_bias must be 8-byte aligned", who);
  if (heads <= 0 || head_dim <= 0 || K <= 0) return fail(AERIS_EINVAL, "%s: heads, head_dim, K must be positive", who);
  if (int rc = check_window_geometry(B, H, W, ws_y, ws_x, shift_y, shift_x)) return rc;
  if (!(scale > 0.f)) return fail(AERIS_EINVAL, "%s: scale must be positive", who);
  if (!aeris::qkv_attention_supported(ws_y, ws_x, head_dim, K, (int64_t)H * W))
    return fail(AERIS_EUNSUPPORTED,
                "%s: built for 16x16 windows, head_dim 64, K a multiple of 128 and at least 256, H*W*K*2 < 2^32 (got %dx%d, head_dim %d, "
                "K %d, H*W %lld): use aeris_gemm_heads_fwd + aeris_window_attention_heads_fwd", who, ws_y, ws_x, head_dim, K,
                (long long)H * W);
  if ((int64_t)3 * heads * head_dim * K * 2 >= (int64_t(1) << 31))
    return fail(AERIS_EUNSUPPORTED, "%s: the to_qkv weight must be smaller than 2 GiB", who);
  if ((int64_t)B * (H / ws_y) * (W / ws_x) * heads > 0x7fffffffLL || (int64_t)B * H * W > 0x7fffffffLL)
    return fail(AERIS_EUNSUPPORTED, "%s: more than 2^31-1 (window, head) units or tokens", who);
  if (int rc = ensure_init(stream, true)) return rc;
  hipError_t e = aeris::qkv_attention_launch(y, w, qkv_bias, reinterpret_cast<const float*>(bias4), out, B, H, W, heads, K, shift_y,
                                             shift_x, use_mask, scale, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_qkv_window_attention_fwd launch");
  return AERIS_OK;
}

int aeris_norm_modulate_fwd(const void* x, int x_dtype, void* y, int y_dtype, const void* gamma, const void* beta,
                            int param_dtype, const float* shift, const float* scale, int64_t mod_batch_stride, int64_t B,
                            int64_t rows_per_batch, int d, int kind, int order, float eps, void* stream) {
  if (!x || !y || !gamma) return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: x/y/gamma is NULL");
  if (!aligned16(x) || !aligned16(y)) return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: x/y must be 16-byte aligned");
  if (B <= 0 || rows_per_batch <= 0) return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: B and rows_per_batch must be positive");
  if ((x_dtype != AERIS_BF16 && x_dtype != AERIS_F32) || (y_dtype != AERIS_BF16 && y_dtype != AERIS_F32) ||
      (param_dtype != AERIS_BF16 && param_dtype != AERIS_F32))
    return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: dtype must be AERIS_BF16 or AERIS_F32");
  if (kind != AERIS_NORM_LAYER && kind != AERIS_NORM_RMS) return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: unknown norm kind %d", kind);
  if (order != AERIS_NORM_THEN_MOD && order != AERIS_MOD_THEN_NORM) return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: unknown order %d", order);
  if (mod_batch_stride < 0) return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: negative mod_batch_stride");
  // the per-column parameters are read 16 bytes at a time
  if (!aligned16(gamma) || (beta && !aligned16(beta)) || (shift && !aligned16(shift)) || (scale && !aligned16(scale)) ||
      ((shift || scale) && (mod_batch_stride & 3)))
    return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: gamma/beta/shift/scale must be 16-byte aligned, mod_batch_stride a multiple of 4");
  if (!(eps >= 0.f)) return fail(AERIS_EINVAL, "aeris_norm_modulate_fwd: eps must be non-negative");
  if (!aeris::norm_supported(d)) return fail(AERIS_EUNSUPPORTED, "aeris_norm_modulate_fwd: d=%d (need d %% 8 == 0 and d <= 6144)", d);
  hipError_t e = aeris::norm_modulate_launch(x, x_dtype, y, y_dtype, gamma, beta, param_dtype, shift, scale, mod_batch_stride, B,
                                             rows_per_batch, d, kind, order, eps, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_norm_modulate_fwd launch");
  return AERIS_OK;
}

int64_t aeris_output_stage_workspace_bytes(int N, int d, int B_mod) {
  if (B_mod <= 0 || !aeris::output_stage_supported(N, d)) return 0;
  return aeris::output_stage_workspace_bytes(N, d, B_mod);
}

namespace {
// shared argument checks of the output-stage entry points; sets *B_mod to the number of modulation rows in use
int check_output_stage(const char* who, const void* x, int x_dtype, const void* gamma, const void* beta, int param_dtype,
                       const float* shift, const float* scale, int64_t mod_batch_stride, const float* head_w, float* out,
                       int64_t B, int64_t rows_per_batch, int N, int d, int kind, float eps, int* B_mod) {
  if (!x || !gamma || !head_w || !out) return fail(AERIS_EINVAL, "%s: x/gamma/head_w/out is NULL", who);
  if (!aligned16(x) || !aligned16(out) || !aligned16(head_w)) return fail(AERIS_EINVAL, "%s: x/out/head_w must be 16-byte aligned", who);
  if (B <= 0 || rows_per_batch <= 0) return fail(AERIS_EINVAL, "%s: B and rows_per_batch must be positive", who);
  if ((x_dtype != AERIS_BF16 && x_dtype != AERIS_F32) || (param_dtype != AERIS_BF16 && param_dtype != AERIS_F32))
    return fail(AERIS_EINVAL, "%s: dtype must be AERIS_BF16 or AERIS_F32", who);
  if (kind != AERIS_NORM_LAYER && kind != AERIS_NORM_RMS) return fail(AERIS_EINVAL, "%s: unknown norm kind %d", who, kind);
  if (mod_batch_stride < 0) return fail(AERIS_EINVAL, "%s: negative mod_batch_stride", who);
  if (!(eps >= 0.f)) return fail(AERIS_EINVAL, "%s: eps must be non-negative", who);
  if (N <= 0 || d <= 0) return fail(AERIS_EINVAL, "%s: N and d must be positive", who);
  if (!aeris::output_stage_supported(N, d))
    return fail(AERIS_EUNSUPPORTED, "%s: N=%d, d=%d (need N <= 80 and d a multiple of 64)", who, N, d);
  const bool batched = (shift || scale) && mod_batch_stride != 0 && B > 1;
  if (batched && rows_per_batch % 64)
    return fail(AERIS_EUNSUPPORTED, "%s: with one modulation row per batch entry rows_per_batch=%lld must be a multiple of 64",
                who, (long long)rows_per_batch);
  if (batched && B > 0x7fffffffLL / 1024) return fail(AERIS_EUNSUPPORTED, "%s: too many batch entries", who);
  if ((B * rows_per_batch + 63) / 64 > 0x7fffffffLL) return fail(AERIS_EUNSUPPORTED, "%s: too many rows", who);
  *B_mod = batched ? (int)B : 1;
  return AERIS_OK;
}
}  // namespace

int aeris_output_stage_fwd(const void* x, int x_dtype, const void* gamma, const void* beta, int param_dtype,
                           const float* shift, const float* scale, int64_t mod_batch_stride, const float* head_w, float* out,
                           int64_t B, int64_t rows_per_batch, int N, int d, int kind, float eps, void* workspace,
                           int64_t workspace_bytes, void* stream) {
  int B_mod = 1;
  if (int rc = check_output_stage("aeris_output_stage_fwd", x, x_dtype, gamma, beta, param_dtype, shift, scale,
                                  mod_batch_stride, head_w, out, B, rows_per_batch, N, d, kind, eps, &B_mod))
    return rc;
  const int64_t need = aeris::output_stage_workspace_bytes(N, d, B_mod);
  if (!workspace || !aligned16(workspace) || workspace_bytes < need)
    return fail(AERIS_EINVAL, "aeris_output_stage_fwd: workspace must be 16-byte aligned and hold %lld bytes (got %lld)",
                (long long)need, (long long)workspace_bytes);
  hipError_t e = aeris::output_stage_launch(x, x_dtype, gamma, beta, param_dtype, shift, scale, mod_batch_stride, head_w, out,
                                            B, rows_per_batch, N, d, kind, eps, workspace, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_output_stage_fwd launch");
  return AERIS_OK;
}

int aeris_output_stage_noalloc_fwd(const void* x, int x_dtype, const void* gamma, const void* beta, int param_dtype,
                                   const float* shift, const float* scale, int64_t mod_batch_stride, const float* head_w,
                                   float* out, int64_t B, int64_t rows_per_batch, int N, int d, int kind, float eps,
                                   void* stream) {
  const char* who = "aeris_output_stage_noalloc_fwd";
  int B_mod = 1;
  if (int rc = check_output_stage(who, x, x_dtype, gamma, beta, param_dtype, shift, scale, mod_batch_stride, head_w, out, B,
                                  rows_per_batch, N, d, kind, eps, &B_mod))
    return rc;
  const int64_t need = aeris::output_stage_workspace_bytes(N, d, B_mod), cap = aeris::output_stage_scratch_capacity();
  if (need > cap)
    return fail(AERIS_EUNSUPPORTED,
                "%s: the fold of %d modulation row(s) at N=%d, d=%d needs %lld bytes, the library's scratch array holds "
                "%lld: use aeris_output_stage_fwd with a workspace",
                who, B_mod, N, d, (long long)need, (long long)cap);
  // the array's address on this device: cached after the first look-up, which must not fall inside a capture
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  const bool capturing =
      hipStreamIsCapturing(reinterpret_cast<hipStream_t>(stream), &st) == hipSuccess && st != hipStreamCaptureStatusNone;
  void* ws = nullptr;
  hipError_t e = aeris::output_stage_scratch(&ws, !capturing);
  if (e == hipErrorNotReady)
    return fail(AERIS_EINVAL, "%s: first use on this device while the stream is being captured: call aeris_init() "
                              "with this device current before the capture begins", who);
  if (e != hipSuccess) return hip_fail(e, "aeris_output_stage_noalloc_fwd (scratch address)");
  e = aeris::output_stage_launch(x, x_dtype, gamma, beta, param_dtype, shift, scale, mod_batch_stride, head_w, out, B,
                                 rows_per_batch, N, d, kind, eps, ws, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_output_stage_noalloc_fwd launch");
  return AERIS_OK;
}

int aeris_gemm_fwd(const void* A, const void* W, void* C, const void* bias, const float* gate, const void* residual,
                   int64_t M, int N, int K, int64_t ldc, int act, int res_dtype, int c_dtype,
                   int64_t gate_batch_stride, int64_t rows_per_batch, void* stream) {
  if (!A || !W || !C) return fail(AERIS_EINVAL, "aeris_gemm_fwd: A/W/C is NULL");
  if (M <= 0 || N <= 0 || K <= 0) return fail(AERIS_EINVAL, "aeris_gemm_fwd: M, N, K must be positive");
  if (!aligned16(A) || !aligned16(W) || !aligned16(C) || (residual && !aligned16(residual)))
    return fail(AERIS_EINVAL, "aeris_gemm_fwd: A/W/C/residual must be 16-byte aligned");
  if (K % 64) return fail(AERIS_EUNSUPPORTED, "aeris_gemm_fwd: K=%d must be a multiple of 64", K);
  if (ldc < N) return fail(AERIS_EINVAL, "aeris_gemm_fwd: ldc < N");
  if (act < AERIS_ACT_NONE || act > AERIS_ACT_SILU) return fail(AERIS_EINVAL, "aeris_gemm_fwd: unknown activation %d", act);
  if (c_dtype != AERIS_BF16 && c_dtype != AERIS_F32) return fail(AERIS_EINVAL, "aeris_gemm_fwd: bad c_dtype");
  if (residual && res_dtype != AERIS_BF16 && res_dtype != AERIS_F32) return fail(AERIS_EINVAL, "aeris_gemm_fwd: bad res_dtype");
  if (gate && gate_batch_stride && rows_per_batch <= 0)
    return fail(AERIS_EINVAL, "aeris_gemm_fwd: rows_per_batch must be positive with a per-batch gate");
  if (gate_batch_stride < 0) return fail(AERIS_EINVAL, "aeris_gemm_fwd: negative gate_batch_stride");
  if ((int64_t)((M + 127) / 128) * ((N + 63) / 64) > 0x7fffffffLL) return fail(AERIS_EUNSUPPORTED, "aeris_gemm_fwd: too many tiles");
  if (int rc = ensure_init(stream, true)) return rc;
  hipError_t e = aeris::gemm_launch(A, W, C, bias, gate, residual, M, N, K, ldc, act, res_dtype, c_dtype,
                                    gate_batch_stride, rows_per_batch, 0, 0, 1.0f, 0, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_gemm_fwd launch");
  return AERIS_OK;
}

int aeris_gemm_heads_fwd(const void* A, const void* W, void* C, const void* bias, int64_t M, int N, int K, int head_dim,
                         int64_t plane_stride, float q_scale, int q_planes, void* stream) {
  if (!A || !W || !C) return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: A/W/C is NULL");
  if (M <= 0 || N <= 0 || K <= 0) return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: M, N, K must be positive");
  if (!aligned16(A) || !aligned16(W) || !aligned16(C)) return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: A/W/C must be 16-byte aligned");
  if (K % 64) return fail(AERIS_EUNSUPPORTED, "aeris_gemm_heads_fwd: K=%d must be a multiple of 64", K);
  if (head_dim <= 0 || head_dim % 8) return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: head_dim=%d must be a positive multiple of 8", head_dim);
  if (N % head_dim) return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: N=%d is not a multiple of head_dim=%d", N, head_dim);
  if (plane_stride < M * head_dim || plane_stride % 8)
    return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: plane_stride must be a multiple of 8 and at least M * head_dim");
  if ((int64_t)((M + 127) / 128) * ((N + 63) / 64) > 0x7fffffffLL) return fail(AERIS_EUNSUPPORTED, "aeris_gemm_heads_fwd: too many tiles");
  if (q_planes < 0 || (int64_t)q_planes * head_dim > N)
    return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: q_planes=%d must lie in [0, N / head_dim]", q_planes);
  if (q_planes > 0 && !(q_scale > 0.f && q_scale < 3.0e38f)) return fail(AERIS_EINVAL, "aeris_gemm_heads_fwd: q_scale must be positive and finite");
  if (int rc = ensure_init(stream, true)) return rc;
  hipError_t e = aeris::gemm_launch(A, W, C, bias, nullptr, nullptr, M, N, K, N, AERIS_ACT_NONE, -1, AERIS_BF16, 0, M, head_dim,
                                    plane_stride, q_planes > 0 ? q_scale : 1.0f, q_planes * head_dim,
                                    reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_gemm_heads_fwd launch");
  return AERIS_OK;
}

int aeris_modulation_linear_fwd(const float* x, const void* W, const void* bias, float* y, int B, int N, int K,
                                int w_dtype, int act, void* stream) {
  if (!x || !W || !y) return fail(AERIS_EINVAL, "aeris_modulation_linear_fwd: x/W/y is NULL");
  if (B <= 0 || N <= 0 || K <= 0) return fail(AERIS_EINVAL, "aeris_modulation_linear_fwd: B, N, K must be positive");
  if (K % 8) return fail(AERIS_EUNSUPPORTED, "aeris_modulation_linear_fwd: K=%d must be a multiple of 8", K);
  if (!aligned16(x) || !aligned16(W)) return fail(AERIS_EINVAL, "aeris_modulation_linear_fwd: x/W must be 16-byte aligned");
  if (w_dtype != AERIS_BF16 && w_dtype != AERIS_F32) return fail(AERIS_EINVAL, "aeris_modulation_linear_fwd: bad w_dtype");
  if (act != AERIS_ACT_NONE && act != AERIS_ACT_SILU) return fail(AERIS_EINVAL, "aeris_modulation_linear_fwd: act must be NONE or SILU");
  hipError_t e = aeris::modulation_linear_launch(x, W, bias, y, B, N, K, w_dtype, act, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_modulation_linear_fwd launch");
  return AERIS_OK;
}

int aeris_timestep_embedding_fwd(const float* t, float* emb, int B, int dim, float max_period, void* stream) {
  if (!t || !emb) return fail(AERIS_EINVAL, "aeris_timestep_embedding_fwd: t/emb is NULL");
  if (B <= 0 || dim <= 0 || dim % 2) return fail(AERIS_EINVAL, "aeris_timestep_embedding_fwd: B > 0 and even dim > 0 required");
  if (!(max_period > 1.f)) return fail(AERIS_EINVAL, "aeris_timestep_embedding_fwd: max_period must exceed 1");
  hipError_t e = aeris::timestep_embedding_launch(t, emb, B, dim, max_period, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_timestep_embedding_fwd launch");
  return AERIS_OK;
}

int aeris_embed_prepare_fwd(const float* x, const float* ape, void* out, int64_t M, int64_t M_ape, int C, int K_pad,
                            int split, void* stream) {
  if (!x || !out) return fail(AERIS_EINVAL, "aeris_embed_prepare_fwd: x/out is NULL");
  if (M <= 0 || C <= 0 || K_pad < (split ? 3 * (int64_t)C + 2 : (int64_t)C) || K_pad % 64)
    return fail(AERIS_EINVAL, "aeris_embed_prepare_fwd: need M > 0, C > 0, K_pad >= C (3 C + 2 with split), K_pad %% 64 == 0");
  if (ape && M_ape <= 0) return fail(AERIS_EINVAL, "aeris_embed_prepare_fwd: M_ape must be positive when ape is given");
  if (!aligned16(out)) return fail(AERIS_EINVAL, "aeris_embed_prepare_fwd: out must be 16-byte aligned");
  hipError_t e = aeris::embed_prepare_launch(x, C, 1.0f, nullptr, 0, ape, out, M, M_ape > 0 ? M_ape : 1, K_pad, split,
                                             reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_embed_prepare_fwd launch");
  return AERIS_OK;
}

int aeris_embed_concat_fwd(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape, void* out,
                           int64_t M, int64_t M_ape, int K_pad, int split, void* stream) {
  if (!x0 || !x1 || !out) return fail(AERIS_EINVAL, "aeris_embed_concat_fwd: x0/x1/out is NULL");
  if (M <= 0 || C0 <= 0 || C1 <= 0 || K_pad < (split ? 3 * ((int64_t)C0 + C1) + 2 : (int64_t)C0 + C1) || K_pad % 64)
    return fail(AERIS_EINVAL, "aeris_embed_concat_fwd: need M > 0, C0 > 0, C1 > 0, K_pad >= C0 + C1 (3 (C0 + C1) + 2 with split), K_pad %% 64 == 0");
  if (!(div0 != 0.0f)) return fail(AERIS_EINVAL, "aeris_embed_concat_fwd: div0 must be non-zero");
  if (ape && M_ape <= 0) return fail(AERIS_EINVAL, "aeris_embed_concat_fwd: M_ape must be positive when ape is given");
  if (!aligned16(out)) return fail(AERIS_EINVAL, "aeris_embed_concat_fwd: out must be 16-byte aligned");
  hipError_t e = aeris::embed_prepare_launch(x0, C0, div0, x1, C1, ape, out, M, M_ape > 0 ? M_ape : 1, K_pad, split,
                                             reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_embed_concat_fwd launch");
  return AERIS_OK;
}

int64_t aeris_input_stage_weight_bytes(int C, int d) {
  if (!aeris::input_stage_supported(C, d)) return 0;
  return aeris::input_stage_weight_bytes(C, d);
}

int aeris_input_stage_pack_weight(const float* W, const float* bias, void* packed, int C, int d, void* stream) {
  if (!W || !packed) return fail(AERIS_EINVAL, "aeris_input_stage_pack_weight: W/packed is NULL");
  if (!aeris::input_stage_supported(C, d))
    return fail(AERIS_EUNSUPPORTED, "aeris_input_stage_pack_weight: need 1 <= C <= 159 and d a multiple of 64 (got C = %d, d = %d)", C, d);
  if (!aligned16(packed)) return fail(AERIS_EINVAL, "aeris_input_stage_pack_weight: packed must be 16-byte aligned");
  hipError_t e = aeris::input_stage_pack_weight_launch(W, bias, packed, C, d, reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_input_stage_pack_weight launch");
  return AERIS_OK;
}

int aeris_input_stage_fwd(const float* x0, int C0, float div0, const float* x1, int C1, const float* ape, int64_t M_ape,
                          const void* packed_w, void* out, int out_dtype, int64_t M, int d, void* stream) {
  if (!x0 || !packed_w || !out) return fail(AERIS_EINVAL, "aeris_input_stage_fwd: x0/packed_w/out is NULL");
  if (M <= 0 || C0 <= 0 || C1 < 0 || (x1 == nullptr) != (C1 == 0))
    return fail(AERIS_EINVAL, "aeris_input_stage_fwd: need M > 0, C0 > 0, and x1 given exactly when C1 > 0");
  if (!aeris::input_stage_supported(C0 + C1, d))
    return fail(AERIS_EUNSUPPORTED, "aeris_input_stage_fwd: need C0 + C1 <= 159 and d a multiple of 64 (got C = %d, d = %d)",
                C0 + C1, d);
  if (!(div0 != 0.0f)) return fail(AERIS_EINVAL, "aeris_input_stage_fwd: div0 must be non-zero");
  if (ape && M_ape <= 0) return fail(AERIS_EINVAL, "aeris_input_stage_fwd: M_ape must be positive when ape is given");
  if (ape && (M_ape < 64 || M_ape > 0x7fffff00))
    return fail(AERIS_EUNSUPPORTED, "aeris_input_stage_fwd: a positional encoding of fewer than 64 rows (or 2^31 and more) is not "
                                    "taken (got %lld)", (long long)M_ape);
  if (out_dtype != AERIS_F32 && out_dtype != AERIS_BF16) return fail(AERIS_EINVAL, "aeris_input_stage_fwd: out_dtype must be f32 or bf16");
  if (!aligned16(out) || !aligned16(packed_w)) return fail(AERIS_EINVAL, "aeris_input_stage_fwd: out and packed_w must be 16-byte aligned");
  if (int rc = ensure_init(stream, true)) return rc;
  hipError_t e = aeris::input_stage_launch(x0, C0, div0, x1, C1, ape, M_ape, packed_w, out, out_dtype, M, d,
                                           reinterpret_cast<hipStream_t>(stream));
  if (e != hipSuccess) return hip_fail(e, "aeris_input_stage_fwd launch");
  return AERIS_OK;
}

}  // extern "C"
