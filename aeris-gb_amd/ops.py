"""Tensor-level wrappers over the C ABI: check tensors, pass raw pointers and the current HIP stream.

torch is used for device memory and streams only; all arithmetic happens in libaeris_hip.so.
"""
from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch

from . import _lib as L

_DT = {torch.bfloat16: L.BF16, torch.float32: L.F32}


def _stream():
    return torch.cuda.current_stream().cuda_stream


# Optional per-launch timing (used by bench.py): HIP events recorded on the launch stream around each kernel.
_profile = None


def profile_begin():
    global _profile
    _profile = []


def profile_end():
    """-> list of (tag, algorithmic work, unit, milliseconds); synchronises."""
    global _profile
    rec, _profile = _profile or [], None
    torch.cuda.synchronize()
    return [(tag, work, unit, a.elapsed_time(b)) for tag, work, unit, a, b in rec]


class _timed:
    def __init__(self, tag, work, unit):
        self.on = _profile is not None
        if self.on:
            self.rec = [tag, work, unit, torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)]

    def __enter__(self):
        if self.on:
            self.rec[3].record()

    def __exit__(self, *exc):
        if self.on:
            self.rec[4].record()
            _profile.append(tuple(self.rec))


def gemm_uses_big_tiles(M, N, act=None):
    """Mirror of the tile choice in csrc/gemm.hip (256x256 tiles vs 128x128), used to label timings."""
    bn = 128 if act == "swiglu" else 256
    return M >= 256 and (N % bn == 0 or N >= 4 * bn) and ((M + 255) // 256) * ((N + bn - 1) // bn) >= 256 and N % 4 == 0


_WORKSPACE = {}
_WS_OWNER = {}  # key -> the stream whose work last used the buffer
_RETIRED = []  # outgrown buffers stay allocated: a captured HIP graph may still point into them


def workspace(tag: str, shape, dtype, device) -> torch.Tensor:
    """Reusable scratch tensor for an intermediate that never leaves the block (normalised tokens, qkv, attention
    output, MLP hidden).  One buffer per (tag, device, dtype), grown on demand and never freed, so eager calls and
    captured graphs share it instead of each holding a pool of their own (at batch 4 on the 720x1440 grid the four
    intermediates are 115 GB).

    Every model, layer and captured graph on the device shares these buffers, which is safe as long as their uses are
    ordered on one stream.  The buffer remembers the stream that used it last: a request from another stream is
    accepted only when that stream has no work pending (then the buffer changes hands), otherwise two streams would be
    writing one scratch area at the same time and this raises instead.  Calls made while a stream is being captured
    are not checked, and replays of a captured graph do not pass through here: a graph must not be replayed on one
    stream while model calls run on another."""
    n = 1
    for d in shape:
        n *= int(d)
    key = (tag, str(device), dtype)
    if not torch.cuda.is_current_stream_capturing():
        # (a capture queues no work and nothing may be queried while it runs: it neither checks nor takes the buffer)
        cur = torch.cuda.current_stream(device)
        owner = _WS_OWNER.get(key)
        if owner is not None and owner != cur and not owner.query():
            raise RuntimeError(f"workspace {tag!r} on {device} is in use by work pending on another stream: the block "
                               "intermediates are shared per device, run the models of one device on one stream "
                               "(or synchronise the other stream first)")
        _WS_OWNER[key] = cur
    buf = _WORKSPACE.get(key)
    if buf is None or buf.numel() < n:
        if buf is not None:
            _RETIRED.append(buf)
        buf = torch.empty(n, dtype=dtype, device=device)
        _WORKSPACE[key] = buf
    return buf[:n].view(*shape)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _dev(t: torch.Tensor, name: str, dtype=None):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (the HIP kernels have no CPU fallback)")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise RuntimeError(f"{name} must be {dtype}, got {t.dtype}")
    return t


# ------------------------------------------------------------------------------------------
# host-only index maps (no GPU needed)

def window_index_map(B, H, W, ws_y, ws_x, shift_y=0, shift_x=0) -> np.ndarray:
    if min(B, H, W, ws_y, ws_x) <= 0 or H % ws_y or W % ws_x:
        n = 1
    else:
        n = B * H * W
    out = np.empty(n, dtype=np.int64)
    L.call("aeris_window_index_map", B, H, W, ws_y, ws_x, shift_y, shift_x, out.ctypes.data)
    return out.reshape(B * (H // ws_y) * (W // ws_x), ws_y * ws_x)


def relative_position_index(ws_y, ws_x) -> np.ndarray:
    n = max(1, ws_y * ws_x)
    out = np.empty(n * n, dtype=np.int32)
    L.call("aeris_relative_position_index", ws_y, ws_x, out.ctypes.data)
    return out.reshape(n, n)


def shift_region_ids(H, W, ws_y, ws_x, shift_y, shift_x) -> np.ndarray:
    ok = min(H, W, ws_y, ws_x) > 0 and H % ws_y == 0 and W % ws_x == 0
    out = np.empty(H * W if ok else 1, dtype=np.int32)
    L.call("aeris_shift_region_ids", H, W, ws_y, ws_x, shift_y, shift_x, out.ctypes.data)
    return out.reshape((H // ws_y) * (W // ws_x), ws_y * ws_x)


# ------------------------------------------------------------------------------------------
# device ops

def window_attention(qkv: torch.Tensor, B: int, image_shape: Tuple[int, int], heads: int, head_dim: int,
                     window_size: Tuple[int, int], shift: Tuple[int, int] = (0, 0),
                     bias_table: Optional[torch.Tensor] = None, use_mask: bool = False,
                     scale: Optional[float] = None, out: Optional[torch.Tensor] = None,
                     head_planes: bool = False, q_prescaled: bool = False) -> torch.Tensor:
    """qkv bf16 [B*H*W, 3*heads*head_dim] (natural token order) -> bf16 [B*H*W, heads*head_dim].

    ``head_planes``: qkv is [3*heads, B*H*W, head_dim] instead (plane c*heads + h = part c of head h), the layout
    ``gemm_heads`` writes.  ``q_prescaled`` (head planes only): the q planes already hold q * scale * log2(e), as
    ``gemm_heads(..., q_scale=scale * LOG2E, q_planes=heads)`` writes them."""
    H, W = image_shape
    inner = heads * head_dim
    _dev(qkv, "qkv", torch.bfloat16)
    if qkv.numel() != B * H * W * 3 * inner:
        raise RuntimeError(f"qkv has {qkv.numel()} elements, expected {B}*{H}*{W}*3*{inner}")
    if head_planes and tuple(qkv.shape) != (3 * heads, B * H * W, head_dim):
        raise RuntimeError(f"qkv planes must be [{3 * heads}, {B * H * W}, {head_dim}], got {tuple(qkv.shape)}")
    if q_prescaled and not head_planes:
        raise RuntimeError("q_prescaled needs head_planes=True (the row-matrix entry point scales q itself)")
    if bias_table is not None:
        _dev(bias_table, "bias_table", torch.bfloat16)
        n = (2 * window_size[0] - 1) * (2 * window_size[1] - 1)
        if tuple(bias_table.shape) != (n, heads):
            raise RuntimeError(f"bias_table must be [{n}, {heads}], got {tuple(bias_table.shape)}")
    if out is None:
        out = torch.empty(B * H * W, inner, dtype=torch.bfloat16, device=qkv.device)
    else:
        _dev(out, "out", torch.bfloat16)
        if out.numel() != B * H * W * inner:
            raise RuntimeError("out has the wrong size")
    Lw = window_size[0] * window_size[1]
    with _timed("window_attention", 4.0 * B * H * W * Lw * inner, "flop"):
        if head_planes:
            L.call("aeris_window_attention_heads_fwd", qkv.data_ptr(), out.data_ptr(), _ptr(bias_table), B, H, W, heads,
                   head_dim, window_size[0], window_size[1], shift[0], shift[1], int(bool(use_mask)),
                   float(head_dim ** -0.5 if scale is None else scale), int(bool(q_prescaled)), B * H * W * head_dim,
                   _stream())
        else:
            L.call("aeris_window_attention_fwd", qkv.data_ptr(), out.data_ptr(), _ptr(bias_table), B, H, W, heads, head_dim,
                   window_size[0], window_size[1], shift[0], shift[1], int(bool(use_mask)),
                   float(head_dim ** -0.5 if scale is None else scale), _stream())
    return out


def qkv_attention_supported(K: int, heads: int, head_dim: int, window_size, image_shape) -> bool:
    """Whether the fused to_qkv + window attention kernel takes this shape (16x16 windows, head_dim 64, K % 128 == 0)."""
    H, W = image_shape
    return (tuple(window_size) == (16, 16) and head_dim == 64 and K % 128 == 0 and K >= 256 and H % 16 == 0 and W % 16 == 0
            and H * W * K * 2 < 0xFFFFFFF0 and 3 * heads * head_dim * K * 2 < 2 ** 31)


def qkv_attention_pack_bias(table: torch.Tensor, window_size) -> torch.Tensor:
    """The relative-position bias table [(2ws-1)^2, heads] bf16 in the form ``qkv_window_attention`` reads."""
    _dev(table, "bias_table", torch.bfloat16)
    heads = table.shape[1]
    n = int(L.lib().aeris_qkv_attention_bias_bytes(heads, window_size[0], window_size[1]))
    if n <= 0 or table.shape[0] != (2 * window_size[0] - 1) * (2 * window_size[1] - 1):
        raise RuntimeError(f"no fused kernel for windows {tuple(window_size)} / table {tuple(table.shape)}")
    out = torch.empty(n // 4, dtype=torch.float32, device=table.device)
    L.call("aeris_qkv_attention_prepare_bias", table.data_ptr(), heads, window_size[0], window_size[1], out.data_ptr(), _stream())
    return out


def qkv_window_attention(y: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], bias4: Optional[torch.Tensor], B: int,
                         image_shape: Tuple[int, int], heads: int, head_dim: int, window_size: Tuple[int, int],
                         shift: Tuple[int, int] = (0, 0), use_mask: bool = False, scale: Optional[float] = None,
                         out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y bf16 [B*H*W, K] -> attention output bf16 [B*H*W, heads*head_dim] with the to_qkv projection (w [3*inner, K],
    bias [3*inner] | None) inside the kernel; ``bias4`` from ``qkv_attention_pack_bias`` (None: no rel-pos bias)."""
    H, W = image_shape
    inner = heads * head_dim
    _dev(y, "y", torch.bfloat16)
    _dev(w, "w", torch.bfloat16)
    K = y.shape[-1]
    if y.numel() != B * H * W * K or tuple(w.shape) != (3 * inner, K):
        raise RuntimeError(f"y must hold {B}*{H}*{W} rows of {K}, w must be [{3 * inner}, {K}]")
    if bias is not None:
        _dev(bias, "bias", torch.bfloat16)
        if bias.numel() != 3 * inner:
            raise RuntimeError("bias has the wrong size")
    if bias4 is not None:
        _dev(bias4, "bias4", torch.float32)
    if out is None:
        out = torch.empty(B * H * W, inner, dtype=torch.bfloat16, device=y.device)
    else:
        _dev(out, "out", torch.bfloat16)
        if out.numel() != B * H * W * inner:
            raise RuntimeError("out has the wrong size")
    Lw = window_size[0] * window_size[1]
    S = B * H * W
    with _timed("qkv_window_attention", 2.0 * S * 3 * inner * K + 4.0 * S * Lw * inner, "flop"):
        L.call("aeris_qkv_window_attention_fwd", y.data_ptr(), w.data_ptr(), _ptr(bias), _ptr(bias4), out.data_ptr(), B, H, W,
               heads, head_dim, K, window_size[0], window_size[1], shift[0], shift[1], int(bool(use_mask)),
               float(head_dim ** -0.5 if scale is None else scale), _stream())
    return out


def _rowvec(t: Optional[torch.Tensor], name: str, d: int, B: int):
    """f32 [1|B, d] row vectors, rows possibly strided (a chunk of a wider matrix): -> (ptr, batch stride)."""
    if t is None:
        return None, 0
    if not t.is_cuda or t.dtype != torch.float32:
        raise RuntimeError(f"{name} must be a float32 GPU tensor")
    if t.dim() != 2 or t.shape[1] != d or t.stride(1) != 1 or t.shape[0] not in (1, B):
        raise RuntimeError(f"{name} must be [1, {d}] or [{B}, {d}] with unit column stride, got {tuple(t.shape)}")
    return t.data_ptr(), (t.stride(0) if t.shape[0] > 1 else 0)


def norm_modulate(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor] = None,
                  shift: Optional[torch.Tensor] = None, scale: Optional[torch.Tensor] = None, *, kind: str = "layernorm",
                  order: str = "norm_then_mod", eps: float = 1e-5, out: Optional[torch.Tensor] = None,
                  out_dtype=torch.bfloat16) -> torch.Tensor:
    """x [B, S, d] (bf16 | f32) -> y [B, S, d]; gamma/beta bf16 | f32 [d]; shift/scale f32 [1|B, d]."""
    _dev(x, "x")
    if x.dim() != 3:
        raise RuntimeError("x must be [B, S, d]")
    B, S, d = x.shape
    _dev(gamma, "gamma")
    if gamma.dtype not in _DT or gamma.numel() != d:
        raise RuntimeError("gamma must be bf16 or f32 [d]")
    if beta is not None:
        _dev(beta, "beta", gamma.dtype)
    sh_ptr, st1 = _rowvec(shift, "shift", d, B)
    sc_ptr, st2 = _rowvec(scale, "scale", d, B)
    if shift is not None and scale is not None and st1 != st2:
        raise RuntimeError("shift and scale must share their batch stride")
    if out is None:
        out = torch.empty(B, S, d, dtype=out_dtype, device=x.device)
    else:
        _dev(out, "out")
    with _timed("norm_modulate", float(B * S * d * (x.element_size() + out.element_size())), "byte"):
        L.call("aeris_norm_modulate_fwd", x.data_ptr(), _DT[x.dtype], out.data_ptr(), _DT[out.dtype], gamma.data_ptr(),
               _ptr(beta), _DT[gamma.dtype], sh_ptr, sc_ptr, max(st1, st2), B, S, d,
               L.NORM_LAYER if kind == "layernorm" else L.NORM_RMS,
               L.NORM_THEN_MOD if order == "norm_then_mod" else L.MOD_THEN_NORM, float(eps), _stream())
    return out


def output_stage_supported(N: int, d: int, B_mod: int, rows_per_batch: int) -> bool:
    return L.lib().aeris_output_stage_workspace_bytes(N, d, max(B_mod, 1)) > 0 and (B_mod <= 1 or rows_per_batch % 64 == 0)


def output_stage(x: torch.Tensor, gamma: torch.Tensor, beta: Optional[torch.Tensor], shift: Optional[torch.Tensor],
                 scale: Optional[torch.Tensor], head_w: torch.Tensor, *, kind: str = "rmsnorm", eps: float = 1e-5,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [B, S, d] (bf16 | f32) -> f32 [B, S, N] = head_w[N, d] applied to modulate(norm(x), shift, scale), one pass."""
    _dev(x, "x")
    if x.dim() != 3:
        raise RuntimeError("x must be [B, S, d]")
    B, S, d = x.shape
    _dev(gamma, "gamma")
    if gamma.dtype not in _DT or gamma.numel() != d:
        raise RuntimeError("gamma must be bf16 or f32 [d]")
    if beta is not None:
        _dev(beta, "beta", gamma.dtype)
    _dev(head_w, "head_w", torch.float32)
    N = head_w.shape[0]
    if head_w.shape[1] != d:
        raise RuntimeError(f"head_w must be [N, {d}]")
    sh_ptr, st1 = _rowvec(shift, "shift", d, B)
    sc_ptr, st2 = _rowvec(scale, "scale", d, B)
    if shift is not None and scale is not None and st1 != st2:
        raise RuntimeError("shift and scale must share their batch stride")
    stride = max(st1, st2)
    b_mod = B if (stride and B > 1) else 1
    need = L.lib().aeris_output_stage_workspace_bytes(N, d, b_mod)
    ws = workspace("output_stage", (max(need, 16),), torch.uint8, x.device)
    if out is None:
        out = torch.empty(B, S, N, dtype=torch.float32, device=x.device)
    else:
        _dev(out, "out", torch.float32)
    with _timed("output_stage", float(B * S * d * x.element_size() + B * S * N * 4), "byte"):
        L.call("aeris_output_stage_fwd", x.data_ptr(), _DT[x.dtype], gamma.data_ptr(), _ptr(beta), _DT[gamma.dtype], sh_ptr,
               sc_ptr, stride, head_w.data_ptr(), out.data_ptr(), B, S, N, d,
               L.NORM_LAYER if kind == "layernorm" else L.NORM_RMS, float(eps), ws.data_ptr(), ws.numel(), _stream())
    return out


_ACT = {None: L.ACT_NONE, "none": L.ACT_NONE, "gelu": L.ACT_GELU, "swiglu": L.ACT_SWIGLU, "silu": L.ACT_SILU}


def gemm(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, *, act: Optional[str] = None,
         gate: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None, rows_per_batch: int = 0,
         out: Optional[torch.Tensor] = None, out_dtype=torch.bfloat16) -> torch.Tensor:
    """out[M, N] = epilogue(a[M, K] @ w[N, K]^T); see aeris_gemm_fwd in include/aeris_hip.h."""
    _dev(a, "a", torch.bfloat16)
    _dev(w, "w", torch.bfloat16)
    K = a.shape[-1]
    M = a.numel() // K
    n_w = w.shape[0]
    if w.shape[1] != K:
        raise RuntimeError(f"w must be [N, {K}], got {tuple(w.shape)}")
    N = n_w // 2 if act == "swiglu" else n_w
    if bias is not None:
        _dev(bias, "bias", torch.bfloat16)
        if bias.numel() != n_w:
            raise RuntimeError("bias has the wrong size")
    nb = gate.shape[0] if gate is not None and gate.dim() == 2 else 1
    if nb > 1 and (rows_per_batch <= 0 or nb * rows_per_batch != M):
        raise RuntimeError("per-batch gate needs rows_per_batch with B * rows_per_batch == M")
    g_ptr, gstride = _rowvec(gate, "gate", N, nb)
    if out is None:
        out = torch.empty(*a.shape[:-1], N, dtype=out_dtype, device=a.device)
    else:
        _dev(out, "out")
        if out.numel() != M * N:
            raise RuntimeError("out has the wrong size")
    if residual is not None:
        _dev(residual, "residual")
        if residual.numel() != M * N:
            raise RuntimeError("residual has the wrong size")
    big = gemm_uses_big_tiles(M, N, act) and act != "silu"
    tag = "gemm_128x128"
    if big:  # one tag per instantiation of the persistent kernel ("plain": neither gate nor residual in the epilogue;
        # "res": bf16 output with a bf16 residual)
        res_bf16 = residual is not None and residual.dtype == torch.bfloat16 and out.dtype == torch.bfloat16
        tag = (f"gemm_256x256_{act or 'none'}_{'f32' if out.dtype == torch.float32 else 'bf16'}"
               + ("_plain" if gate is None and residual is None else "_res" if res_bf16 else ""))
    with _timed(tag, 2.0 * M * n_w * K, "flop"):
        L.call("aeris_gemm_fwd", a.data_ptr(), w.data_ptr(), out.data_ptr(), _ptr(bias), g_ptr, _ptr(residual), M, N, K,
               N, _ACT[act], _DT[residual.dtype] if residual is not None else 0, _DT[out.dtype], gstride,
               rows_per_batch if rows_per_batch > 0 else M, _stream())
    return out


LOG2E = 1.4426950408889634


def gemm_heads(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], head_dim: int,
               out: Optional[torch.Tensor] = None, q_scale: float = 1.0, q_planes: int = 0) -> torch.Tensor:
    """a[M, K] @ w[N, K]^T + bias as N / head_dim planes: bf16 [N / head_dim, M, head_dim] (see aeris_gemm_heads_fwd).
    The first ``q_planes`` planes are multiplied by ``q_scale`` in fp32 before the rounding to bf16."""
    _dev(a, "a", torch.bfloat16)
    _dev(w, "w", torch.bfloat16)
    K = a.shape[-1]
    M = a.numel() // K
    N = w.shape[0]
    if w.shape[1] != K:
        raise RuntimeError(f"w must be [N, {K}], got {tuple(w.shape)}")
    if bias is not None:
        _dev(bias, "bias", torch.bfloat16)
        if bias.numel() != N:
            raise RuntimeError(f"bias must have {N} elements")
    if head_dim <= 0 or N % head_dim:
        raise RuntimeError(f"N={N} is not a multiple of head_dim={head_dim}")
    if out is None:
        out = torch.empty(N // head_dim, M, head_dim, dtype=torch.bfloat16, device=a.device)
    else:
        _dev(out, "out", torch.bfloat16)
        if tuple(out.shape) != (N // head_dim, M, head_dim):
            raise RuntimeError("out has the wrong shape")
    big = gemm_uses_big_tiles(M, N, None)
    with _timed("gemm_256x256_none_bf16_plain" if big else "gemm_128x128", 2.0 * M * N * K, "flop"):
        L.call("aeris_gemm_heads_fwd", a.data_ptr(), w.data_ptr(), out.data_ptr(), _ptr(bias), M, N, K, head_dim,
               M * head_dim, float(q_scale), int(q_planes), _stream())
    return out


def modulation_linear(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, *, silu: bool = False,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y f32 [B, N] = act(x f32 [B, K] @ w[N, K]^T + bias)."""
    _dev(x, "x", torch.float32)
    _dev(w, "w")
    B, K = x.shape
    N = w.shape[0]
    if w.shape[1] != K or w.dtype not in _DT:
        raise RuntimeError("w must be bf16 or f32 [N, K]")
    if bias is not None:
        _dev(bias, "bias", w.dtype)
    if out is None:
        out = torch.empty(B, N, dtype=torch.float32, device=x.device)
    L.call("aeris_modulation_linear_fwd", x.data_ptr(), w.data_ptr(), _ptr(bias), out.data_ptr(), B, N, K, _DT[w.dtype],
           L.ACT_SILU if silu else L.ACT_NONE, _stream())
    return out


def timestep_embedding(t: torch.Tensor, dim: int, max_period: float = 10_000.0,
                       out: Optional[torch.Tensor] = None) -> torch.Tensor:
    _dev(t, "t", torch.float32)
    B = t.numel()
    if out is None:
        out = torch.empty(B, dim, dtype=torch.float32, device=t.device)
    L.call("aeris_timestep_embedding_fwd", t.data_ptr(), out.data_ptr(), B, dim, float(max_period), _stream())
    return out


def embed_prepare(x: torch.Tensor, ape: Optional[torch.Tensor], k_pad: int, out: Optional[torch.Tensor] = None,
                  split: bool = False):
    """bf16 [M, k_pad] = x f32 [M, C] (+ ape f32 [M_ape, C], row m % M_ape), zero padded; ``split``: [hi | lo | hi]."""
    _dev(x, "x", torch.float32)
    C = x.shape[-1]
    M = x.numel() // C
    m_ape = 0
    if ape is not None:
        _dev(ape, "ape", torch.float32)
        m_ape = ape.numel() // C
        if ape.shape[-1] != C or M % m_ape:
            raise RuntimeError("ape must be [M_ape, C] with M a multiple of M_ape")
    if out is None:
        out = torch.empty(M, k_pad, dtype=torch.bfloat16, device=x.device)
    L.call("aeris_embed_prepare_fwd", x.data_ptr(), _ptr(ape), out.data_ptr(), M, m_ape, C, k_pad, int(split), _stream())
    return out


def embed_concat(x0: torch.Tensor, div0: float, x1: torch.Tensor, ape: Optional[torch.Tensor], k_pad: int,
                 out: Optional[torch.Tensor] = None, split: bool = False):
    """bf16 [M, k_pad] = [x0 f32 [M, C0] / div0 | x1 f32 [M, C1]] (+ ape f32 [M_ape, C0 + C1]), zero padded;
    ``split``: the values three times as [hi | lo | hi]."""
    _dev(x0, "x0", torch.float32)
    _dev(x1, "x1", torch.float32)
    C0, C1 = x0.shape[-1], x1.shape[-1]
    M = x0.numel() // C0
    if x1.numel() // C1 != M:
        raise RuntimeError("x0 and x1 must have the same number of rows")
    m_ape = 0
    if ape is not None:
        _dev(ape, "ape", torch.float32)
        m_ape = ape.numel() // (C0 + C1)
        if ape.shape[-1] != C0 + C1 or M % m_ape:
            raise RuntimeError("ape must be [M_ape, C0 + C1] with M a multiple of M_ape")
    if out is None:
        out = torch.empty(M, k_pad, dtype=torch.bfloat16, device=x0.device)
    L.call("aeris_embed_concat_fwd", x0.data_ptr(), C0, float(div0), x1.data_ptr(), C1, _ptr(ape), out.data_ptr(), M,
           m_ape, k_pad, int(split), _stream())
    return out


def input_stage_supported(C: int, d: int) -> bool:
    """Whether the one-pass input embedding takes Linear(C -> d) (C <= 159 channels, d a multiple of 64)."""
    return int(L.lib().aeris_input_stage_weight_bytes(int(C), int(d))) > 0


def input_stage_pack_weight(w: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """The packed split-bf16 form of Linear(C -> d)'s f32 parameters that ``input_stage`` multiplies by."""
    _dev(w, "w", torch.float32)
    d, C = w.shape
    if bias is not None:
        _dev(bias, "bias", torch.float32)
        if bias.numel() != d:
            raise RuntimeError(f"bias must have {d} elements")
    nbytes = int(L.lib().aeris_input_stage_weight_bytes(C, d))
    if nbytes <= 0:
        raise RuntimeError(f"the one-pass input embedding does not take C = {C}, d = {d}")
    packed = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    L.call("aeris_input_stage_pack_weight", w.data_ptr(), _ptr(bias), packed.data_ptr(), C, d, _stream())
    return packed


def input_stage(x0: torch.Tensor, div0: float, x1: Optional[torch.Tensor], ape: Optional[torch.Tensor],
                packed_w: torch.Tensor, d: int, out_dtype: torch.dtype = torch.float32,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out [M, d] = ([x0 f32 [M, C0] / div0 | x1 f32 [M, C1]] + ape f32 [M_ape, C0 + C1]) W^T + b in one kernel, fp32
    accuracy; ``packed_w`` from ``input_stage_pack_weight``."""
    _dev(x0, "x0", torch.float32)
    C0 = x0.shape[-1]
    M = x0.numel() // C0
    C1 = 0
    if x1 is not None:
        _dev(x1, "x1", torch.float32)
        C1 = x1.shape[-1]
        if x1.numel() // C1 != M:
            raise RuntimeError("x0 and x1 must have the same number of rows")
    m_ape = 0
    if ape is not None:
        _dev(ape, "ape", torch.float32)
        m_ape = ape.numel() // (C0 + C1)
        if ape.shape[-1] != C0 + C1 or M % m_ape:
            raise RuntimeError("ape must be [M_ape, C0 + C1] with M a multiple of M_ape")
    need = int(L.lib().aeris_input_stage_weight_bytes(C0 + C1, d))
    if need <= 0 or packed_w.numel() * packed_w.element_size() != need:
        raise RuntimeError(f"packed_w does not fit C = {C0 + C1}, d = {d}")
    if out is None:
        out = torch.empty(M, d, dtype=out_dtype, device=x0.device)
    else:
        _dev(out, "out")
        if out.numel() != M * d or out.dtype not in (torch.float32, torch.bfloat16):
            raise RuntimeError("out must be f32 or bf16 [M, d]")
    with _timed("input_stage", float(M) * ((C0 + C1) * 4 * (2 if ape is not None else 1) + d * out.element_size()), "byte"):
        L.call("aeris_input_stage_fwd", x0.data_ptr(), C0, float(div0), _ptr(x1), C1, _ptr(ape), m_ape, packed_w.data_ptr(),
               out.data_ptr(), _DT[out.dtype], M, d, _stream())
    return out
