"""The entry point that allocates nothing: aeris_output_stage_noalloc_fwd against aeris_output_stage_fwd.

Called through the C ABI with raw pointers.  Both run the same kernels - one folds into the caller's workspace, the
other into the library's own scratch array - so the outputs have to be bit-identical, on a first call and on a
second, smaller one that reuses the array with the first call's contents still in it.
"""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _run(pkg, cuda, B, S, d, N, kind, mod_rows, seed):
    L = pkg._lib
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(B, S, d, generator=g).to(cuda)
    gamma, beta = (1 + 0.1 * torch.randn(d, generator=g)).to(cuda), (0.1 * torch.randn(d, generator=g)).to(cuda)
    w = (torch.randn(N, d, generator=g) / d ** 0.5).to(cuda)
    m = (0.3 * torch.randn(mod_rows, 2 * d, generator=g)).to(cuda)
    shift, scale = m[:, :d], m[:, d:]
    stride = 2 * d if mod_rows > 1 else 0
    kind_c = L.NORM_LAYER if kind == "layernorm" else L.NORM_RMS
    need = L.lib().aeris_output_stage_workspace_bytes(N, d, mod_rows)
    assert 0 < need <= 2 << 20
    ws = torch.empty(need, dtype=torch.uint8, device=cuda)
    want = torch.full((B, S, N), float("nan"), device=cuda)
    got = torch.full((B, S, N), float("nan"), device=cuda)
    stream = torch.cuda.current_stream().cuda_stream
    common = (x.data_ptr(), L.F32, gamma.data_ptr(), beta.data_ptr() if kind == "layernorm" else None, L.F32,
              shift.data_ptr(), scale.data_ptr(), stride, w.data_ptr())
    L.call("aeris_output_stage_fwd", *common, want.data_ptr(), B, S, N, d, kind_c, 1e-5, ws.data_ptr(), need, stream)
    before = torch.cuda.memory_allocated()
    L.call("aeris_output_stage_noalloc_fwd", *common, got.data_ptr(), B, S, N, d, kind_c, 1e-5, stream)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert bool(torch.isfinite(want).all())
    assert torch.equal(got, want), float((got - want).abs().max())
    return want


def test_noalloc_output_stage_matches_the_workspace_entry_point(pkg, cuda):
    big = _run(pkg, cuda, 2, 4096, 1536, 69, "layernorm", 2, 1)     # two modulation rows, 128 tiles
    small = _run(pkg, cuda, 1, 200, 512, 8, "rmsnorm", 1, 2)        # smaller in every dimension, ragged rows
    assert big.shape == (2, 4096, 69) and small.shape == (1, 200, 8)
    # beyond the array: refused with a message that names the limit, nothing launched
    L = pkg._lib
    p16 = 1 << 20
    rc = L.lib().aeris_output_stage_noalloc_fwd(p16, L.F32, p16, None, L.F32, p16, p16, 3072, p16, p16, 8, 128, 80, 1536,
                                                 L.NORM_RMS, 1e-6, None)
    assert rc == L.EUNSUPPORTED and "scratch array holds" in L.last_error()
