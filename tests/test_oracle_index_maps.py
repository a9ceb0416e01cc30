"""Pin the oracle's integer maps against library routines (einops, torch.roll) and explicit loops.

The reference expresses these maps as einops patterns (src/aeris_wp_inference/model.py:300,302,307)
composed with torch.roll (model.py:111-114); einops and torch are used here as libraries.
"""
import numpy as np
import pytest
import torch
from einops import rearrange
from hypothesis import given, settings, strategies as st

import oracle

CASES = [(1, 4, 8, 2, 4, 0, 0), (1, 4, 8, 2, 4, 1, 2), (2, 6, 6, 3, 2, 1, 1), (1, 32, 64, 8, 8, 4, 4),
         (1, 24, 36, 12, 12, 6, 6), (3, 32, 48, 16, 16, 8, 8)]


def _einops_map(B, H, W, wy, wx, sy, sx):
    tok = torch.arange(B * H * W, dtype=torch.int64).reshape(B, H * W, 1)
    g = tok.reshape(B, H, W, 1)
    g = torch.roll(g, shifts=(-sy, -sx), dims=(1, 2))  # shift-up of the residual stream before an odd layer
    flat = g.reshape(B, H * W, 1, 1)  # [b, n, h=1, d=1]
    win = rearrange(flat, "b (wcl_y ws_y wcl_x ws_x) h d -> (b wcl_y wcl_x) h (ws_y ws_x) d",
                    wcl_y=H // wy, wcl_x=W // wx, ws_y=wy, ws_x=wx)
    return win[:, 0, :, 0].numpy()


@pytest.mark.parametrize("case", CASES)
def test_window_token_index_matches_einops_and_roll(case):
    got = oracle.window_token_index(*case)
    np.testing.assert_array_equal(got, _einops_map(*case))


@pytest.mark.parametrize("case", CASES[:3])
def test_window_token_index_matches_loops(case):
    np.testing.assert_array_equal(oracle.window_token_index(*case), oracle.window_token_index_loops(*case))


@settings(max_examples=40, deadline=None)
@given(B=st.integers(1, 2), ny=st.integers(1, 4), nx=st.integers(1, 4), wy=st.integers(1, 5), wx=st.integers(1, 5),
       data=st.data())
def test_window_token_index_properties(B, ny, nx, wy, wx, data):
    sy = data.draw(st.integers(0, wy - 1))
    sx = data.draw(st.integers(0, wx - 1))
    H, W = ny * wy, nx * wx
    idx = oracle.window_token_index(B, H, W, wy, wx, sy, sx)
    # a permutation of all tokens
    assert sorted(idx.reshape(-1).tolist()) == list(range(B * H * W))
    np.testing.assert_array_equal(idx, _einops_map(B, H, W, wy, wx, sy, sx))
    np.testing.assert_array_equal(idx, oracle.window_token_index_loops(B, H, W, wy, wx, sy, sx))


def test_reverse_is_inverse_of_partition():
    B, H, W, wy, wx = 2, 8, 12, 4, 4
    x = torch.randn(B, H * W, 6)
    from oracle.swin_oracle import _partition, _reverse
    win = _partition(x, B, H, W, wy, wx)
    want = rearrange(x, "b (a p c q) d -> (b a c) (p q) d", a=H // wy, p=wy, c=W // wx, q=wx)
    torch.testing.assert_close(win, want, rtol=0, atol=0)
    back = _reverse(win, B, H, W, wy, wx)
    torch.testing.assert_close(back, x, rtol=0, atol=0)
    # reverse pattern of the reference (model.py:307) with h*d flattened
    want_back = rearrange(win.reshape(-1, 1, wy * wx, 6), "(b a c) h (p q) d -> b (a p c q) (h d)", a=H // wy, c=W // wx, p=wy, q=wx)
    torch.testing.assert_close(back, want_back, rtol=0, atol=0)


@pytest.mark.parametrize("ws", [(2, 2), (3, 5), (8, 8), (12, 12), (16, 16)])
def test_relative_position_index(ws):
    got = oracle.relative_position_index(*ws)
    np.testing.assert_array_equal(got, oracle.relative_position_index_loops(*ws))
    L = ws[0] * ws[1]
    assert got.min() == 0 and got.max() == (2 * ws[0] - 1) * (2 * ws[1] - 1) - 1
    # depends only on the displacement: same value along "diagonals" of equal (dy, dx)
    assert (np.diag(got) == got[0, 0]).all()
    # known answer for 2x2 (Swin-v1 paper layout)
    if ws == (2, 2):
        np.testing.assert_array_equal(got, np.array([[4, 3, 1, 0], [5, 4, 2, 1], [7, 6, 4, 3], [8, 7, 5, 4]]))


def test_shift_mask_brute_force():
    H, W, wy, wx, sy, sx = 8, 12, 4, 4, 2, 2
    mask = oracle.shift_attention_mask(H, W, wy, wx, sy, sx)
    nWy, nWx = H // wy, W // wx
    # brute force from first principles: two tokens of a window may attend to each other iff they were
    # neighbours before the roll, i.e. neither axis wrapped between them
    for w in range(nWy * nWx):
        wyi, wxi = divmod(w, nWx)
        for p in range(wy * wx):
            for q in range(wy * wx):
                Yp, Xp = wyi * wy + p // wx, wxi * wx + p % wx  # rolled-grid coordinates
                Yq, Xq = wyi * wy + q // wx, wxi * wx + q % wx
                # original coordinates
                oYp, oYq = (Yp + sy) % H, (Yq + sy) % H
                oXp, oXq = (Xp + sx) % W, (Xq + sx) % W
                # contiguous in the original image <=> |difference| stays below the window extent
                same = abs(oYp - oYq) < wy and abs(oXp - oXq) < wx
                assert (mask[w, p, q] == 0.0) == same, (w, p, q)
    assert set(np.unique(mask)) == {-100.0, 0.0}


def test_shift_mask_zero_shift_axis():
    m = oracle.shift_attention_mask(8, 8, 4, 4, 0, 0)
    assert (m == 0).all()
    ids = oracle.shift_region_ids(8, 8, 4, 4, 2, 0)
    assert set(np.unique(ids)) == {0, 3, 6}
