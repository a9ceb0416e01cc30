"""Integer index maps of the windowed attention path (numpy, CPU).  TEST INFRASTRUCTURE ONLY.

Follows the reference's token ordering:
  * tokens are row-major over the lat x lon grid, n = Y*W + X
    (src/aeris_wp_inference/model.py:302, src/aeris_wp_inference/era5.py:263);
  * window partition "b (wy iy wx ix) h d -> (b wy wx) h (iy ix) d"
    (src/aeris_wp_inference/model.py:302) and its inverse (model.py:307);
  * cyclic shift = torch.roll by (-ws_y//2, -ws_x//2) on the 2-D grid before an odd layer
    and the inverse roll after it (model.py:49-50,111-114,471-475).

The relative-position index and the cyclic-shift mask are the textbook Swin-v1
definitions; the reference has neither.
"""
from __future__ import annotations

import numpy as np


def window_token_index(B, H, W, ws_y, ws_x, shift_y=0, shift_x=0):
    """Folded partition+roll map.

    Returns int64 ``idx[B*nWy*nWx, ws_y*ws_x]`` where ``idx[w, p]`` is the row of the
    natural-order ``[B*H*W, C]`` token matrix that window ``w`` holds at position ``p``
    after the grid was rolled by ``(-shift_y, -shift_x)``:
    ``rolled[Y, X] = x[(Y + shift_y) % H, (X + shift_x) % W]`` (model.py:111-112).
    """
    assert H % ws_y == 0 and W % ws_x == 0
    nWy, nWx = H // ws_y, W // ws_x
    b = np.arange(B, dtype=np.int64).reshape(B, 1, 1, 1, 1)
    wy = np.arange(nWy, dtype=np.int64).reshape(1, nWy, 1, 1, 1)
    wx = np.arange(nWx, dtype=np.int64).reshape(1, 1, nWx, 1, 1)
    iy = np.arange(ws_y, dtype=np.int64).reshape(1, 1, 1, ws_y, 1)
    ix = np.arange(ws_x, dtype=np.int64).reshape(1, 1, 1, 1, ws_x)
    Y = (wy * ws_y + iy + shift_y) % H
    X = (wx * ws_x + ix + shift_x) % W
    idx = b * (H * W) + Y * W + X
    return np.ascontiguousarray(idx.reshape(B * nWy * nWx, ws_y * ws_x))


def window_token_index_loops(B, H, W, ws_y, ws_x, shift_y=0, shift_x=0):
    """Same map by explicit loops (for tiny grids only)."""
    nWy, nWx = H // ws_y, W // ws_x
    out = np.zeros((B * nWy * nWx, ws_y * ws_x), dtype=np.int64)
    for b in range(B):
        for wy in range(nWy):
            for wx in range(nWx):
                w = (b * nWy + wy) * nWx + wx
                for iy in range(ws_y):
                    for ix in range(ws_x):
                        Yr, Xr = wy * ws_y + iy, wx * ws_x + ix  # position on the rolled grid
                        Y, X = (Yr + shift_y) % H, (Xr + shift_x) % W  # where that token came from
                        out[w, iy * ws_x + ix] = b * H * W + Y * W + X
    return out


def relative_position_index(ws_y, ws_x):
    """Swin-v1 relative position index ``[L, L]`` into a ``[(2ws_y-1)(2ws_x-1), heads]`` table."""
    coords = np.stack(np.meshgrid(np.arange(ws_y), np.arange(ws_x), indexing="ij")).reshape(2, -1)
    rel = coords[:, :, None] - coords[:, None, :]
    rel = rel.astype(np.int64)
    rel[0] += ws_y - 1
    rel[1] += ws_x - 1
    rel[0] *= 2 * ws_x - 1
    return rel.sum(0)


def relative_position_index_loops(ws_y, ws_x):
    L = ws_y * ws_x
    out = np.zeros((L, L), dtype=np.int64)
    for p in range(L):
        for q in range(L):
            dy = p // ws_x - q // ws_x
            dx = p % ws_x - q % ws_x
            out[p, q] = (dy + ws_y - 1) * (2 * ws_x - 1) + (dx + ws_x - 1)
    return out


def shift_region_ids(H, W, ws_y, ws_x, shift_y, shift_x):
    """Region id (0..8) of every position of the ROLLED grid, ``[H, W]`` (Swin-v1 ``img_mask``).

    An axis whose shift is 0 gets a single region (no wrap happened along it).
    """
    def axis_ids(n, ws, sh):
        ids = np.zeros(n, dtype=np.int64)
        if sh > 0:
            ids[n - ws:n - sh] = 1
            ids[n - sh:] = 2
        return ids

    ry = axis_ids(H, ws_y, shift_y)
    rx = axis_ids(W, ws_x, shift_x)
    return 3 * ry[:, None] + rx[None, :]


def shift_attention_mask(H, W, ws_y, ws_x, shift_y, shift_x, neg=-100.0):
    """Swin-v1 additive mask ``[nW, L, L]``: 0 where query and key share a region, ``neg`` otherwise."""
    nWy, nWx = H // ws_y, W // ws_x
    ids = shift_region_ids(H, W, ws_y, ws_x, shift_y, shift_x)
    win = ids.reshape(nWy, ws_y, nWx, ws_x).transpose(0, 2, 1, 3).reshape(nWy * nWx, ws_y * ws_x)
    diff = win[:, :, None] != win[:, None, :]
    return np.where(diff, np.float32(neg), np.float32(0.0)).astype(np.float32)
