"""HBM layout of the quantized operands, as index maps between logical and stored order.

Logical order is ``[B, H, L, D]``.  Q is stored row-major (padded to a multiple of 128 rows).
K and V are stored one 8 KiB tile per 64-key block, in the order the gfx950 MFMA operands are
read, so the attention kernel moves tiles to LDS as flat copies and every lane's operand is one
16-byte LDS read at ``fragment*1024 + lane*16``:

* K tile: fragment ``(t, s)`` = keys ``32t..32t+31`` x channels ``32s..32s+31``;
  lane ``32*c + r`` holds key ``32t + r``, channels ``32s + 16c .. +15``.
* V^T tile: chunk ``(dt, tt)`` = channels ``32dt..`` x keys ``32tt..``; lane ``32*hh + m`` holds
  channel ``32dt + m``; byte ``4g + c`` holds key ``32tt + 8g + 4hh + c`` - the order in which the
  S^T accumulators of ``v_mfma_i32_32x32x32_i8`` leave the keys of one query in a lane, so P is
  packed to fp8 in registers and V meets it (what ``transpose_pad_permute_cuda`` does for the
  CUDA MMA at ksana/operations/attention/backends/sage_sla.py:222-225).
"""

from __future__ import annotations

import functools

import torch

TILE_KEYS = 64
D = 128
TILE_BYTES = TILE_KEYS * D


@functools.lru_cache(maxsize=None)
def k_tile_index() -> torch.Tensor:
    """``idx[key, d]`` = byte offset inside the K tile of logical element (key, d)."""
    key = torch.arange(TILE_KEYS).view(-1, 1)
    d = torch.arange(D).view(1, -1)
    t, r = key // 32, key % 32
    s, c, e = d // 32, (d % 32) // 16, d % 16
    return (((t * 4 + s) * 64 + c * 32 + r) * 16 + e).long()


@functools.lru_cache(maxsize=None)
def v_tile_index() -> torch.Tensor:
    """``idx[key, d]`` = byte offset inside the V^T tile of logical element (key, d)."""
    key = torch.arange(TILE_KEYS).view(-1, 1)
    d = torch.arange(D).view(1, -1)
    tt, w = key // 32, key % 32
    g, hh, c = w // 8, (w % 8) // 4, w % 4
    dt, m = d // 32, d % 32
    return (((dt * 2 + tt) * 64 + hh * 32 + m) * 16 + 4 * g + c).long()


def _untile(tiles: torch.Tensor, idx: torch.Tensor, L: int) -> torch.Tensor:
    """tiles: [B, H, nkb, 8192] bytes -> logical [B, H, L, D] (padding rows dropped)."""
    B, H, nkb, _ = tiles.shape
    flat = idx.to(tiles.device).view(-1)
    out = tiles.index_select(3, flat).view(B, H, nkb * TILE_KEYS, D)
    return out[:, :, :L].contiguous()


def untile_k(k_tiles: torch.Tensor, L: int) -> torch.Tensor:
    return _untile(k_tiles, k_tile_index(), L)


def untile_v(v_tiles: torch.Tensor, L: int) -> torch.Tensor:
    return _untile(v_tiles, v_tile_index(), L)
