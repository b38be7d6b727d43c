"""The streaming layout of bfloat16 weight matrices on the GPU.

A matrix ``[rows, K]`` ("[out, in]") is cut into tiles of 16 rows x 32 k, and each tile is stored
as the 1024 contiguous bytes that one MFMA A-operand load of a wavefront reads: lane
``g * 16 + r`` holds row ``r``, elements ``8 g .. 8 g + 7`` - so the tile is ``[4 (g), 16 (r), 8]``.
Tiles follow each other along K, then along rows.  A wavefront that walks along K then reads
one contiguous kilobyte per instruction instead of sixteen 64-byte pieces 2 K bytes apart, which on
MI355X is the difference between about 5.3 and 6.1 TB/s of weight streaming.  Only the hand-written
product kernels read this layout; matrices that go to the BLAS library stay row-major.
"""
from __future__ import annotations

import torch

TILE_ROWS, TILE_K = 16, 32


def can_tile(w: torch.Tensor) -> bool:
    return (w.is_cuda and w.dtype == torch.bfloat16 and w.dim() in (2, 3) and w.shape[-2] % TILE_ROWS == 0
            and w.shape[-1] % TILE_K == 0)


def _tiled(m: torch.Tensor) -> torch.Tensor:
    rows, k = m.shape
    return m.view(rows // TILE_ROWS, TILE_ROWS, k // TILE_K, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(rows, k)


def _untiled(m: torch.Tensor) -> torch.Tensor:
    rows, k = m.shape
    return m.view(rows // TILE_ROWS, k // TILE_K, 4, TILE_ROWS, 8).permute(0, 3, 1, 2, 4).contiguous().view(rows, k)


@torch.no_grad()
def tile_(w: torch.Tensor) -> None:
    """Re-lays ``w`` (``[rows, K]`` or ``[groups, rows, K]``) in place, one group at a time."""
    if not can_tile(w):
        raise ValueError(f"a {tuple(w.shape)} {w.dtype} tensor cannot take the streaming layout")
    for m in (w if w.dim() == 3 else [w]):
        m.copy_(_tiled(m))


@torch.no_grad()
def untiled(w: torch.Tensor) -> torch.Tensor:
    """A row-major copy of a tensor that :func:`tile_` has re-laid."""
    if w.dim() == 3:
        return torch.stack([_untiled(m) for m in w])
    return _untiled(w)
