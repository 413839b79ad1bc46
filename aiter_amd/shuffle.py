"""Weight pre-shuffle for the block-scale GEMM (host-side layout transform, plain torch).

Counterpart of ``shuffle_weight`` in aiter/ops/shuffle.py:148-205 for the one layout the
block-scale GEMM uses: (16, 16) on one-byte elements.
"""

from __future__ import annotations

import torch

ROWS_PER_TILE = 16   # weight rows that one MFMA operand covers
CHUNK = 32           # K elements per lane of that operand, stored as two halves of 16


def shuffle_weight(x: torch.Tensor, layout=(16, 16)) -> torch.Tensor:
    """[..., N, K] fp8 -> same shape and dtype, bytes re-ordered tile by tile.

    For every tile of 16 rows and every 32-wide K chunk the output holds the 16 rows' first
    16 bytes back to back, then the 16 rows' second 16 bytes; chunks follow each other along K,
    tiles along N.  A lane of a 16-row MFMA operand then finds its 2 x 16 bytes at
    ``tile*16*K + chunk*512 + half*256 + row*16``, and 16 neighbouring lanes read 256 contiguous
    bytes.  N must be a multiple of 16 and K of 32.
    """
    if tuple(layout) != (16, 16):
        raise NotImplementedError("only layout=(16, 16) is part of this library")
    if x.element_size() != 1:
        raise NotImplementedError("only one-byte element types (fp8) are part of this library")
    n, k = x.shape[-2], x.shape[-1]
    if n % ROWS_PER_TILE or k % CHUNK:
        raise ValueError(f"shuffle_weight needs N % 16 == 0 and K % 32 == 0, got N={n}, K={k}")
    half = CHUNK // 2
    tiles = x.reshape(-1, n // ROWS_PER_TILE, ROWS_PER_TILE, k // CHUNK, 2, half)
    out = tiles.permute(0, 1, 3, 4, 2, 5).contiguous().view(x.shape)
    out.is_shuffled = True
    return out
