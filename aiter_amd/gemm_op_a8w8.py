"""Block-scale FP8 GEMM: drop-in for ``gemm_a8w8_blockscale`` (aiter/ops/gemm_op_a8w8.py:804-872)
and its low-level binding ``gemm_a8w8_blockscale_ck`` (:285-298).

The reference picks between CK, CK-Tile, ASM and Triton backends through tuned CSV tables;
here one library holds every kernel and chooses by shape inside C++, so the dispatch above the
boundary disappears while the call signatures stay.
"""

from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from . import _ffi, dtypes


def gemm_a8w8_blockscale_ck(
    XQ: Tensor,
    WQ: Tensor,
    x_scale: Tensor,
    w_scale: Tensor,
    Out: Tensor,
    splitK: int = 0,
    kernelName: str = "",
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:285-298: writes ``Out`` and returns it.  ``splitK`` is the log2
    of the number of K partitions, ``kernelName`` one of :func:`gemm_kernel_names` or ""."""
    _ffi.call("gemm_a8w8_blockscale", XQ, WQ, x_scale, w_scale, Out, int(splitK), kernelName or "")
    return Out


def gemm_a8w8_blockscale(
    XQ: Tensor,
    WQ: Tensor,
    x_scale: Tensor,
    w_scale: Tensor,
    dtype: torch.dtype = dtypes.bf16,
    isBpreshuffled: bool = False,
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:804-872.

    XQ [M,K] fp8, WQ [N,K] fp8, x_scale [M,K/128] fp32, w_scale [ceil(N/128),K/128] fp32;
    returns a fresh [M,N] tensor of ``dtype`` (bf16 or fp16).
    """
    assert dtype in [dtypes.bf16, dtypes.fp16], f"Output {dtype=} is currently not supported in gemm_a8w8"
    if isBpreshuffled:
        raise NotImplementedError("the pre-shuffled weight layout is not part of this library")
    m = XQ.shape[0]
    n = WQ.shape[0]
    Y = torch.empty(m, n, dtype=dtype, device=XQ.device)
    # -1: the library chooses kernel and K split from the shape
    _ffi.call("gemm_a8w8_blockscale", XQ, WQ, x_scale, w_scale, Y, -1, "")
    return Y


def gemm_a8w8_blockscale_bpreshuffle_ck(
    XQ: Tensor,
    WQ: Tensor,
    x_scale: Tensor,
    w_scale: Tensor,
    Out: Tensor,
    kernelName: str = "",
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:318-330: ``WQ`` holds ``shuffle_weight(w, layout=(16, 16))`` and
    ``x_scale`` is column-major; writes ``Out`` and returns it."""
    _ffi.call("gemm_a8w8_blockscale_bpreshuffle", XQ, WQ, x_scale, w_scale, Out, kernelName or "")
    return Out


def gemm_a8w8_blockscale_bpreshuffle(
    XQ: Tensor,
    WQ: Tensor,
    x_scale: Tensor,
    w_scale: Tensor,
    dtype: torch.dtype = dtypes.bf16,
    out: Optional[Tensor] = None,
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:908-1087.

    XQ [M,K] fp8; WQ [N,K] fp8 pre-shuffled with :func:`aiter_amd.shuffle_weight` (layout
    (16,16)); x_scale the [M,K/128] scales stored column-major (what the quant kernels write
    with ``transpose_scale=True``), either as a contiguous buffer or as a strided [M,K/128]
    view; w_scale [ceil(N/128),K/128] fp32.  ``out``, when given, receives the result.
    """
    assert dtype in [dtypes.bf16, dtypes.fp16], f"Output {dtype=} is currently not supported in gemm_a8w8"
    m = XQ.shape[0]
    n = WQ.shape[0]
    if out is not None:
        assert out.shape == (m, n) and out.dtype == dtype and out.device == XQ.device, (
            f"gemm_a8w8_blockscale_bpreshuffle: out buffer {tuple(out.shape)}/{out.dtype} != expected "
            f"({m},{n})/{dtype}"
        )
        Y = out
    else:
        Y = torch.empty(m, n, dtype=dtype, device=XQ.device)
    _ffi.call("gemm_a8w8_blockscale_bpreshuffle", XQ, WQ, x_scale, w_scale, Y, "")
    return Y


def gemm_kernel_names():
    """Names accepted as ``kernelName`` (the counterpart of the reference's kernel zoo,
    csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale_instance.py:73-117)."""
    return _ffi.gemm_kernel_names()
