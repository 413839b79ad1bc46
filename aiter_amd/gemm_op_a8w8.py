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
from .torch_ops import fake_none, torch_op


@torch_op(
    "gemm_a8w8_blockscale_ck(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor(a!) Out, int splitK=0, "
    'str kernelName="") -> ()',
    fake_none,
)
def _blockscale_into(XQ: Tensor, WQ: Tensor, x_scale: Tensor, w_scale: Tensor, Out: Tensor, splitK: int = 0,
                     kernelName: str = "") -> None:
    _ffi.call("gemm_a8w8_blockscale", XQ, WQ, x_scale, w_scale, Out, int(splitK), kernelName or "")


def gemm_a8w8_blockscale_ck(
    XQ: Tensor,
    WQ: Tensor,
    x_scale: Tensor,
    w_scale: Tensor,
    Out: Tensor,
    splitK: int = 0,
    kernelName: str = "",
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:285-298: writes ``Out`` and returns it.  ``kernelName`` is one of
    :func:`gemm_kernel_names`, "" (the library chooses) or a name of the reference's own zoo as its
    tuned tables carry them (dropped, together with the ``splitK`` tuned for it).  ``splitK`` (the
    log2 of the number of K partitions) is a hint: honoured by the kernels that can split K, clamped
    to what the problem allows, ignored by the others; with no name, 0 and -1 let the library choose."""
    _blockscale_into(XQ, WQ, x_scale, w_scale, Out, splitK, kernelName or "")
    return Out


def _gemm_fake(XQ, WQ, x_scale, w_scale, dtype=dtypes.bf16, *args, **kwargs):
    return torch.empty(XQ.shape[0], WQ.shape[0], dtype=dtype, device=XQ.device)


@torch_op(
    "gemm_a8w8_blockscale(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, ScalarType dtype=bfloat16, "
    "bool isBpreshuffled=False) -> Tensor",
    _gemm_fake,
)
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
    returns a fresh [M,N] tensor of ``dtype`` (bf16 or fp16).  With ``isBpreshuffled`` the
    operands are those of :func:`gemm_a8w8_blockscale_bpreshuffle` (weights shuffled (16,16),
    ``x_scale`` stored column-major), which the reference hands to its gfx950 assembly kernel for
    M >= 16, K >= 512, bf16 (:821-825); no such limits here.
    """
    assert dtype in [dtypes.bf16, dtypes.fp16], f"Output {dtype=} is currently not supported in gemm_a8w8"
    m = XQ.shape[0]
    n = WQ.shape[0]
    Y = torch.empty(m, n, dtype=dtype, device=XQ.device)
    if isBpreshuffled:
        _ffi.call("gemm_a8w8_blockscale_bpreshuffle", XQ, WQ, x_scale, w_scale, Y, "")
    else:
        # -1: the library chooses kernel and K split from the shape
        _ffi.call("gemm_a8w8_blockscale", XQ, WQ, x_scale, w_scale, Y, -1, "")
    return Y


@torch_op(
    "gemm_a8w8_blockscale_bpreshuffle_ck(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor(a!) Out, "
    'str kernelName="") -> ()',
    fake_none,
)
def _bpreshuffle_into(XQ: Tensor, WQ: Tensor, x_scale: Tensor, w_scale: Tensor, Out: Tensor,
                      kernelName: str = "") -> None:
    _ffi.call("gemm_a8w8_blockscale_bpreshuffle", XQ, WQ, x_scale, w_scale, Out, kernelName or "")


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
    _bpreshuffle_into(XQ, WQ, x_scale, w_scale, Out, kernelName or "")
    return Out


def gemm_a8w8_blockscale_cktile(
    XQ: Tensor,
    WQ: Tensor,
    x_scale: Tensor,
    w_scale: Tensor,
    Out: Tensor,
    isBpreshuffled: bool = False,
    splitK: int = 0,
    kernelName: str = "",
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:301-315, the reference's second kernel family behind the same
    operands (csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale_cktile.cu:62-93): row-major weights
    and x_scale, or, with ``isBpreshuffled``, shuffled weights and column-major x_scale
    (include/gemm_a8w8_blockscale_cktile_common.cuh:334-358).  One library serves both families."""
    if isBpreshuffled:
        _bpreshuffle_into(XQ, WQ, x_scale, w_scale, Out, kernelName or "")
    else:
        _blockscale_into(XQ, WQ, x_scale, w_scale, Out, splitK, kernelName or "")
    return Out


def gemm_a8w8_blockscale_bpreshuffle_cktile(
    XQ: Tensor,
    WQ: Tensor,
    x_scale: Tensor,
    w_scale: Tensor,
    Out: Tensor,
    isBpreshuffled: bool = True,
    kernelName: str = "",
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:333-346 (gemm_a8w8_blockscale_cktile.cu:96-107)."""
    return gemm_a8w8_blockscale_cktile(XQ, WQ, x_scale, w_scale, Out, isBpreshuffled, 0, kernelName)


def gemm_a8w8_blockscale_bpreshuffle_asm(
    A: Tensor,
    B: Tensor,
    out: Tensor,
    A_scale: Tensor,
    B_scale: Tensor,
    bias: Optional[Tensor] = None,
    splitK: Optional[int] = None,
    kernelName: Optional[str] = None,
    bpreshuffle: Optional[bool] = True,
    zero_bias_buf: Optional[Tensor] = None,
) -> Tensor:
    """aiter/ops/gemm_op_a8w8.py:404-430: the reference's hand-scheduled kernel for the same
    operands as :func:`gemm_a8w8_blockscale_bpreshuffle_ck` (argument order differs: ``out``
    third).  ``splitK`` and the reference's kernel names are tuning hints of that kernel and are
    not interpreted.  ``bias`` (fp32 [N] or [1, N]) is added onto the stored result by a second
    launch: ``out = round(float(round(acc)) + bias)``."""
    if not bpreshuffle:
        raise NotImplementedError("gemm_a8w8_blockscale_bpreshuffle_asm: only pre-shuffled weights (bpreshuffle=True)")
    _ffi.call("gemm_a8w8_blockscale_bpreshuffle_asm", A, B, out, A_scale, B_scale, bias,
              -1 if splitK is None else int(splitK), kernelName or "", 1, None)
    return out


def _bpreshuffle_fake(XQ, WQ, x_scale, w_scale, dtype=dtypes.bf16, out=None):
    return torch.empty(XQ.shape[0], WQ.shape[0], dtype=dtype, device=XQ.device)


def _bpreshuffle_eager(XQ, WQ, x_scale, w_scale, dtype=dtypes.bf16, out=None):
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


_bpreshuffle_op = torch_op(
    "gemm_a8w8_blockscale_bpreshuffle(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, "
    "ScalarType dtype=bfloat16, Tensor(a!)? out=None) -> Tensor",
    _bpreshuffle_fake,
)(_bpreshuffle_eager)


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
    view; w_scale [ceil(N/128),K/128] fp32.  ``out``, when given, receives the result and is
    returned.
    """
    if out is not None and torch.compiler.is_compiling():
        # traced as "write into out": an op must not return one of its arguments
        assert dtype in [dtypes.bf16, dtypes.fp16], f"Output {dtype=} is currently not supported in gemm_a8w8"
        _bpreshuffle_into(XQ, WQ, x_scale, w_scale, out, "")
        return out
    return _bpreshuffle_op(XQ, WQ, x_scale, w_scale, dtype, out)


def get_CKGEMM_config(M: int, N: int, K: int, tuned_file: Optional[str] = None, isBpreshuffled: bool = False):
    """aiter/ops/gemm_op_a8w8.py:448-490 looks (M, N, K) up in tuned CSV tables and returns the row as a
    dict (``kernelName``, ``splitK``, ``libtype`` ...) or None.  Here the choice is a shape rule inside the
    library and every shape has one; it is returned in the same form, with a ``kernelName`` that the
    low-level entry points accept.  ``tuned_file`` is accepted and not read."""
    name = _ffi.gemm_choice(M, N, K, isBpreshuffled)
    splits = int(name.split(":s=")[1]) if ":s=" in name else 1
    return {"M": M, "N": N, "K": K, "libtype": "hip", "kernelName": name, "splitK": max(splits - 1, 0).bit_length(),
            "kRanges": splits}


def gemm_kernel_names():
    """Names accepted as ``kernelName`` (the counterpart of the reference's kernel zoo,
    csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale_instance.py:73-117)."""
    return _ffi.gemm_kernel_names()
