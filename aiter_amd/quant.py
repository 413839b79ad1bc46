"""1 x G dynamic FP8 group quant: drop-in for the reference's ``aiter/ops/quant.py`` entry
points on this path (``get_hip_quant`` :367-387, ``per_group_quant_hip`` :439-483,
``dynamic_per_token_scaled_quant`` :754-763).  Same signatures, shapes and scale layout.
"""

from __future__ import annotations

import functools
from typing import Optional

import torch
from torch import Tensor

from . import _ffi, dtypes
from .enums import QuantType
from .torch_ops import fake_none, torch_op


@torch_op(
    "dynamic_per_token_scaled_quant(Tensor(a!) out, Tensor input, Tensor(b!) scales, Tensor? scale_ub=None, "
    "bool shuffle_scale=False, Tensor? num_rows=None, int num_rows_factor=1) -> ()",
    fake_none,
)
def dynamic_per_token_scaled_quant(
    out: Tensor,
    input: Tensor,
    scales: Tensor,
    scale_ub: Optional[Tensor] = None,
    shuffle_scale: bool = False,
    num_rows: Optional[Tensor] = None,
    num_rows_factor: int = 1,
) -> None:
    """Native binding (aiter/ops/quant.py:754-763).  ``input`` is the [-1, G] view."""
    _ffi.call(
        "dynamic_per_token_scaled_quant",
        out,
        input,
        scales,
        scale_ub,
        bool(shuffle_scale),
        num_rows,
        int(num_rows_factor),
    )


def _per_group_quant_fake(x, scale=None, quant_dtype=dtypes.fp8, group_size=128, transpose_scale=False,
                          num_rows=None, num_rows_factor=1, scale_type=dtypes.fp32):
    shape = x.shape
    return (torch.empty(shape, dtype=quant_dtype, device=x.device),
            torch.empty((*shape[:-1], shape[-1] // group_size), dtype=scale_type, device=x.device))


@torch_op(
    "per_group_quant_hip(Tensor x, Tensor? scale=None, ScalarType quant_dtype=float8_e4m3fn, int group_size=128, "
    "bool transpose_scale=False, Tensor? num_rows=None, int num_rows_factor=1, ScalarType scale_type=float32) "
    "-> (Tensor, Tensor)",
    _per_group_quant_fake,
)
def per_group_quant_hip(
    x: Tensor,
    scale: Optional[Tensor] = None,
    quant_dtype: torch.dtype = dtypes.fp8,
    group_size: int = 128,
    transpose_scale: bool = False,
    num_rows: Optional[Tensor] = None,
    num_rows_factor: int = 1,
    scale_type: torch.dtype = dtypes.fp32,
) -> "tuple[Tensor, Tensor]":
    """aiter/ops/quant.py:439-483.  Returns (y fp8 with x's shape, scale fp32 [..., K/G]).

    With ``transpose_scale`` the scale buffer keeps that shape but is filled in [K/G, rows]
    order, as the reference kernel does (csrc/kernels/quant_kernels.cu:141-148).
    """
    shape = x.shape
    device = x.device
    if scale is not None:
        raise ValueError("unsupported: static per token quant")
    assert group_size in [32, 64, 128], f"unsupported group size {group_size=}, only support [32, 64, 128]"
    if quant_dtype != dtypes.fp8:
        raise NotImplementedError(f"only {dtypes.fp8} output is implemented on this path, got {quant_dtype}")
    if scale_type != dtypes.fp32:
        raise NotImplementedError(f"only fp32 scales are implemented on this path, got {scale_type}")
    scale = torch.empty((*shape[:-1], shape[-1] // group_size), dtype=scale_type, device=device)
    y = torch.empty(shape, dtype=quant_dtype, device=device)
    dynamic_per_token_scaled_quant(
        y,
        x.view(-1, group_size),
        scale,
        shuffle_scale=transpose_scale,
        num_rows=num_rows,
        num_rows_factor=num_rows_factor,
    )
    return y, scale


@functools.lru_cache
def get_hip_quant(qType):
    """aiter/ops/quant.py:367-387; only the 1x128 flavour exists in this library."""
    table = {
        QuantType.No.value: lambda *a, **k: (a[0], None),
        QuantType.per_1x128.value: functools.partial(per_group_quant_hip, group_size=128),
    }

    def raise_NotImplementedError(*a, **k):
        raise NotImplementedError(f"unsupported quant type {qType=}")

    return table.get(int(getattr(qType, "value", qType)), raise_NotImplementedError)


def weight_per_128x128_quant(w: torch.Tensor, quant_dtype: torch.dtype = dtypes.fp8):
    """[N, K] bf16/fp16 weights -> (fp8 codes [N, K], fp32 scales [ceil(N/128), K/128]).

    The 128x128 block quantiser that produces the GEMM's ``WQ`` / ``w_scale``.  The reference
    does this offline with torch ops (``pertoken_quant``, aiter/ops/quant.py:64-94, on
    ``[n_blocks, 128*128]`` views, op_tests/multigpu_tests/test_dispatch_combine.py:180-204);
    the result here is the same bit for bit.  K must be a multiple of 128; a ragged last row
    block is quantised as if padded with zeros.
    """
    assert w.dim() == 2, "weight_per_128x128_quant expects a [N, K] matrix"
    n, k = w.shape
    wq = torch.empty(n, k, dtype=quant_dtype, device=w.device)
    ws = torch.empty((n + 127) // 128, k // 128, dtype=torch.float32, device=w.device)
    _ffi.call("weight_per_128x128_quant", wq, w, ws)
    return wq, ws
