"""RMSNorm fused with the 1 x G FP8 group quant: drop-in for the grouped branch of
``rmsnorm2d_fwd_with_dynamicquant`` / ``rmsnorm2d_fwd_with_add_dynamicquant``
(aiter/ops/rmsnorm.py:506-582) and the ``module_rmsnorm_quant`` bindings (:585-632).
"""

from __future__ import annotations

import torch
from torch import Tensor

from . import _ffi
from .torch_ops import fake_none, torch_op


@torch_op("rmsnorm(Tensor(a!) out, Tensor input, Tensor weight, float epsilon, bool gemma_norm=False) -> ()", fake_none)
def rmsnorm(out: Tensor, input: Tensor, weight: Tensor, epsilon: float, gemma_norm: bool = False) -> None:
    """aiter/ops/rmsnorm.py:625-632."""
    _ffi.call("rmsnorm", out, input, weight, float(epsilon), bool(gemma_norm))


@torch_op(
    "rmsnorm_quant(Tensor(a!) out, Tensor input, Tensor(b!) scale, Tensor weight, float epsilon, int group_size=0, "
    "bool shuffle_scale=False, bool gemma_norm=False) -> ()",
    fake_none,
)
def rmsnorm_quant(
    out: Tensor,
    input: Tensor,
    scale: Tensor,
    weight: Tensor,
    epsilon: float,
    group_size: int = 0,
    shuffle_scale: bool = False,
    gemma_norm: bool = False,
) -> None:
    """aiter/ops/rmsnorm.py:612-622 (grouped fp8 output only)."""
    _ffi.call(
        "rmsnorm_quant", out, input, scale, weight, float(epsilon), int(group_size), bool(shuffle_scale),
        bool(gemma_norm),
    )


@torch_op(
    "add_rmsnorm(Tensor(a!) out, Tensor input, Tensor residual_in, Tensor(b!) residual_out, Tensor weight, "
    "float epsilon, bool gemma_norm=False) -> ()",
    fake_none,
)
def add_rmsnorm(
    out: Tensor,
    input: Tensor,
    residual_in: Tensor,
    residual_out: Tensor,
    weight: Tensor,
    epsilon: float,
    gemma_norm: bool = False,
) -> None:
    """aiter/ops/rmsnorm.py:599-609."""
    _ffi.call("add_rmsnorm", out, input, residual_in, residual_out, weight, float(epsilon), bool(gemma_norm))


@torch_op(
    "add_rmsnorm_quant(Tensor(a!) out, Tensor input, Tensor residual_in, Tensor(b!) residual_out, Tensor(c!) scale, "
    "Tensor weight, float epsilon, int group_size=0, bool shuffle_scale=False, bool gemma_norm=False) -> ()",
    fake_none,
)
def add_rmsnorm_quant(
    out: Tensor,
    input: Tensor,
    residual_in: Tensor,
    residual_out: Tensor,
    scale: Tensor,
    weight: Tensor,
    epsilon: float,
    group_size: int = 0,
    shuffle_scale: bool = False,
    gemma_norm: bool = False,
) -> None:
    """aiter/ops/rmsnorm.py:585-597 (grouped fp8 output only)."""
    _ffi.call(
        "add_rmsnorm_quant", out, input, residual_in, residual_out, scale, weight, float(epsilon),
        int(group_size), bool(shuffle_scale), bool(gemma_norm),
    )


def _require_common(input: Tensor, use_model_sensitive_rmsnorm: int, what: str) -> None:
    # aiter/ops/rmsnorm.py:386-397: the case the reference routes to module_rmsnorm_quant; the rest
    # (fp32, hidden > 8192, the model-sensitive variant) goes to kernels outside this path
    if use_model_sensitive_rmsnorm != 0 or input.element_size() != 2 or input.shape[-1] > 8192:
        raise NotImplementedError(
            f"{what}: only bf16/fp16 rows of up to 8192 elements with use_model_sensitive_rmsnorm=0 are part of "
            "this library"
        )


def _rms_norm_fake(input, weight, epsilon, use_model_sensitive_rmsnorm=0):
    return torch.empty_like(input)


@torch_op("rms_norm(Tensor input, Tensor weight, float epsilon, int use_model_sensitive_rmsnorm=0) -> Tensor",
          _rms_norm_fake)
def rms_norm(input: Tensor, weight: Tensor, epsilon: float, use_model_sensitive_rmsnorm: int = 0) -> Tensor:
    """aiter/ops/rmsnorm.py:415-423: returns a fresh tensor."""
    _require_common(input, use_model_sensitive_rmsnorm, "rms_norm")
    out = torch.empty_like(input)
    _ffi.call("rmsnorm", out, input, weight, float(epsilon), False)
    return out


def rmsnorm2d_fwd(input: Tensor, weight: Tensor, epsilon: float, use_model_sensitive_rmsnorm: int = 0) -> Tensor:
    """aiter/ops/rmsnorm.py:426-433."""
    return rms_norm(input, weight, epsilon, use_model_sensitive_rmsnorm)


def rmsnorm2d_fwd_with_add(
    out: Tensor,
    input: Tensor,
    residual_in: Tensor,
    residual_out: Tensor,
    weight: Tensor,
    epsilon: float,
    gemma_norm: bool = False,
    use_model_sensitive_rmsnorm: int = 0,
) -> None:
    """aiter/ops/rmsnorm.py:436-465: residual_out = input + residual_in, out = rmsnorm(residual_out)."""
    _require_common(input, use_model_sensitive_rmsnorm, "rmsnorm2d_fwd_with_add")
    add_rmsnorm(out, input, residual_in, residual_out, weight, epsilon, gemma_norm)


def _require_grouped(yscale: Tensor, group_size: int, what: str) -> None:
    if yscale.element_size() == 1:
        raise NotImplementedError(f"{what}: e8m0 scales are not part of this library")
    if group_size == 0:
        raise NotImplementedError(
            f"{what}: only the grouped path (group_size in 32/64/128) is part of this library; "
            "per-token dynamic quant (group_size=0) is not"
        )


def rmsnorm2d_fwd_with_dynamicquant(
    out: Tensor,
    input: Tensor,
    yscale: Tensor,
    weight: Tensor,
    epsilon: float,
    use_model_sensitive_rmsnorm: int = 0,
    group_size: int = 0,
    shuffle_scale: bool = False,
) -> None:
    """aiter/ops/rmsnorm.py:506-532, grouped branch (:527-532)."""
    _require_grouped(yscale, group_size, "rmsnorm2d_fwd_with_dynamicquant")
    assert input.shape[-1] <= 8192, "grouped/shuffle rmsnorm dynamicquant supports hidden<=8192"
    rmsnorm_quant(out, input, yscale, weight, epsilon, group_size, shuffle_scale)


def rmsnorm2d_fwd_with_add_dynamicquant(
    out: Tensor,
    input: Tensor,
    residual_in: Tensor,
    residual_out: Tensor,
    yscale: Tensor,
    weight: Tensor,
    epsilon: float,
    use_model_sensitive_rmsnorm: int = 0,
    group_size: int = 0,
    shuffle_scale: bool = False,
) -> None:
    """aiter/ops/rmsnorm.py:535-582, grouped branch (:567-582)."""
    _require_grouped(yscale, group_size, "rmsnorm2d_fwd_with_add_dynamicquant")
    assert input.shape[-1] <= 8192, "grouped/shuffle rmsnorm add_dynamicquant supports hidden<=8192"
    add_rmsnorm_quant(out, input, residual_in, residual_out, yscale, weight, epsilon, group_size, shuffle_scale)
