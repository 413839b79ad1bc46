"""torch-CPU restatement of the reference's torch functions for the FP8 block-scale path.

TEST INFRASTRUCTURE ONLY (checker and CPU baseline); the product never imports this.

Each function names the reference lines it follows (paths relative to the reference
checkout).  They are deliberately plain torch so that they run on host cores exactly as
the reference's own test oracles do.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

FP8 = torch.float8_e4m3fn
FP8_MAX = 448.0  # torch.finfo(torch.float8_e4m3fn).max, aiter/ops/quant.py:55-61


def pertoken_quant(x: torch.Tensor, quant_dtype=FP8, dtype_max: float | None = None):
    """aiter/ops/quant.py:64-94 (dynamic branch, no smooth scale).

    fp32 view of x, amax over the last dim, scale = amax / dtypeMax, exact-zero scales
    become 1, y = (x / scale) cast to the quantised dtype; scale returned as fp32.
    """
    xf = x.to(torch.float32)
    if dtype_max is None:
        dtype_max = torch.finfo(quant_dtype).max
    amax, _ = torch.max(torch.abs(xf), dim=-1, keepdim=True)
    scale = amax / dtype_max
    scale[scale == 0] = 1
    y = (xf / scale).to(quant_dtype)
    return y, scale.to(torch.float32)


def per_1x128_quant(x: torch.Tensor, group: int = 128, quant_dtype=FP8):
    """aiter/ops/quant.py:331-346 per_block_quant_wrapper((1,128))(pertoken_quant)."""
    assert x.shape[-1] % group == 0, f"block size {group} not match {x.shape[-1]}"
    lead, n = x.shape[:-1], x.shape[-1]
    y, s = pertoken_quant(x.reshape(-1, group), quant_dtype=quant_dtype)
    return y.view(*lead, n), s.view(*lead, n // group)


def weight_per_128x128_quant(w: torch.Tensor, block=(128, 128), quant_dtype=FP8):
    """op_tests/multigpu_tests/test_dispatch_combine.py:180-204 for one [N,K] matrix.

    Every 128x128 tile is flattened to one row for ``pertoken_quant``.  The reference only
    handles multiples of 128; ragged edge tiles (N=2112 has a 64-row last tile) are padded
    with zeros here, which changes neither amax nor any code, and cropped afterwards.
    """
    bn, bk = block
    n, k = w.shape
    nb, kb = (n + bn - 1) // bn, (k + bk - 1) // bk
    wp = torch.zeros(nb * bn, kb * bk, dtype=w.dtype)
    wp[:n, :k] = w
    blocks = wp.view(nb, bn, kb, bk).permute(0, 2, 1, 3).contiguous().view(-1, bn * bk)
    q, s = pertoken_quant(blocks, quant_dtype=quant_dtype)
    q = q.view(nb, kb, bn, bk).permute(0, 2, 1, 3).contiguous().view(nb * bn, kb * bk)
    return q[:n, :k].contiguous(), s.view(nb, kb)


def dequant_blockscale(xq, wq, x_scale, w_scale, block=(128, 128)):
    """The operand preparation of op_tests/test_gemm_a8w8_blockscale.py:28-50."""
    bn, bk = block
    m, k = xq.shape
    n = wq.shape[0]
    sk = (k + bk - 1) // bk
    x = xq.to(torch.float32).view(m, k // bk, bk) * x_scale.unsqueeze(-1)
    x = x.view(m, k)
    ws = w_scale.repeat_interleave(bn, dim=0).repeat_interleave(bk, dim=1)[:n, :k]
    assert w_scale.shape[1] == sk
    w = wq.to(torch.float32) * ws
    return x, w


def gemm_a8w8_blockscale_ref(xq, wq, x_scale, w_scale, dtype=torch.bfloat16, block=(128, 128)):
    """op_tests/test_gemm_a8w8_blockscale.py:28-54 run_torch: fp32 F.linear on dequantised
    operands, cast to the output dtype."""
    x, w = dequant_blockscale(xq, wq, x_scale, w_scale, block)
    return F.linear(x, w).to(dtype)


def gemm_a8w8_blockscale_ref_f64(xq, wq, x_scale, w_scale, block=(128, 128)):
    """Same operands, fp64 accumulation: the textbook answer the fp32 one approximates."""
    x, w = dequant_blockscale(xq, wq, x_scale, w_scale, block)
    return F.linear(x.double(), w.double())


def rmsnorm_ref(x, weight, eps, residual=None):
    """op_tests/test_rmsnorm2dFusedAddQuant.py:23-46: F.rms_norm in the input dtype, with the
    optional residual added first (the sum is rounded to the input dtype)."""
    res_out = None
    if residual is not None:
        res_out = x + residual
        x = res_out
    out = F.rms_norm(x, (x.shape[-1],), weight=weight, eps=eps)
    return out, res_out


def rmsnorm_quant_ref(x, weight, eps, residual=None, group: int = 128):
    """op_tests/test_rmsnorm2dFusedAddQuant.py:23-55 with quant_type=per_1x128: the bf16 norm
    output is quantised per 1x128 group."""
    out, res_out = rmsnorm_ref(x, weight, eps, residual)
    y, s = per_1x128_quant(out, group)
    return y, s, out, res_out


def check_allclose_ratio(a, b, rtol=1e-2, atol=1e-2):
    """aiter/test_common.py:479-493: fraction of elements outside |a-b| <= atol + rtol*|b|."""
    close = torch.isclose(a.float(), b.float(), rtol=rtol, atol=atol)
    return 1.0 - close.float().mean().item()


# ---------------------------------------------------------------- synthetic inputs


def make_activation(m, k, seed=0, outlier_frac=0.0, outlier_gain=50.0):
    """x ~ N(0,1) bf16; optionally the first ``outlier_frac`` of a random channel
    permutation is multiplied by ``outlier_gain`` (1 % x50 in the bandwidth config)."""
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    if outlier_frac > 0:
        n_out = max(1, int(round(k * outlier_frac)))
        ch = torch.randperm(k, generator=g)[:n_out]
        x[:, ch] *= outlier_gain
    return x.bfloat16()


def make_weight(n, k, seed=1, std=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(n, k, generator=g) * std).bfloat16()
