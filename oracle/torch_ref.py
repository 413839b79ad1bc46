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


def per_1x128_quant_device_formula(x: torch.Tensor, group: int = 128, quant_dtype=FP8):
    """The arithmetic of the reference's HIP kernel behind the same entry point,
    csrc/kernels/quant_kernels.cu:87-166 (with aiter_opus_plus.h:49-75 for the store): amax floored
    at 1e-10, scale = amax * float(1/448), codes = fp8(clamp(x * (1 / scale), +-448)).  It differs
    from :func:`per_1x128_quant` (the torch definition this build matches bit for bit) by
    reciprocal-multiply roundings and on all-zero groups; kept so that a test can bound that
    difference.  Bitwise parity with the reference's kernel itself is unpinned: it needs a GPU run
    of the reference, and its 1/scale may be compiled as an approximate reciprocal."""
    assert x.shape[-1] % group == 0
    lead, n = x.shape[:-1], x.shape[-1]
    xf = x.reshape(-1, group).to(torch.float32)
    dtype_max = torch.finfo(quant_dtype).max
    amax = torch.clamp(xf.abs().amax(dim=-1, keepdim=True), min=1e-10)
    scale = amax * torch.tensor(1.0 / dtype_max, dtype=torch.float32)
    inv = torch.tensor(1.0, dtype=torch.float32) / scale
    y = torch.clamp(xf * inv, -dtype_max, dtype_max).to(quant_dtype)
    return y.view(*lead, n), scale.view(*lead, n // group)


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


# ---------------------------------------------------------------------------------------------
# mixture of experts


def fused_topk_ref(gating_output: torch.Tensor, topk: int, renormalize: bool):
    """What aiter/fused_moe.py:4058-4130 asks of topk_softmax: softmax over the experts in fp32,
    the k largest (ties to the lower expert index), optionally renormalised to sum 1."""
    probs = torch.softmax(gating_output.to(torch.float32), dim=-1)
    # stable descending sort = ties to the lower index
    order = torch.sort(probs, dim=-1, descending=True, stable=True).indices[:, :topk]
    weights = torch.gather(probs, 1, order)
    if renormalize:
        weights = weights / weights.sum(dim=-1, keepdim=True)
    return weights, order.to(torch.int32)


def moe_sorting_ref(topk_ids, topk_weights, num_experts, block_size=32, expert_mask=None, num_local_tokens=None):
    """op_tests/test_moe_sorting.py:44-105 (run_torch_moe_sorting).

    Returns (sorted_ids, sorted_weights, sorted_expert_ids, num_tokens_post_pad); entries of
    sorted_weights that the reference leaves uninitialised are returned as NaN."""
    m, topk = topk_ids.shape
    max_num_tokens_padded = topk_ids.numel() + num_experts * block_size - topk
    max_num_m_blocks = (max_num_tokens_padded + block_size - 1) // block_size
    init_val = topk << 24 | m
    sorted_ids = torch.full((max_num_tokens_padded,), init_val, dtype=torch.int32)
    sorted_weights = torch.full((max_num_tokens_padded,), float("nan"), dtype=torch.float32)
    sorted_expert_ids = torch.full((max_num_m_blocks,), -1, dtype=torch.int32)
    if num_local_tokens is not None:
        topk_ids = topk_ids[: int(num_local_tokens)]
    begin = 0
    blk = 0
    skipped = 0
    for e in range(num_experts):
        if expert_mask is not None and int(expert_mask[e]) == 0:
            skipped += 1
            continue
        token_id, topk_id = torch.where(topk_ids == e)
        n = token_id.numel()
        nblk = (n + block_size - 1) // block_size
        sorted_ids[begin : begin + n] = (topk_id << 24 | token_id).to(torch.int32)
        sorted_weights[begin : begin + n] = topk_weights[token_id, topk_id]
        begin += nblk * block_size
        sorted_expert_ids[blk : blk + nblk] = e - skipped
        blk += nblk
    post_pad = torch.tensor([begin, topk_ids.shape[0]], dtype=torch.int32)
    return sorted_ids, sorted_weights, sorted_expert_ids, post_pad


def moe_blockscale_ref(a_q, w1_q, w2_q, topk_weights, topk_ids, a_scale, fc1_scale, fc2_scale,
                       block=(128, 128), activation="silu", expert_mask=None, compute=torch.float32,
                       a2_quant=False):
    """op_tests/test_moe_blockscale.py:19-101 (torch_moe_blockscale), g1u1 case.

    a2_quant=True adds what the reference's kernels do between the two GEMMs and its stage-wise
    oracles model (aiter/fused_moe.py:3330-3337 quant_func on the first stage's 16-bit output,
    torch_moe_stage2 :3732-3745): the activation product is rounded to bf16, quantised 1x128 to
    fp8 by the torch definition, and dequantised for the second GEMM.

    a_q [tokens, dim] fp8 with a_scale [tokens, dim/128]; w1_q [E, 2*inter, dim] (gate rows then
    up rows) with fc1_scale [E, (2*inter/128)*(dim/128)]; w2_q [E, dim, inter] with fc2_scale
    [E, (dim/128)*(inter/128)].  Everything is dequantised to `compute` and evaluated expert by
    expert; the result is returned in `compute` (the reference casts to the model dtype)."""
    blk_n, blk_k = block
    tokens, topk = topk_ids.shape
    E, dim, inter = w2_q.shape
    x = a_q.to(compute).view(tokens, -1, blk_k) * a_scale.to(compute).unsqueeze(-1)
    x = x.view(tokens, dim)
    s1 = fc1_scale.to(compute).view(E, 2 * inter // blk_n, dim // blk_k)
    s1 = s1.repeat_interleave(blk_n, dim=1).repeat_interleave(blk_k, dim=2)
    s2 = fc2_scale.to(compute).view(E, dim // blk_n, inter // blk_k)
    s2 = s2.repeat_interleave(blk_n, dim=1).repeat_interleave(blk_k, dim=2)
    ids = topk_ids.to(torch.int64)
    if expert_mask is not None:
        local = expert_mask.to(torch.int64).cumsum(0) - 1
        local[expert_mask == 0] = -1
        ids = local[ids]
    out = torch.zeros(tokens, topk, dim, dtype=compute)
    for e in range(E):
        mask = ids == e
        if not mask.any():
            continue
        w1 = w1_q[e].to(compute) * s1[e]
        w2 = w2_q[e].to(compute) * s2[e]
        t_idx, k_idx = torch.where(mask)
        act_in = x[t_idx] @ w1.t()
        gate, up = act_in.split([inter, inter], dim=-1)
        if activation == "silu":
            act = F.silu(gate) * up
        else:
            act = F.gelu(gate) * up
        if a2_quant:
            q, sc = per_1x128_quant(act.to(torch.bfloat16), group=blk_k)
            act = (q.to(compute).view(act.shape[0], -1, blk_k) * sc.to(compute).unsqueeze(-1)).view(act.shape)
        out[t_idx, k_idx] = act @ w2.t()
    return (out * topk_weights.to(compute).view(tokens, topk, 1)).sum(dim=1)
