"""Block-scale FP8 mixture of experts: routing, sorting and the gated-expert kernel.

Host-side mirror of the reference's Python surface for this path:
``fused_topk`` (aiter/fused_moe.py:4058-4130), ``moe_sorting`` (aiter/fused_moe.py:341-416 with
the allocation rules of ``_moe_sorting_impl`` :175-224), ``fmoe_fp8_blockscale_g1u1``
(aiter/ops/moe_op.py:224-244) and the composition the reference's test performs
(op_tests/test_moe_blockscale.py:130-162).  All compute happens in ``libaiter_fp8bs.so``.
"""

from __future__ import annotations

from enum import IntEnum

import torch

from . import _ffi, dtypes
from .enums import QuantType
from .torch_ops import fake_none, torch_op

BLOCK_SIZE_M = 32  # aiter/fused_moe.py: rows per sorted block


class ActivationType(IntEnum):
    # csrc/include/aiter_enum.h:5-14 (the two the block-scale kernel accepts)
    Silu = 0
    Gelu = 1


@torch_op(
    "topk_softmax(Tensor(a!) topk_weights, Tensor(b!) topk_indices, Tensor(c!)? token_expert_indices, "
    'Tensor gating_output, bool need_renorm, int num_shared_experts=0, str shared_expert_scoring_func="") -> ()',
    fake_none,
)
def topk_softmax(topk_weights, topk_indices, token_expert_indices, gating_output, need_renorm,
                 num_shared_experts=0, shared_expert_scoring_func=""):
    """Native binding (aiter/ops/moe_op.py:29-66): softmax over the experts, top-k (ties to the lower
    index), optional renormalisation; ``token_expert_indices`` (may be None) receives
    ``slot * tokens + token``."""
    if num_shared_experts:
        raise NotImplementedError("topk_softmax: shared-expert scoring is not part of this library")
    _ffi.call("topk_softmax", topk_weights, topk_indices, token_expert_indices, gating_output, bool(need_renorm))


@torch_op(
    "moe_sorting_fwd(Tensor topk_ids, Tensor topk_weights, Tensor(a!) sorted_token_ids, Tensor(b!) sorted_weights, "
    "Tensor(c!) sorted_expert_ids, Tensor(d!) num_valid_ids, Tensor(e!) moe_buf, int num_experts, int unit_size, "
    "Tensor? local_expert_mask=None, Tensor? num_local_tokens=None, int dispatch_policy=0) -> ()",
    fake_none,
)
def moe_sorting_fwd(topk_ids, topk_weights, sorted_token_ids, sorted_weights, sorted_expert_ids, num_valid_ids,
                    moe_buf, num_experts, unit_size, local_expert_mask=None, num_local_tokens=None,
                    dispatch_policy=0):
    """Native binding (aiter/ops/moe_sorting.py:11-25): fills the sorted arrays and zeroes ``moe_buf``."""
    _ffi.call("moe_sorting_fwd", topk_ids, topk_weights, sorted_token_ids, sorted_weights, sorted_expert_ids,
              num_valid_ids, moe_buf, int(num_experts), int(unit_size), local_expert_mask, num_local_tokens,
              int(dispatch_policy))


def fused_topk(hidden_states, gating_output, topk, renormalize, topk_ids=None, topk_weights=None):
    """softmax over the experts, top-k, optional renormalisation -> (topk_weights fp32, topk_ids int32)."""
    assert hidden_states.shape[0] == gating_output.shape[0], "Number of tokens mismatch"
    M = hidden_states.shape[0]
    dev = gating_output.device
    if topk_weights is None:
        topk_weights = torch.empty(M, topk, dtype=dtypes.fp32, device=dev)
    if topk_ids is None:
        topk_ids = torch.empty(M, topk, dtype=dtypes.i32, device=dev)
    topk_weights, topk_ids = topk_weights[:M], topk_ids[:M]
    if M:
        topk_softmax(topk_weights, topk_ids, None, gating_output.contiguous(), bool(renormalize))
    return topk_weights, topk_ids


def moe_sorting(topk_ids, topk_weights, num_experts, model_dim, moebuf_dtype, block_size=BLOCK_SIZE_M,
                expert_mask=None, num_local_tokens=None, dispatch_policy=0, return_local_topk_ids=False,
                accumulate=True, flat=False, output_aux=False):
    """Returns (sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf), sized as the
    reference sizes them (aiter/fused_moe.py:208-224); moe_buf [M, model_dim] comes back zeroed.  With
    ``accumulate=False`` and no expert mask moe_buf is the reference's (0, 0) placeholder.  The
    reference's other extras (local top-k ids, flat routing, auxiliary outputs) belong to kernels
    outside this path."""
    for name, value in (("return_local_topk_ids", return_local_topk_ids), ("flat", flat), ("output_aux", output_aux)):
        if value:
            raise NotImplementedError(f"moe_sorting: {name} is not part of this library")
    dev = topk_ids.device
    M, topk = topk_ids.shape
    max_num_tokens_padded = int(topk_ids.numel() + num_experts * block_size - topk)
    max_num_m_blocks = int((max_num_tokens_padded + block_size - 1) // block_size)
    sorted_ids = torch.empty(max_num_tokens_padded, dtype=dtypes.i32, device=dev)
    sorted_weights = torch.empty(max_num_tokens_padded, dtype=dtypes.fp32, device=dev)
    sorted_expert_ids = torch.empty(max_num_m_blocks, dtype=dtypes.i32, device=dev)
    num_valid_ids = torch.empty(2, dtype=dtypes.i32, device=dev)
    if expert_mask is not None or accumulate:
        moe_buf = torch.empty((M, model_dim), dtype=moebuf_dtype, device=dev)
    else:
        moe_buf = torch.empty((0, 0), dtype=moebuf_dtype, device=dev)
    moe_sorting_fwd(topk_ids, topk_weights, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf,
                    int(num_experts), int(block_size), expert_mask, num_local_tokens, int(dispatch_policy))
    return sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf


@torch_op(
    "fmoe_fp8_blockscale_g1u1(Tensor(a!) out, Tensor input, Tensor gate, Tensor down, Tensor sorted_token_ids, "
    "Tensor sorted_weights, Tensor sorted_expert_ids, Tensor num_valid_ids, int topk, Tensor? input_scale, "
    'Tensor fc1_scale, Tensor fc2_scale, str? kernelName="", int fc_scale_blkn=128, int fc_scale_blkk=128, '
    "Tensor? fc2_smooth_scale=None, int? activation=0, int block_size_M=32) -> ()",
    fake_none,
)
def fmoe_fp8_blockscale_g1u1(out, input, gate, down, sorted_token_ids, sorted_weights, sorted_expert_ids,
                             num_valid_ids, topk, input_scale, fc1_scale, fc2_scale, kernelName="",
                             fc_scale_blkn=128, fc_scale_blkk=128, fc2_smooth_scale=None,
                             activation=ActivationType.Silu.value, block_size_M=32):
    """out[token] += sum_k weight_k * down_e(act(gate_e x) * up_e x) on sorted tokens (in place)."""
    _ffi.call("fmoe_fp8_blockscale_g1u1", out, input, gate, down, sorted_token_ids, sorted_weights,
              sorted_expert_ids, num_valid_ids, int(topk), input_scale, fc1_scale, fc2_scale, kernelName or "",
              int(fc_scale_blkn), int(fc_scale_blkk), fc2_smooth_scale, int(activation or 0), int(block_size_M))
    return None


def fused_moe_blockscale(hidden_states_q, w1_shuffled, w2_shuffled, topk_weights, topk_ids, w1_scale, w2_scale,
                         a1_scale_t, dtype=torch.bfloat16, scale_blk=(128, 128), activation=ActivationType.Silu,
                         expert_mask=None):
    """The call sequence of op_tests/test_moe_blockscale.py:130-162: sort, then the expert kernel."""
    E = w1_shuffled.shape[0]
    model_dim = hidden_states_q.shape[-1]
    topk = topk_ids.shape[-1]
    sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, out = moe_sorting(
        topk_ids, topk_weights, E if expert_mask is None else expert_mask.numel(), model_dim, dtype,
        expert_mask=expert_mask)
    fmoe_fp8_blockscale_g1u1(out, hidden_states_q, w1_shuffled, w2_shuffled, sorted_ids, sorted_weights,
                             sorted_expert_ids, num_valid_ids, topk, a1_scale_t, w1_scale, w2_scale, "",
                             scale_blk[0], scale_blk[1], None, int(activation))
    return out


def fused_moe(hidden_states, w1, w2, topk_weight, topk_ids, expert_mask=None, activation=ActivationType.Silu,
              quant_type=QuantType.per_1x128, doweight_stage1=False, w1_scale=None, w2_scale=None, a1_scale=None,
              a2_scale=None, block_size_M=None, num_local_tokens=None, moe_sorting_dispatch_policy=0, dtype=None,
              **other):
    """The block-scale flavour of aiter/fused_moe.py:458-577: ``quant_type`` per_1x128 (or per_128x128,
    which the reference maps onto it, :1310), gate/up experts (g1u1), fp8 weights pre-shuffled with layout
    (16,16) and their 128x128 scales.

    hidden_states: bf16/fp16 [tokens, dim] (quantised 1x128 inside, as the reference's kernel does,
    :1133-1136), or fp8 with ``a1_scale`` [tokens, dim/128] (transposed here, as the reference does with
    partial_transpose, :1152-1158).  Returns the bf16/fp16 result [tokens, dim].  Every other option of the
    reference's entry point raises NotImplementedError naming it."""
    qt = QuantType(quant_type)
    if qt not in (QuantType.per_1x128, QuantType.per_128x128):
        raise NotImplementedError(f"fused_moe: only the block-scale flavour (per_1x128) is part of this library, got {qt!r}")
    for name, value, neutral in (("doweight_stage1", doweight_stage1, False), ("a2_scale", a2_scale, None)):
        if value is not neutral and value:
            raise NotImplementedError(f"fused_moe: {name} is not supported by the block-scale kernel")
    def neutral(v):
        return v is None or (isinstance(v, (bool, int)) and v in (0, -1)) or (isinstance(v, str) and v == "separated")

    unsupported = {k: v for k, v in other.items() if not neutral(v)}
    if unsupported:
        raise NotImplementedError(f"fused_moe: unsupported options {sorted(unsupported)}")
    # the reference's block-scale kernels exist for blocks of 16, 32 and 64 sorted rows
    # (hsa/gfx950/fmoe/silu/fmoe_bf16_blockscaleFp8_g1u1_silu.csv); 128 is taken as well
    block_m = BLOCK_SIZE_M if block_size_M in (None, -1, 0) else int(block_size_M)
    if block_m not in (16, 32, 64, 128):
        raise NotImplementedError(f"fused_moe: block_size_M must be 16, 32, 64 or 128, got {block_size_M}")
    if w1_scale is None or w2_scale is None:
        raise ValueError("fused_moe: w1_scale and w2_scale are required for per_1x128")
    tokens, dim = hidden_states.shape
    E = w1.shape[0]
    topk = topk_ids.shape[1]
    if w1.shape[1] != 2 * w2.shape[2]:
        raise NotImplementedError("fused_moe: only gated experts (w1 = [E, 2*inter_dim, dim]) are supported")
    if dtype is None:
        dtype = hidden_states.dtype if hidden_states.dtype in (torch.bfloat16, torch.float16) else torch.bfloat16
    num_experts = E if expert_mask is None else expert_mask.numel()
    sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, out = moe_sorting(
        topk_ids, topk_weight, num_experts, dim, dtype, block_m, expert_mask, num_local_tokens,
        moe_sorting_dispatch_policy)
    if hidden_states.dtype in (torch.bfloat16, torch.float16):
        a1, scale_t = hidden_states, None
    else:
        if a1_scale is None:
            raise ValueError("a1_scale must be provided for quantized input for fused_moe")
        a1 = hidden_states
        scale_t = a1_scale.reshape(tokens, dim // 128).t().contiguous()
    fmoe_fp8_blockscale_g1u1(out, a1, w1, w2, sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, topk,
                             scale_t, w1_scale.reshape(E, -1), w2_scale.reshape(E, -1), "", 128, 128, None,
                             int(ActivationType(activation)), block_m)
    return out
