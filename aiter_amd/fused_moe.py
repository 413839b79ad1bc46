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

BLOCK_SIZE_M = 32  # aiter/fused_moe.py: rows per sorted block


class ActivationType(IntEnum):
    # csrc/include/aiter_enum.h:5-14 (the two the block-scale kernel accepts)
    Silu = 0
    Gelu = 1


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
        _ffi.call("topk_softmax", topk_weights, topk_ids, None, gating_output.contiguous(), bool(renormalize))
    return topk_weights, topk_ids


def moe_sorting(topk_ids, topk_weights, num_experts, model_dim, moebuf_dtype, block_size=BLOCK_SIZE_M,
                expert_mask=None, num_local_tokens=None, dispatch_policy=0):
    """Returns (sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf), sized as the
    reference sizes them; moe_buf [M, model_dim] comes back zeroed."""
    dev = topk_ids.device
    M, topk = topk_ids.shape
    max_num_tokens_padded = int(topk_ids.numel() + num_experts * block_size - topk)
    max_num_m_blocks = int((max_num_tokens_padded + block_size - 1) // block_size)
    sorted_ids = torch.empty(max_num_tokens_padded, dtype=dtypes.i32, device=dev)
    sorted_weights = torch.empty(max_num_tokens_padded, dtype=dtypes.fp32, device=dev)
    sorted_expert_ids = torch.empty(max_num_m_blocks, dtype=dtypes.i32, device=dev)
    num_valid_ids = torch.empty(2, dtype=dtypes.i32, device=dev)
    moe_buf = torch.empty((M, model_dim), dtype=moebuf_dtype, device=dev)
    _ffi.call("moe_sorting_fwd", topk_ids, topk_weights, sorted_ids, sorted_weights, sorted_expert_ids,
              num_valid_ids, moe_buf, int(num_experts), int(block_size), expert_mask, num_local_tokens,
              int(dispatch_policy))
    return sorted_ids, sorted_weights, sorted_expert_ids, num_valid_ids, moe_buf


def fmoe_fp8_blockscale_g1u1(out, input, gate, down, sorted_token_ids, sorted_weights, sorted_expert_ids,
                             num_valid_ids, topk, input_scale, fc1_scale, fc2_scale, kernelName="",
                             fc_scale_blkn=128, fc_scale_blkk=128, fc2_smooth_scale=None,
                             activation=ActivationType.Silu.value, block_size_M=32):
    """out[token] += sum_k weight_k * down_e(act(gate_e x) * up_e x) on sorted tokens (in place)."""
    _ffi.call("fmoe_fp8_blockscale_g1u1", out, input, gate, down, sorted_token_ids, sorted_weights,
              sorted_expert_ids, num_valid_ids, int(topk), input_scale, fc1_scale, fc2_scale, kernelName or "",
              int(fc_scale_blkn), int(fc_scale_blkk), fc2_smooth_scale, int(activation), int(block_size_M))
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
