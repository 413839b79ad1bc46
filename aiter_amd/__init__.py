"""MI355X-native FP8 block-scale path behind the reference's Python entry points.

    y, s = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(x, quant_dtype=aiter_amd.dtypes.fp8)
    out  = aiter_amd.gemm_a8w8_blockscale(y, wq, s, w_scale, dtype=torch.bfloat16)
    aiter_amd.rmsnorm2d_fwd_with_dynamicquant(out8, x, yscale, weight, eps, 0, group_size=128)

Everything computes in ``libaiter_fp8bs.so`` (hand-written HIP for gfx950, C ABI declared in
``include/aiter_fp8bs.h``).  There is no other backend and no CPU fallback.
"""

from . import dtypes
from .enums import QuantType
from .gemm_op_a8w8 import (
    gemm_a8w8_blockscale,
    gemm_a8w8_blockscale_bpreshuffle,
    gemm_a8w8_blockscale_bpreshuffle_asm,
    gemm_a8w8_blockscale_bpreshuffle_ck,
    gemm_a8w8_blockscale_bpreshuffle_cktile,
    gemm_a8w8_blockscale_ck,
    gemm_a8w8_blockscale_cktile,
    gemm_kernel_names,
    get_CKGEMM_config,
)
from .shuffle import shuffle_weight
from .fused_moe import (
    ActivationType,
    fmoe_fp8_blockscale_g1u1,
    fused_moe,
    fused_moe_blockscale,
    fused_topk,
    moe_sorting,
    moe_sorting_fwd,
    topk_softmax,
)
from .quant import (
    dynamic_per_token_scaled_quant,
    get_hip_quant,
    per_group_quant_hip,
    weight_per_128x128_quant,
)
from .rmsnorm import (
    add_rmsnorm,
    add_rmsnorm_quant,
    rms_norm,
    rmsnorm,
    rmsnorm2d_fwd,
    rmsnorm2d_fwd_with_add,
    rmsnorm2d_fwd_with_add_dynamicquant,
    rmsnorm2d_fwd_with_dynamicquant,
    rmsnorm_quant,
)

__all__ = [
    "dtypes",
    "QuantType",
    "get_hip_quant",
    "shuffle_weight",
    "weight_per_128x128_quant",
    "gemm_a8w8_blockscale_bpreshuffle",
    "gemm_a8w8_blockscale_bpreshuffle_ck",
    "gemm_a8w8_blockscale_bpreshuffle_asm",
    "per_group_quant_hip",
    "dynamic_per_token_scaled_quant",
    "gemm_a8w8_blockscale",
    "gemm_a8w8_blockscale_ck",
    "gemm_a8w8_blockscale_cktile",
    "gemm_a8w8_blockscale_bpreshuffle_cktile",
    "gemm_kernel_names",
    "get_CKGEMM_config",
    "rmsnorm",
    "rmsnorm_quant",
    "rms_norm",
    "rmsnorm2d_fwd",
    "rmsnorm2d_fwd_with_add",
    "add_rmsnorm",
    "add_rmsnorm_quant",
    "rmsnorm2d_fwd_with_dynamicquant",
    "rmsnorm2d_fwd_with_add_dynamicquant",
    "ActivationType",
    "fused_topk",
    "moe_sorting",
    "moe_sorting_fwd",
    "topk_softmax",
    "fmoe_fp8_blockscale_g1u1",
    "fused_moe_blockscale",
    "fused_moe",
]
