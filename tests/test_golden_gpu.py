"""The library, through its entry points, against the committed golden vectors
(tests/golden/*.npz; how they were made: tests/golden/make_fixtures.py).  Bit-exact for codes,
scales and indices; the GEMM and the expert layer within the reference's tolerances."""

import numpy as np
import pytest
import torch

import aiter_amd
from aiter_amd import dtypes

from tests.test_golden import bf16, f32, fp8, load, same_scales

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def u8(t):
    return t.contiguous().view(torch.uint8).cpu().numpy()


def u16(t):
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def u32(t):
    return t.contiguous().view(torch.int32).cpu().numpy().view(np.uint32)


def test_group_quant():
    g = load("quant_1x128.npz")
    y, s = aiter_amd.per_group_quant_hip(bf16(g["x_bf16"]).to(DEV), group_size=128)
    assert np.array_equal(u8(y), g["y"]) and same_scales(u32(s), g["scale_bits"])
    y, s = aiter_amd.per_group_quant_hip(bf16(g["x_bf16"]).to(DEV), group_size=128, transpose_scale=True)
    assert np.array_equal(u8(y), g["y"]) and same_scales(u32(s).reshape(8, -1).T, g["scale_bits"])
    x16 = torch.from_numpy(g["x_fp16"].view(np.int16).copy()).view(torch.float16).to(DEV)
    y, s = aiter_amd.per_group_quant_hip(x16, group_size=64)
    assert np.array_equal(u8(y), g["y_fp16_g64"]) and np.array_equal(u32(s), g["scale_fp16_g64_bits"])


def test_weight_block_quant():
    g = load("weight_128x128.npz")
    q, s = aiter_amd.weight_per_128x128_quant(bf16(g["w_bf16"]).to(DEV))
    assert np.array_equal(u8(q), g["q"]) and np.array_equal(u32(s), g["scale_bits"])


def test_gemm_blockscale_all_layouts():
    g = load("gemm_blockscale.npz")
    xq, wq = fp8(g["xq"]).to(DEV), fp8(g["wq"]).to(DEV)
    xs, ws = f32(g["x_scale_bits"]).to(DEV), f32(g["w_scale_bits"]).to(DEV)
    want = torch.from_numpy(g["out_f64"])
    outs = [aiter_amd.gemm_a8w8_blockscale(xq, wq, xs, ws),
            aiter_amd.gemm_a8w8_blockscale(xq, wq, xs, ws, dtype=torch.float16),
            aiter_amd.gemm_a8w8_blockscale_bpreshuffle(xq, aiter_amd.shuffle_weight(wq, layout=(16, 16)),
                                                       xs.t().contiguous().view(*xs.shape), ws)]
    for out in outs:
        # rtol = atol = 1e-2: op_tests/test_gemm_a8w8_blockscale.py:118
        assert torch.allclose(out.double().cpu(), want, rtol=1e-2, atol=1e-2)
    # against the fp32 evaluation rounded to bf16: the same code almost everywhere (sums that nearly
    # cancel may land a few codes apart)
    assert (u16(outs[0]) == g["out_bf16"]).mean() > 0.9


def test_rmsnorm_and_quant():
    g = load("rmsnorm_quant.npz")
    x, res, w = bf16(g["x"]).to(DEV), bf16(g["residual"]).to(DEV), bf16(g["weight"]).to(DEV)
    eps = float(g["eps"])
    out = torch.empty_like(x)
    aiter_amd.rmsnorm(out, x, w, eps)
    assert np.array_equal(u16(out), g["out_exact"])
    y = torch.empty(x.shape, dtype=dtypes.fp8, device=DEV)
    s = torch.empty(x.shape[0], x.shape[1] // 128, device=DEV)
    aiter_amd.rmsnorm2d_fwd_with_dynamicquant(y, x, s, w, eps, 0, group_size=128)
    assert np.array_equal(u8(y), g["y"]) and np.array_equal(u32(s), g["scale_bits"])
    res_out = torch.empty_like(x)
    aiter_amd.rmsnorm2d_fwd_with_add_dynamicquant(y, x, res, res_out, s, w, eps, 0, group_size=128)
    assert np.array_equal(u16(res_out), g["residual_out"])
    assert np.array_equal(u8(y), g["y_add"]) and np.array_equal(u32(s), g["scale_add_bits"])
    aiter_amd.add_rmsnorm(out, x, res, res_out, w, eps)
    assert np.array_equal(u16(out), g["out_add_exact"])


def test_moe_routing_and_sorting():
    g = load("moe_routing.npz")
    block, tokens = int(g["block"]), g["gating"].shape[0]
    gating = torch.from_numpy(g["gating"]).to(DEV)
    w, ids = aiter_amd.fused_topk(gating, gating, 3, False)
    assert np.array_equal(ids.cpu().numpy(), g["topk_ids"])
    assert np.allclose(w.cpu().numpy(), g["topk_weights"], rtol=2e-6, atol=0)
    w, ids = aiter_amd.fused_topk(gating, gating, 3, True)
    assert np.allclose(w.cpu().numpy(), g["topk_weights_renorm"], rtol=2e-6, atol=0)
    ids_t, w_t = torch.from_numpy(g["topk_ids"]).to(DEV), torch.from_numpy(g["topk_weights_renorm"]).to(DEV)
    for prefix, mask in (("", None), ("masked_", torch.from_numpy(g["expert_mask"]).to(DEV))):
        s_ids, s_w, s_e, nv, buf = aiter_amd.moe_sorting(ids_t, w_t, 6, 64, torch.bfloat16, block, expert_mask=mask)
        n = len(g[prefix + "sorted_ids"])
        assert nv.cpu().tolist() == [n, tokens] and not bool(buf.any())
        assert np.array_equal(s_ids[:n].cpu().numpy(), g[prefix + "sorted_ids"])
        assert np.array_equal(s_e[: n // block].cpu().numpy(), g[prefix + "sorted_expert_ids"])
        real = (g[prefix + "sorted_ids"] & 0xFFFFFF) < tokens
        assert np.array_equal(s_w[:n].cpu().numpy()[real], g[prefix + "sorted_weights"][real])
        # beyond the valid part: padding ids and no expert
        assert bool(((s_ids[n:] & 0xFFFFFF) == tokens).all()) and bool((s_e[n // block:] == -1).all())


@pytest.mark.parametrize("hint", ["", "down=rows"])
def test_moe_layer(hint):
    g = load("moe_layer.npz")
    E = g["w1q"].shape[0]
    w1 = aiter_amd.shuffle_weight(torch.from_numpy(g["w1q"]).to(DEV), layout=(16, 16)).view(dtypes.fp8)
    w2 = aiter_amd.shuffle_weight(torch.from_numpy(g["w2q"]).to(DEV), layout=(16, 16)).view(dtypes.fp8)
    ids, wts = torch.from_numpy(g["topk_ids"]).to(DEV), torch.from_numpy(g["topk_weights"]).to(DEV)
    xq, xs = fp8(g["xq"]).to(DEV), f32(g["x_scale_bits"]).to(DEV)
    s_ids, s_w, s_e, nv, out = aiter_amd.moe_sorting(ids, wts, E, xq.shape[1], torch.bfloat16)
    aiter_amd.fmoe_fp8_blockscale_g1u1(out, xq, w1, w2, s_ids, s_w, s_e, nv, ids.shape[1], xs.t().contiguous(),
                                       f32(g["w1_scale_bits"]).to(DEV), f32(g["w2_scale_bits"]).to(DEV), hint)
    got = out.double().cpu()
    rounded, plain = torch.from_numpy(g["out_f64_fp8_product"]), torch.from_numpy(g["out_f64"])
    assert ((got - rounded).norm() / rounded.norm()).item() < 5e-3  # bf16 output of an exact evaluation
    assert ((got - plain).norm() / plain.norm()).item() < 3e-2      # without the inter-stage fp8 rounding
