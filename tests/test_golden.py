"""The oracle against the committed golden vectors (tests/golden/*.npz, written by
tests/golden/make_fixtures.py from torch CPU library routines, IEEE fp32 arithmetic, float64
matmul and exact rational sums).  Bitwise wherever the definition is exact."""

import os

import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import torch_ref as tr

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FP8 = torch.float8_e4m3fn


def load(name):
    return np.load(os.path.join(GOLDEN, name))


def bf16(codes):
    return torch.from_numpy(codes.view(np.int16).copy()).view(torch.bfloat16)


def fp8(codes):
    return torch.from_numpy(codes.copy()).view(FP8)


def f32(bits):
    return torch.from_numpy(bits.view(np.float32).copy())


def same_scales(got_bits, want_bits):
    """Bitwise, except that a NaN scale (a group that holds a NaN) may carry any payload: which of a
    group's NaNs torch's vectorised max returns, and so its payload, depends on the tensor's size."""
    got_bits, want_bits = np.asarray(got_bits, dtype=np.uint32), np.asarray(want_bits, dtype=np.uint32)
    nan_g, nan_w = (got_bits & 0x7FFFFFFF) > 0x7F800000, (want_bits & 0x7FFFFFFF) > 0x7F800000
    return bool(np.array_equal(nan_g, nan_w) and np.array_equal(got_bits[~nan_g], want_bits[~nan_w]))


@pytest.fixture(scope="module", autouse=True)
def _built(oracle_lib):
    return oracle_lib


def test_fp8_cast():
    g = load("fp8_cast.npz")
    x = g["f32_bits"].view(np.float32)
    assert np.array_equal(co.f32_to_e4m3fn(x), g["codes"])
    # the library routine the vectors came from still says the same
    assert np.array_equal(torch.from_numpy(x.copy()).to(FP8).view(torch.uint8).numpy(), g["codes"])
    finite = (g["codes"] & 0x7F) != 0x7F
    back = co.e4m3fn_to_f32(g["codes"][finite])
    assert np.array_equal(co.f32_to_e4m3fn(back), g["codes"][finite])


def test_group_quant():
    g = load("quant_1x128.npz")
    y, s = co.group_quant(g["x_bf16"], "bf16", 128)
    assert np.array_equal(y, g["y"]) and same_scales(s.view(np.uint32), g["scale_bits"])
    y, s = co.group_quant(g["x_fp16"], "fp16", 64)
    assert np.array_equal(y, g["y_fp16_g64"]) and np.array_equal(s.view(np.uint32), g["scale_fp16_g64_bits"])
    yt, st = tr.per_1x128_quant(bf16(g["x_bf16"]))
    assert np.array_equal(yt.view(torch.uint8).numpy(), g["y"])
    assert same_scales(st.contiguous().view(torch.int32).numpy().view(np.uint32), g["scale_bits"])


def test_weight_block_quant():
    g = load("weight_128x128.npz")
    q, s = co.weight_block_quant(g["w_bf16"])
    assert np.array_equal(q, g["q"]) and np.array_equal(s.view(np.uint32), g["scale_bits"])
    qt, st = tr.weight_per_128x128_quant(bf16(g["w_bf16"]))
    assert np.array_equal(qt.view(torch.uint8).numpy(), g["q"])
    assert np.array_equal(st.contiguous().view(torch.int32).numpy().view(np.uint32), g["scale_bits"])


def test_gemm_blockscale():
    g = load("gemm_blockscale.npz")
    xs, ws = g["x_scale_bits"].view(np.float32), g["w_scale_bits"].view(np.float32)
    out, _ = co.gemm_blockscale(g["xq"], g["wq"], xs, ws, "f64")
    want = g["out_f64"]
    assert np.abs(out - want).max() <= 1e-6 * np.abs(want).max()  # the oracle returns its f64 sums as fp32
    ref = tr.gemm_a8w8_blockscale_ref(fp8(g["xq"]), fp8(g["wq"]), f32(g["x_scale_bits"]), f32(g["w_scale_bits"]))
    assert np.array_equal(co.codes16(ref), g["out_bf16"])
    ref64 = tr.gemm_a8w8_blockscale_ref_f64(fp8(g["xq"]), fp8(g["wq"]), f32(g["x_scale_bits"]), f32(g["w_scale_bits"]))
    # (the restatement dequantises in fp32, as run_torch does, before its float64 product)
    assert np.allclose(ref64.numpy(), want, rtol=1e-6, atol=1e-6)


def test_rmsnorm_and_quant():
    g = load("rmsnorm_quant.npz")
    eps = float(g["eps"])
    out = co.rmsnorm_bf16(g["x"], g["weight"], eps)
    assert np.array_equal(out, g["out_exact"])
    # torch's F.rms_norm sums in fp32: at most one bf16 step away, and rarely
    step = np.abs(out.astype(np.int32) - g["out_torch"].astype(np.int32))
    assert step.max() <= 1 and (step != 0).mean() < 0.02
    y, s = co.group_quant(out, "bf16", 128)
    assert np.array_equal(y, g["y"]) and np.array_equal(s.view(np.uint32), g["scale_bits"])
    out_add, res_out = co.add_rmsnorm_bf16(g["x"], g["residual"], g["weight"], eps)
    assert np.array_equal(res_out, g["residual_out"]) and np.array_equal(out_add, g["out_add_exact"])
    y, s = co.group_quant(out_add, "bf16", 128)
    assert np.array_equal(y, g["y_add"]) and np.array_equal(s.view(np.uint32), g["scale_add_bits"])


def test_moe_routing_and_sorting():
    g = load("moe_routing.npz")
    block = int(g["block"])
    w, ids = tr.fused_topk_ref(torch.from_numpy(g["gating"]), 3, False)
    assert np.array_equal(ids.numpy(), g["topk_ids"]) and np.allclose(w.numpy(), g["topk_weights"], rtol=2e-6, atol=0)
    w, _ = tr.fused_topk_ref(torch.from_numpy(g["gating"]), 3, True)
    assert np.allclose(w.numpy(), g["topk_weights_renorm"], rtol=2e-6, atol=0)
    ids_t, w_t = torch.from_numpy(g["topk_ids"]), torch.from_numpy(g["topk_weights_renorm"])
    for prefix, mask in (("", None), ("masked_", torch.from_numpy(g["expert_mask"]))):
        s_ids, s_w, s_e, post = tr.moe_sorting_ref(ids_t, w_t, 6, block, expert_mask=mask)
        n = len(g[prefix + "sorted_ids"])
        assert int(post[0]) == n and int(post[1]) == ids_t.shape[0]
        assert np.array_equal(s_ids[:n].numpy(), g[prefix + "sorted_ids"])
        assert np.array_equal(s_e[: n // block].numpy(), g[prefix + "sorted_expert_ids"])
        real = (g[prefix + "sorted_ids"] & 0xFFFFFF) < ids_t.shape[0]
        assert np.array_equal(s_w[:n].numpy()[real], g[prefix + "sorted_weights"][real])


def test_moe_layer():
    g = load("moe_layer.npz")
    args = (fp8(g["xq"]), fp8(g["w1q"]), fp8(g["w2q"]), torch.from_numpy(g["topk_weights"]),
            torch.from_numpy(g["topk_ids"]), f32(g["x_scale_bits"]), f32(g["w1_scale_bits"]), f32(g["w2_scale_bits"]))
    plain = tr.moe_blockscale_ref(*args, compute=torch.float64)
    assert np.allclose(plain.numpy(), g["out_f64"], rtol=1e-9, atol=1e-9)
    rounded = tr.moe_blockscale_ref(*args, compute=torch.float64, a2_quant=True)
    assert np.allclose(rounded.numpy(), g["out_f64_fp8_product"], rtol=1e-9, atol=1e-9)
