"""GPU parity: RMSNorm (+residual add) fused with the 1x128 FP8 quant, through the C-ABI."""

import numpy as np
import pytest
import torch

import aiter_amd
from aiter_amd import dtypes
from oracle import c_oracle as co
from oracle import torch_ref as tr
from tests.helpers import assert_quant_bit_exact, bits32, codes8, codes16, from_codes16, guarded_empty

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def make_norm_inputs(m, k, seed):
    x = tr.make_activation(m, k, seed=seed)
    g = torch.Generator().manual_seed(seed + 100)
    w = (torch.rand(k, generator=g) + 0.5).bfloat16()  # U(0.5, 1.5), benchmark config 5
    return x, w


def gpu_rmsnorm(x, w, eps, gemma=False):
    out = torch.empty_like(x)
    aiter_amd.rmsnorm(out, x, w, eps, gemma)
    return out


def gpu_rmsnorm_quant(x, w, eps, group=128, shuffle=False):
    m, k = x.shape
    out = torch.empty(m, k, dtype=dtypes.fp8, device=x.device)
    s = torch.empty(m, k // group, dtype=torch.float32, device=x.device)
    aiter_amd.rmsnorm2d_fwd_with_dynamicquant(out, x, s, w, eps, 0, group_size=group, shuffle_scale=shuffle)
    return out, s


@pytest.mark.parametrize("m,k", [(1, 128), (7, 1024), (64, 7168), (33, 8192), (5, 1536), (16, 4096)])
def test_rmsnorm_matches_oracle_bit_exact(m, k):
    x, w = make_norm_inputs(m, k, seed=m + k)
    out = gpu_rmsnorm(x.to(DEV), w.to(DEV), 1e-6)
    torch.cuda.synchronize()
    expect = co.rmsnorm_bf16(codes16(x), codes16(w), 1e-6)
    assert np.array_equal(codes16(out), expect)


def test_rmsnorm_vs_torch_reference_within_one_ulp():
    # torch sums squares in its own fp32 order, so a few results may sit one bf16 ulp away
    x, w = make_norm_inputs(256, 7168, seed=1)
    out = gpu_rmsnorm(x.to(DEV), w.to(DEV), 1e-6)
    ref, _ = tr.rmsnorm_ref(x, w, 1e-6)
    a, b = codes16(out).astype(np.int32), codes16(ref).astype(np.int32)
    assert np.abs(a - b).max() <= 1
    assert (a != b).mean() < 1e-4
    assert torch.allclose(out.cpu().float(), ref.float(), rtol=1e-2, atol=1e-2)


def test_rmsnorm_constant_rows_closed_form():
    # x = c everywhere, w = 1: mean(x^2) = c^2, result = c / sqrt(c^2 + eps)
    k = 2048
    cs = [0.5, -2.0, 3.0, 100.0]
    x = torch.tensor(cs).view(-1, 1).repeat(1, k).bfloat16()
    w = torch.ones(k, dtype=torch.bfloat16)
    out = gpu_rmsnorm(x.to(DEV), w.to(DEV), 1e-6).cpu().float()
    for i, c in enumerate(cs):
        expect = np.float32(c) * (np.float32(1.0) / np.sqrt(np.float32(c * c) + np.float32(1e-6)))
        assert torch.all(out[i] == torch.tensor(float(expect)).bfloat16().float())


def test_gemma_norm_uses_one_plus_weight():
    x, w = make_norm_inputs(9, 1024, seed=4)
    out = gpu_rmsnorm(x.to(DEV), w.to(DEV), 1e-6, gemma=True)
    expect = co.rmsnorm_bf16(codes16(x), codes16(w), 1e-6, gemma_norm=True)
    assert np.array_equal(codes16(out), expect)


@pytest.mark.parametrize("m,k,group", [(2048, 7168, 128), (3, 256, 128), (40, 8192, 128), (12, 1024, 64), (12, 1024, 32)])
def test_fused_equals_unfused_bitwise(m, k, group):
    # benchmark config 5: fused norm+quant must equal norm -> bf16 -> quant exactly
    x, w = make_norm_inputs(m, k, seed=7)
    xd, wd = x.to(DEV), w.to(DEV)
    yf, sf = gpu_rmsnorm_quant(xd, wd, 1e-6, group)
    normed = gpu_rmsnorm(xd, wd, 1e-6)
    yu, su = aiter_amd.per_group_quant_hip(normed, quant_dtype=dtypes.fp8, group_size=group)
    torch.cuda.synchronize()
    assert torch.equal(yf.view(torch.uint8), yu.view(torch.uint8))
    assert torch.equal(sf.view(torch.int32), su.view(torch.int32))


def test_fused_matches_oracle_bit_exact():
    x, w = make_norm_inputs(128, 7168, seed=21)
    y, s = gpu_rmsnorm_quant(x.to(DEV), w.to(DEV), 1e-6)
    torch.cuda.synchronize()
    normed = co.rmsnorm_bf16(codes16(x), codes16(w), 1e-6)
    assert_quant_bit_exact(y, s, from_codes16(normed), what="fused vs oracle")


def test_fused_vs_torch_reference_tolerances():
    # op_tests/test_rmsnorm2dFusedAddQuant.py:221,275-285: dequantised codes atol 1e-2, scales close
    x, w = make_norm_inputs(512, 7168, seed=0)
    y, s = gpu_rmsnorm_quant(x.to(DEV), w.to(DEV), 1e-6)
    yt, st, _, _ = tr.rmsnorm_quant_ref(x, w, 1e-6)
    deq_g = y.cpu().float().view(512, 56, 128) * s.cpu().unsqueeze(-1)
    deq_t = yt.float().view(512, 56, 128) * st.unsqueeze(-1)
    assert torch.allclose(s.cpu(), st, rtol=1e-2, atol=1e-6)
    ratio = tr.check_allclose_ratio(deq_g, deq_t, rtol=1e-2, atol=1e-2)
    assert ratio < 1e-3, ratio
    # almost every code is identical; the rest come from single-ulp differences in the norm
    assert (codes8(y) != codes8(yt)).mean() < 1e-3


def test_fused_add_variant():
    m, k = 96, 7168
    x, w = make_norm_inputs(m, k, seed=31)
    res = tr.make_activation(m, k, seed=32)
    xd, wd, rd = x.to(DEV), w.to(DEV), res.to(DEV)
    y = torch.empty(m, k, dtype=dtypes.fp8, device=DEV)
    s = torch.empty(m, k // 128, dtype=torch.float32, device=DEV)
    res_out = torch.empty_like(xd)
    aiter_amd.rmsnorm2d_fwd_with_add_dynamicquant(y, xd, rd, res_out, s, wd, 1e-6, 0, group_size=128)
    torch.cuda.synchronize()
    normed, ro = co.add_rmsnorm_bf16(codes16(x), codes16(res), codes16(w), 1e-6)
    assert np.array_equal(codes16(res_out), ro)
    assert np.array_equal(codes16(res_out), codes16(x + res))  # torch bf16 add, one rounding
    assert_quant_bit_exact(y, s, from_codes16(normed), what="add fused")
    # unfused add variant agrees too
    out16 = torch.empty_like(xd)
    res_out2 = torch.empty_like(xd)
    aiter_amd.add_rmsnorm(out16, xd, rd, res_out2, wd, 1e-6)
    assert np.array_equal(codes16(out16), normed)
    assert torch.equal(res_out2.view(torch.int16), res_out.view(torch.int16))


def test_transposed_scale_and_guards():
    x, w = make_norm_inputs(24, 1024, seed=3)
    xd, wd = x.to(DEV), w.to(DEV)
    y0, s0 = gpu_rmsnorm_quant(xd, wd, 1e-6)
    y, chk_y = guarded_empty((24, 1024), dtypes.fp8, DEV)
    s, chk_s = guarded_empty((24, 8), torch.float32, DEV)
    aiter_amd.rmsnorm_quant(y, xd, s, wd, 1e-6, 128, True)
    torch.cuda.synchronize()
    chk_y()
    chk_s()
    assert torch.equal(y.view(torch.uint8), y0.view(torch.uint8))
    assert np.array_equal(bits32(s).reshape(8, 24), bits32(s0).T)


def test_strided_input_rows():
    x, w = make_norm_inputs(16, 2048, seed=8)
    big = torch.zeros(16, 4096, dtype=torch.bfloat16, device=DEV)
    big[:, :2048] = x.to(DEV)
    view = big[:, :2048]
    y, s = gpu_rmsnorm_quant(view, w.to(DEV), 1e-6)
    y2, s2 = gpu_rmsnorm_quant(x.to(DEV), w.to(DEV), 1e-6)
    assert torch.equal(y.view(torch.uint8), y2.view(torch.uint8)) and torch.equal(s, s2)


def test_fp16_rmsnorm_quant():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(32, 1024, generator=g).half()
    w = (torch.rand(1024, generator=g) + 0.5).half()
    xd, wd = x.to(DEV), w.to(DEV)
    y, s = gpu_rmsnorm_quant(xd, wd, 1e-5)
    normed = torch.empty_like(xd)
    aiter_amd.rmsnorm(normed, xd, wd, 1e-5)
    ref = torch.nn.functional.rms_norm(x, (1024,), w, 1e-5)
    a, b = codes16(normed).astype(np.int32), codes16(ref).astype(np.int32)
    assert np.abs(a - b).max() <= 1 and (a != b).mean() < 1e-3
    assert_quant_bit_exact(y, s, normed.cpu(), in_dtype="fp16", what="fp16 fused")
