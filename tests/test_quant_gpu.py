"""GPU parity: 1x128 dynamic FP8 group quant through the C-ABI vs the oracle (bit-exact)."""

import numpy as np
import pytest
import torch

import aiter_amd
from aiter_amd import QuantType, dtypes
from oracle import c_oracle as co
from oracle import torch_ref as tr
from tests.helpers import assert_quant_bit_exact, bits32, codes8, codes16, from_codes16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def hip_quant(x, **kw):
    return aiter_amd.get_hip_quant(QuantType.per_1x128)(x, quant_dtype=dtypes.fp8, **kw)


def test_config1_plumbing_matches_torch_reference():
    # benchmark config 1: x [32,1024] ~ N(0,1), seed 0
    x = tr.make_activation(32, 1024, seed=0)
    y, s = hip_quant(x.to(DEV))
    torch.cuda.synchronize()
    assert y.dtype == torch.float8_e4m3fn and y.shape == x.shape
    assert s.dtype == torch.float32 and s.shape == (32, 8)
    yt, st = tr.per_1x128_quant(x)
    assert np.array_equal(codes8(y), codes8(yt))
    assert np.array_equal(bits32(s), bits32(st))
    assert_quant_bit_exact(y, s, x, what="config1")


@pytest.mark.parametrize("m,k", [(1, 128), (3, 256), (17, 7168), (256, 4096), (1000, 1536), (4096, 7168)])
def test_random_shapes_bit_exact(m, k):
    x = tr.make_activation(m, k, seed=m * 7 + k, outlier_frac=0.01)
    y, s = hip_quant(x.to(DEV))
    torch.cuda.synchronize()
    assert_quant_bit_exact(y, s, x, what=f"{m}x{k}")


def test_3d_input_and_scale_shape():
    x = tr.make_activation(6 * 5, 512, seed=3).view(6, 5, 512)
    y, s = hip_quant(x.to(DEV))
    assert y.shape == (6, 5, 512) and s.shape == (6, 5, 4)
    assert_quant_bit_exact(y, s, x.reshape(30, 512), what="3d")


def test_empty_input():
    x = torch.empty(0, 256, dtype=torch.bfloat16, device=DEV)
    y, s = hip_quant(x)
    assert y.shape == (0, 256) and s.shape == (0, 2)


def _all_mantissa_pairs(exps_amax, exps_rel):
    """Groups that pair every 8-bit significand of amax with every 8-bit significand of x
    (both signs), at several exponent distances: each group = [amax, 127 other values]."""
    rows = []
    for ea in exps_amax:
        for ma in range(128):
            amax_code = ((ea + 127) << 7) | ma
            for er in exps_rel:
                xs = []
                for mx in range(128):
                    code = ((ea - er + 127) << 7) | mx
                    if code <= amax_code:
                        xs.append(code)
                xs = xs[:127] if len(xs) >= 127 else xs + [0] * (127 - len(xs))
                neg = [(c | 0x8000) if (i & 1) else c for i, c in enumerate(xs)]
                rows.append([amax_code] + neg)
    return np.array(rows, dtype=np.uint16)


def test_every_significand_pair_bit_exact():
    # exhaustive over (significand of amax) x (significand of x) x sign at exponent gaps 0..12:
    # covers every rounding position the division can land on, including fp8 subnormal results
    codes = _all_mantissa_pairs(exps_amax=[-20, 0, 7, 30], exps_rel=list(range(0, 13)))
    x = from_codes16(codes)
    y, s = hip_quant(x.to(DEV))
    torch.cuda.synchronize()
    assert_quant_bit_exact(y, s, x, what="significand pairs")


def test_unit_scale_exercises_hardware_conversion_on_every_bf16():
    # amax = 448 makes scale exactly 1, so codes are the plain e4m3fn rounding of x itself:
    # every bf16 with |x| <= 448 goes through the conversion, ties and fp8 subnormals included
    mags = np.arange(0, 0x43E0 + 1, dtype=np.uint32)  # 0x43E0 = bf16(448)
    vals = np.concatenate([mags, mags | 0x8000]).astype(np.uint16)
    n_groups = (vals.size + 126) // 127
    pad = n_groups * 127 - vals.size
    vals = np.concatenate([vals, np.zeros(pad, dtype=np.uint16)]).reshape(n_groups, 127)
    rows = np.concatenate([np.full((n_groups, 1), 0x43E0, dtype=np.uint16), vals], axis=1)
    x = from_codes16(rows)
    y, s = hip_quant(x.to(DEV))
    torch.cuda.synchronize()
    assert np.all(bits32(s) == 0x3F800000)
    expect = co.f32_to_e4m3fn(x.float().numpy())
    assert np.array_equal(codes8(y), expect)
    assert_quant_bit_exact(y, s, x, what="unit scale")


def test_special_groups_follow_torch():
    inf, nan = float("inf"), float("nan")
    rows = [
        [0.0] * 128,                                  # all zero -> scale 1, codes 0
        [-0.0] + [0.0] * 127,                         # signed zero keeps its sign
        [1.0, 2.0, inf, -3.0] + [0.5] * 124,          # inf amax
        [1.0, -inf, inf, 0.0] + [0.25] * 124,
        [1.0, nan, 2.0, -3.0] + [0.5] * 124,          # NaN group
        [2.0**-133, 2.0**-133, 2.0**-134, 0.0] + [0.0] * 124,  # scale becomes subnormal
        [2.0**-132, -(2.0**-133), 2.0**-133 * 3, 0.0] + [2.0**-133] * 124,  # bf16 subnormals
        [2.0**-81, -(2.0**-81), 2.0**-84, 0.0] + [2.0**-90] * 124,          # just below the fast range
        [2.0**-80, -(2.0**-80), 2.0**-84, 0.0] + [2.0**-99] * 124,          # first fast-path amax
        [2.0**-80, -(2.0**-133), 2.0**-120, 2.0**-100] + [2.0**-98] * 124,  # tiny x beside it
        [2.0**100, -(2.0**100), 2.0**94, 0.0] + [2.0**90] * 124,            # last fast-path amax
        [2.0**101, -(2.0**101), 2.0**94, 0.0] + [2.0**92] * 124,            # just above
        [3.0e38, -3.0e38, 1.0e30, 1.0] + [0.0] * 124, # huge amax
        [2.0**-110, -(2.0**-111), 2.0**-120, 0.0] + [2.0**-126] * 124,
    ]
    x = torch.tensor(rows, dtype=torch.float32).bfloat16()
    y, s = hip_quant(x.to(DEV))
    torch.cuda.synchronize()
    yt, st = tr.per_1x128_quant(x)
    yg, sg = codes8(y), bits32(s)
    for i in range(len(rows)):
        assert np.array_equal(yg[i], codes8(yt)[i]), f"row {i}: codes differ from torch"
        if np.isnan(st[i, 0].item()):
            assert np.isnan(s[i, 0].item())
        else:
            assert sg[i, 0] == bits32(st)[i, 0], f"row {i}: scale differs from torch"
    # negative-NaN element keeps its sign, the rest of the group gets the positive NaN code
    codes = np.full((1, 128), 0x3F80, dtype=np.uint16)
    codes[0, 1] = 0xFFC0
    xn = from_codes16(codes)
    y, s = hip_quant(xn.to(DEV))
    yt, _ = tr.per_1x128_quant(xn)
    assert np.array_equal(codes8(y), codes8(yt))


def test_fp16_input_bit_exact():
    g = torch.Generator().manual_seed(11)
    x = (torch.randn(64, 1024, generator=g) * 3).half()
    x[0, :128] = 0
    x[1, 5] = 65504.0
    x[2, :128] = 6e-8  # fp16 subnormal
    y, s = hip_quant(x.to(DEV))
    torch.cuda.synchronize()
    assert_quant_bit_exact(y, s, x, in_dtype="fp16", what="fp16")


@pytest.mark.parametrize("group", [32, 64])
def test_other_group_sizes(group):
    x = tr.make_activation(33, 1024, seed=group)
    y, s = aiter_amd.per_group_quant_hip(x.to(DEV), quant_dtype=dtypes.fp8, group_size=group)
    assert s.shape == (33, 1024 // group)
    assert_quant_bit_exact(y, s, x, group=group, what=f"group {group}")


@pytest.mark.parametrize("rows,cols", [(48, 1024), (31, 1024), (32, 128), (33, 384), (100, 896), (257, 7168), (2048, 640)])
def test_transposed_scale_layout(rows, cols):
    # csrc/kernels/quant_kernels.cu:141-148: scale[g] goes to index col*rows + row.  From 32 rows on the
    # library quantises by tiles of 32 rows x 2 groups so that a scale column's 32 rows leave as one line:
    # ragged last bands of rows, an odd number of groups per row, fewer than 32 rows (the other kernel).
    x = tr.make_activation(rows, cols, seed=rows + cols)
    y, s = hip_quant(x.to(DEV))
    yt, st = hip_quant(x.to(DEV), transpose_scale=True)
    assert st.shape == s.shape
    assert np.array_equal(codes8(y), codes8(yt))
    assert np.array_equal(bits32(st).reshape(cols // 128, rows), bits32(s).T)
    assert_quant_bit_exact(y, s, x, group=128, what=f"{rows}x{cols}")


def test_transposed_scale_layout_fp16():
    x = tr.make_activation(70, 640, seed=3).half()
    y, s = hip_quant(x.to(DEV))
    yt, st = hip_quant(x.to(DEV), transpose_scale=True)
    assert np.array_equal(codes8(y), codes8(yt))
    assert np.array_equal(bits32(st).reshape(5, 70), bits32(s).T)


def test_num_rows_limits_work_and_leaves_rest_untouched():
    x = tr.make_activation(64, 512, seed=9).to(DEV)
    n = torch.tensor([5], dtype=torch.int32, device=DEV)
    y = torch.full((64, 512), 0, dtype=torch.uint8, device=DEV).fill_(0xA5).view(dtypes.fp8)
    s = torch.full((64, 4), -7.0, dtype=torch.float32, device=DEV)
    aiter_amd.dynamic_per_token_scaled_quant(y, x.view(-1, 128), s, num_rows=n, num_rows_factor=2)
    torch.cuda.synchronize()
    yo, so = co.group_quant(codes16(x.cpu())[:10])
    assert np.array_equal(codes8(y)[:10], yo)
    assert np.array_equal(bits32(s)[:10], so.view(np.uint32))
    assert np.all(codes8(y)[10:] == 0xA5) and np.all(s.cpu().numpy()[10:] == -7.0)


def test_guard_bands_untouched():
    from tests.helpers import guarded_empty

    x = tr.make_activation(37, 640, seed=2).to(DEV)
    y, chk_y = guarded_empty((37, 640), dtypes.fp8, DEV)
    s, chk_s = guarded_empty((37, 5), torch.float32, DEV)
    aiter_amd.dynamic_per_token_scaled_quant(y, x.view(-1, 128), s)
    torch.cuda.synchronize()
    chk_y()
    chk_s()
    assert_quant_bit_exact(y, s, x.cpu(), what="guarded")


def test_full_size_properties():
    # benchmark config 2 at full size: [16384, 7168] with 1 % outlier channels.  Too big for the
    # scalar oracle in seconds, so check 64 sampled rows bit-exactly plus size-independent
    # properties on everything: scale == amax/448 and the amax element encodes +-448.
    x = tr.make_activation(16384, 7168, seed=0, outlier_frac=0.01)
    xd = x.to(DEV)
    y, s = hip_quant(xd)
    torch.cuda.synchronize()
    amax = xd.float().view(16384, 56, 128).abs().amax(dim=-1).cpu()
    expect_s = amax / 448.0  # on the host: the IEEE division the reference's torch CPU path performs
    assert torch.equal(s.cpu().view(torch.int32), expect_s.view(torch.int32))
    mag = (y.view(torch.uint8) & 0x7F).view(16384, 56, 128).amax(dim=-1)
    assert bool((mag == 0x7E).all())
    rows = torch.randperm(16384, generator=torch.Generator().manual_seed(1))[:64]
    assert_quant_bit_exact(y[rows.to(DEV)], s[rows.to(DEV)], x[rows], what="sampled rows")
