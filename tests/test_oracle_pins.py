"""CPU: pin the oracle against independent evidence before anything is checked with it.

The reference stores no golden vectors for this path (its tests regenerate random data), so the
pins are: torch CPU library routines (fp8 / bf16 / fp16 casts, F.linear, F.rms_norm), the torch
restatement of the reference's own oracle functions, closed forms and invariants.
"""

import numpy as np
import pytest
import torch

from oracle import c_oracle as co
from oracle import torch_ref as tr

FP8 = torch.float8_e4m3fn


# ---------------------------------------------------------------- conversions


def test_e4m3fn_known_answers():
    ka = [(448.0, 0x7E), (464.0, 0x7E), (465.0, 0x7F), (480.0, 0x7F), (2.0**-9, 0x01), (2.0**-10, 0x00),
          (1.5 * 2.0**-10, 0x01), (3 * 2.0**-10, 0x02), (-0.0, 0x80), (0.0, 0x00), (1.0, 0x38), (-1.0, 0xB8),
          (2.0**-6, 0x08), (0.9375 * 2.0**-6, 0x08), (float("inf"), 0x7F), (-float("inf"), 0xFF),
          (1.0625, 0x38), (1.1875, 0x3A), (1.125, 0x39)]
    got = co.f32_to_e4m3fn(np.array([k for k, _ in ka], dtype=np.float32))
    assert got.tolist() == [v for _, v in ka]
    assert co.f32_to_e4m3fn(np.array([np.nan], dtype=np.float32))[0] & 0x7F == 0x7F


def test_e4m3fn_encode_matches_torch_on_every_rounding_boundary():
    # every value of the top 20 bits (sign, exponent, 11 mantissa bits) x low bits that sit on,
    # just below and just above each possible tie: 6.3 M inputs
    hi = np.arange(1 << 20, dtype=np.uint32) << 12
    lows = np.array([0x000, 0x001, 0x7FF, 0x800, 0x801, 0xFFF], dtype=np.uint32)
    bits = (hi[:, None] | lows[None, :]).reshape(-1)
    f = bits.view(np.float32)
    mine = co.f32_to_e4m3fn(f)
    theirs = torch.from_numpy(f.copy()).to(FP8).view(torch.uint8).numpy()
    assert np.array_equal(mine, theirs)


def test_e4m3fn_decode_all_codes():
    codes = np.arange(256, dtype=np.uint8)
    mine = co.e4m3fn_to_f32(codes)
    theirs = torch.from_numpy(codes).view(FP8).float().numpy()
    nan = np.isnan(theirs)
    assert np.array_equal(np.isnan(mine), nan) and nan.sum() == 2
    assert np.array_equal(mine[~nan].view(np.uint32), theirs[~nan].view(np.uint32))
    # closed form: normals (8+m) * 2^(e-10), subnormals m * 2^-9
    for c in range(0x7F):
        e, m = c >> 3, c & 7
        want = m * 2.0**-9 if e == 0 else (8 + m) * 2.0 ** (e - 10)
        assert mine[c] == np.float32(want)
    # encode(decode(c)) == c for every finite code
    assert np.array_equal(co.f32_to_e4m3fn(mine[~nan]), codes[~nan])


def test_bf16_and_fp16_conversions_all_codes():
    lib = co.lib()
    codes = np.arange(65536, dtype=np.uint16)
    tb = torch.from_numpy(codes.view(np.int16)).view(torch.bfloat16).float().numpy()
    th = torch.from_numpy(codes.view(np.int16)).view(torch.float16).float().numpy()
    for c in range(0, 65536, 1):
        if c % 257 and c not in (0, 1, 0x7F, 0x80, 0x3FF, 0x400, 0x7BFF, 0x7C00, 0x8000, 0xFFFF):
            continue
        a, b = np.float32(lib.oracle_bf16_to_f32(c)), np.float32(lib.oracle_f16_to_f32(c))
        assert a.view(np.uint32) == tb[c].view(np.uint32) or (np.isnan(a) and np.isnan(tb[c]))
        assert b.view(np.uint32) == th[c].view(np.uint32) or (np.isnan(b) and np.isnan(th[c]))
    # f32 -> bf16 rounding against torch on ties and neighbours
    g = np.random.default_rng(0)
    bits = g.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    bits = np.concatenate([bits, (bits & 0xFFFF0000) | 0x8000, (bits & 0xFFFF0000) | 0x7FFF, (bits & 0xFFFF0000) | 0x8001])
    f = bits.view(np.float32)
    f = f[np.isfinite(f)]
    want = torch.from_numpy(f.copy()).bfloat16().view(torch.int16).numpy().view(np.uint16)
    got = np.array([lib.oracle_f32_to_bf16(float(v)) for v in f[:20000]], dtype=np.uint16)
    assert np.array_equal(got, want[:20000])


# ---------------------------------------------------------------- group quant


def _check_quant(x, in_dtype="bf16", group=128):
    yc, sc = co.group_quant(co.codes16(x), in_dtype=in_dtype, group=group)
    yt, st = tr.per_1x128_quant(x, group)
    assert np.array_equal(yc, co.codes8(yt))
    assert np.array_equal(sc.view(np.uint32), st.numpy().view(np.uint32))
    return yc, sc


def test_quant_config1_matches_torch_restatement():
    # benchmark config 1
    _check_quant(tr.make_activation(32, 1024, seed=0))


@pytest.mark.parametrize("seed", range(3))
def test_quant_random_with_outliers(seed):
    _check_quant(tr.make_activation(257, 1536, seed=seed, outlier_frac=0.01))


def test_quant_fp16_and_small_groups():
    g = torch.Generator().manual_seed(4)
    _check_quant((torch.randn(64, 512, generator=g) * 4).half(), in_dtype="fp16")
    _check_quant(tr.make_activation(16, 512, seed=1), group=64)
    _check_quant(tr.make_activation(16, 512, seed=2), group=32)


def test_quant_closed_forms_and_invariants():
    x = tr.make_activation(64, 1024, seed=7)
    y, s = co.group_quant(co.codes16(x))
    xf = x.float().numpy().reshape(64, 8, 128)
    amax = np.abs(xf).max(-1)
    # scale = RN(amax/448) (numpy float32 division is IEEE)
    assert np.array_equal(s.view(np.uint32), (amax / np.float32(448.0)).astype(np.float32).view(np.uint32))
    yy = y.reshape(64, 8, 128)
    # the element attaining amax encodes +-448
    idx = np.abs(xf).argmax(-1)
    top = np.take_along_axis(yy, idx[..., None], -1)[..., 0]
    assert np.all((top & 0x7F) == 0x7E)
    # reconstruction error bounded by half an fp8 ulp of the quotient (ulp <= 32 at the top binade)
    deq = co.e4m3fn_to_f32(yy) * s[..., None]
    q = np.abs(xf / s[..., None])
    ulp = np.maximum(2.0 ** (np.floor(np.log2(np.maximum(q, 2.0**-6))) - 3), 2.0**-9)
    assert np.all(np.abs(deq - xf) <= (0.5 * ulp + 1e-6) * s[..., None] * 1.0001)
    # sign symmetry and group permutation equivariance
    y2, s2 = co.group_quant(co.codes16(-x))
    assert np.array_equal(y2 ^ 0x80, y) and np.array_equal(s2, s)
    perm = np.random.default_rng(0).permutation(64 * 8)
    xg = co.codes16(x).reshape(-1, 128)[perm]
    y3, s3 = co.group_quant(xg)
    assert np.array_equal(y3, y.reshape(-1, 128)[perm]) and np.array_equal(s3[:, 0], s.reshape(-1)[perm])
    # power-of-two amax: exact scale, amax = 448 -> scale 1 and codes are the plain cast
    row = torch.full((1, 128), 3.0).bfloat16()
    row[0, 0] = 448.0
    y4, s4 = co.group_quant(co.codes16(row))
    assert s4[0, 0] == 1.0 and y4[0, 0] == 0x7E and y4[0, 1] == 0x44
    # all-zero group: scale 1 (quant.py:89), codes zero with the sign kept
    z = torch.zeros(1, 128).bfloat16()
    z[0, 3] = -0.0
    y5, s5 = co.group_quant(co.codes16(z))
    assert s5[0, 0] == 1.0 and y5[0, 3] == 0x80 and y5.sum() == 0x80


def test_quant_special_values_match_torch():
    inf, nan = float("inf"), float("nan")
    rows = [
        [1.0, 2.0, inf, -3.0] + [0.5] * 124,
        [1.0, -inf, inf, 0.0] + [0.25] * 124,
        [1.0, nan, 2.0, -3.0] + [0.5] * 124,
        [2.0**-133, 2.0**-133, 2.0**-133 * 3, 0.0] + [0.0] * 124,
        [2.0**-126, -(2.0**-127), 2.0**-130, 0.0] + [2.0**-133] * 124,
        [3.0e38, -3.0e38, 1.0e30, 1.0] + [0.0] * 124,
    ]
    x = torch.tensor(rows, dtype=torch.float32).bfloat16()
    yc, sc = co.group_quant(co.codes16(x))
    yt, st = tr.per_1x128_quant(x)
    assert np.array_equal(yc, co.codes8(yt))
    finite = ~np.isnan(st.numpy()[:, 0])
    assert np.array_equal(sc.view(np.uint32)[finite], st.numpy().view(np.uint32)[finite])
    assert np.isnan(sc[~finite]).all()


# ---------------------------------------------------------------- weight block quant


@pytest.mark.parametrize("n,k", [(512, 1024), (192, 256), (2112, 384), (128, 128)])
def test_weight_block_quant_matches_torch_restatement(n, k):
    w = tr.make_weight(n, k, seed=n)
    wq, ws = tr.weight_per_128x128_quant(w)
    wqc, wsc = co.weight_block_quant(co.codes16(w))
    assert np.array_equal(wqc, co.codes8(wq))
    assert np.array_equal(wsc.view(np.uint32), ws.numpy().view(np.uint32))
    # closed form: per-block scale is amax/448
    blk = w.float()[:128, :128].abs().max().item()
    assert wsc[0, 0] == np.float32(blk) / np.float32(448.0)


# ---------------------------------------------------------------- GEMM


def _problem(m, n, k, seed=0):
    xq, xs = tr.per_1x128_quant(tr.make_activation(m, k, seed=seed))
    wq, ws = tr.weight_per_128x128_quant(tr.make_weight(n, k, seed=seed + 1))
    return xq, wq, xs, ws


def test_gemm_matches_textbook_fp64_and_torch_linear():
    xq, wq, xs, ws = _problem(32, 512, 1024)  # benchmark config 1
    o, ob = co.gemm_blockscale(co.codes8(xq), co.codes8(wq), xs.numpy(), ws.numpy())
    ref64 = tr.gemm_a8w8_blockscale_ref_f64(xq, wq, xs, ws)
    assert np.array_equal(o, ref64.float().numpy())
    ref32 = tr.gemm_a8w8_blockscale_ref(xq, wq, xs, ws)
    assert tr.check_allclose_ratio(torch.from_numpy(o), ref32.float(), 1e-2, 1e-2) == 0.0
    # an independent formulation: per-block integer-exact dot products scaled afterwards
    x = xq.float().double().view(32, 8, 128)
    w = wq.float().double().view(512, 8, 128)
    blockwise = torch.einsum("mbk,nbk->mnb", x, w)
    wsn = ws.double().repeat_interleave(128, dim=0)[:512]
    alt = (blockwise * xs.double()[:, None, :] * wsn[None, :, :]).sum(-1)
    # (the reference rounds each dequantised operand to fp32 first: ~2^-24 relative per factor)
    assert torch.allclose(alt, ref64, rtol=1e-5, atol=1e-5)
    # fp32 sequential accumulation stays within the reference tolerance of the fp64 answer
    o32, _ = co.gemm_blockscale(co.codes8(xq), co.codes8(wq), xs.numpy(), ws.numpy(), accumulate="f32")
    assert np.allclose(o32, o, rtol=1e-2, atol=1e-2)


def test_gemm_ragged_n_and_one_hot():
    xq, wq, xs, ws = _problem(5, 192, 256, seed=3)  # 192 = 128 + 64: ragged last scale block
    o, _ = co.gemm_blockscale(co.codes8(xq), co.codes8(wq), xs.numpy(), ws.numpy())
    assert np.array_equal(o, tr.gemm_a8w8_blockscale_ref_f64(xq, wq, xs, ws).float().numpy())
    # one-hot operands isolate a single (m, n, kb) scale product
    xq0 = np.zeros((4, 256), np.uint8)
    wq0 = np.zeros((192, 256), np.uint8)
    xq0[2, 130] = 0x40
    wq0[150, 130] = 0x34
    xs0 = np.arange(1, 9, dtype=np.float32).reshape(4, 2)
    ws0 = np.arange(10, 14, dtype=np.float32).reshape(2, 2)
    o, _ = co.gemm_blockscale(xq0, wq0, xs0, ws0)
    want = np.float32(2.0 * 0.75) * np.float32(xs0[2, 1] * ws0[1, 1])
    assert o[2, 150] == want and np.count_nonzero(o) == 1


# ---------------------------------------------------------------- RMSNorm


def test_rmsnorm_vs_torch_library_within_one_ulp():
    x = tr.make_activation(64, 7168, seed=3)
    g = torch.Generator().manual_seed(5)
    w = (torch.rand(7168, generator=g) + 0.5).bfloat16()
    ref, _ = tr.rmsnorm_ref(x, w, 1e-6)
    got = co.rmsnorm_bf16(co.codes16(x), co.codes16(w), 1e-6)
    a, b = got.astype(np.int32), co.codes16(ref).astype(np.int32)
    assert np.abs(a - b).max() <= 1 and (a != b).mean() < 1e-4


def test_rmsnorm_closed_form_and_add():
    k = 1024
    for c in (0.5, -2.0, 3.0):
        x = torch.full((1, k), c).bfloat16()
        w = torch.ones(k).bfloat16()
        got = co.rmsnorm_bf16(co.codes16(x), co.codes16(w), 1e-6)
        want = np.float32(c) * (np.float32(1.0) / np.sqrt(np.float32(c * c) + np.float32(1e-6)))
        assert np.all(got == co.codes16(torch.tensor([float(want)]).bfloat16())[0])
    x = tr.make_activation(8, k, seed=1)
    r = tr.make_activation(8, k, seed=2)
    w = (torch.rand(k) + 0.5).bfloat16()
    out, res_out = co.add_rmsnorm_bf16(co.codes16(x), co.codes16(r), co.codes16(w), 1e-6)
    assert np.array_equal(res_out, co.codes16(x + r))
    assert np.array_equal(out, co.rmsnorm_bf16(res_out, co.codes16(w), 1e-6))
    ref, _ = tr.rmsnorm_ref(x, w, 1e-6, residual=r)
    assert np.abs(out.astype(np.int32) - co.codes16(ref).astype(np.int32)).max() <= 1


def test_device_kernel_formula_stays_within_one_rounding_of_the_torch_definition():
    """The reference has two definitions of the 1x128 quant: the torch one (aiter/ops/quant.py:64-94,
    matched here bit for bit) and its HIP kernel's (csrc/kernels/quant_kernels.cu:87-166: amax floored
    at 1e-10, scale = amax * (1/448), multiply by 1/scale, clamp).  They may differ by one ulp in the
    scale and by one code where a quotient sits on a rounding boundary; nothing more."""
    x = tr.make_activation(512, 7168, seed=5, outlier_frac=0.01)
    x[7, 256:384] = 0                      # an all-zero group
    y_t, s_t = tr.per_1x128_quant(x)
    y_d, s_d = tr.per_1x128_quant_device_formula(x)
    st = s_t.numpy().view(np.uint32).astype(np.int64)
    sd = s_d.numpy().view(np.uint32).astype(np.int64)
    zero_group = (7, 2)
    mask = np.ones(st.shape, dtype=bool)
    mask[zero_group] = False
    assert np.abs(st - sd)[mask].max() <= 1, "scales differ by more than one ulp"
    # (about half of the scales do differ by that ulp: amax * fl(1/448) is not the rounded amax / 448)
    assert s_t[zero_group].item() == 1.0 and abs(s_d[zero_group].item() - 1e-10 / 448) < 1e-17
    ct = y_t.view(torch.uint8).numpy().astype(np.int32)
    cd = y_d.view(torch.uint8).numpy().astype(np.int32)
    assert not ct[7, 256:384].any() and not cd[7, 256:384].any()
    differ = ct != cd
    assert differ.mean() < 2e-3, f"{differ.mean():.2e} of the codes differ"
    # every differing pair is a pair of neighbouring codes of the same sign ...
    assert np.all(np.abs(ct[differ] - cd[differ]) == 1)
    # ... and its exact quotient lies within a few fp32 roundings of the midpoint between them
    table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).double().numpy()
    xq = x.double().numpy()[differ]
    sc = np.repeat(s_t.double().numpy(), 128, axis=-1)[differ]
    mid = (table[ct[differ]] + table[cd[differ]]) / 2
    assert np.all(np.abs(xq / sc - mid) <= 4 * 2.0**-24 * np.abs(mid))
