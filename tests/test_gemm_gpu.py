"""GPU parity: block-scale FP8 GEMM through the C-ABI vs the fp32/fp64 oracles."""

import numpy as np
import pytest
import torch

import aiter_amd
from aiter_amd import _ffi
from aiter_amd import dtypes
from oracle import c_oracle as co
from oracle import torch_ref as tr
from tests.helpers import codes8, codes16, guarded_empty

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
RTOL = ATOL = 1e-2  # aiter/test_common.py:482-483, op_tests/test_gemm_a8w8_blockscale.py:118


def make_problem(m, n, k, seed=0, outliers=0.0):
    x = tr.make_activation(m, k, seed=seed, outlier_frac=outliers)
    w = tr.make_weight(n, k, seed=seed + 1)
    xq, xs = tr.per_1x128_quant(x)
    wq, ws = tr.weight_per_128x128_quant(w)
    return xq, wq, xs, ws


def run_gpu(xq, wq, xs, ws, dtype=torch.bfloat16, kernel=None, splitK=0):
    a = [t.to(DEV) for t in (xq, wq, xs, ws)]
    if kernel is None:
        out = aiter_amd.gemm_a8w8_blockscale(*a, dtype=dtype)
    else:
        out = torch.empty(xq.shape[0], wq.shape[0], dtype=dtype, device=DEV)
        aiter_amd.gemm_a8w8_blockscale_ck(*a, out, splitK=splitK, kernelName=kernel)
    torch.cuda.synchronize()
    return out


def assert_close_to_f64(out, xq, wq, xs, ws, what=""):
    ref = tr.gemm_a8w8_blockscale_ref_f64(xq, wq, xs, ws)
    o = out.cpu().double()
    err = (o - ref).abs()
    bound = ATOL + RTOL * ref.abs()
    bad = (err > bound).sum().item()
    assert bad == 0, f"{what}: {bad} of {o.numel()} outside rtol=atol=1e-2, max abs err {err.max().item():.4g}"
    # much tighter in practice: bf16 rounding (2^-9 relative) plus fp32 accumulation noise
    rel = err.max().item() / max(ref.abs().max().item(), 1e-30)
    assert rel < 6e-3, f"{what}: max error / max |ref| = {rel:.3g}"


def test_config1_plumbing():
    # benchmark config 1: [32,1024] x [512,1024]^T, seed 0
    xq, wq, xs, ws = make_problem(32, 512, 1024, seed=0)
    out = run_gpu(xq, wq, xs, ws)
    assert out.shape == (32, 512) and out.dtype == torch.bfloat16
    ref32 = tr.gemm_a8w8_blockscale_ref(xq, wq, xs, ws)
    assert tr.check_allclose_ratio(out.cpu(), ref32, RTOL, ATOL) == 0.0
    assert_close_to_f64(out, xq, wq, xs, ws, "config1")
    o64, ob = co.gemm_blockscale(codes8(xq), codes8(wq), xs.numpy(), ws.numpy())
    # against the scalar C oracle (fp64 accumulation): nearly all bf16 codes identical; the rest
    # differ by fp32 accumulation noise, which is many bf16 ulps only where sums cancel to ~0
    d = np.abs(codes16(out).astype(np.int32) - ob.astype(np.int32))
    assert (d != 0).mean() < 0.02
    assert np.all(np.abs(out.cpu().float().numpy() - o64) <= 2.0**-8 * np.abs(o64) + 1e-4)


@pytest.mark.parametrize("kernel", [None, "tile_16x256", "tile_64x128", "tile_128x128", "mid_64x64", "mid_64x128",
                                    "mid_128x128", "prefill_256x256", "prefill_256x192", "prefill_256x128", "decode_stream"])
@pytest.mark.parametrize(
    "m,n,k",
    [(1, 128, 128), (1, 2112, 512), (16, 256, 1024), (17, 384, 256), (64, 2112, 1024), (130, 520, 384), (257, 1000, 256)],
)
def test_shapes_and_tiles(kernel, m, n, k):
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n + k)
    out = run_gpu(xq, wq, xs, ws, kernel=kernel)
    assert_close_to_f64(out, xq, wq, xs, ws, f"{kernel} {m}x{n}x{k}")


@pytest.mark.parametrize("name", ["prefill_256x256", "prefill_256x192", "prefill_256x128"])
@pytest.mark.parametrize("m,n,k", [(256, 256, 128), (512, 768, 1024), (300, 1000, 384), (1024, 2112, 512), (257, 260, 256)])
def test_prefill_kernel_shapes(m, n, k, name):
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n + k, outliers=0.01)
    out = run_gpu(xq, wq, xs, ws, kernel=name)
    assert_close_to_f64(out, xq, wq, xs, ws, f"prefill {m}x{n}x{k}")
    # same bits as the generic tile kernel (same per-block products, same accumulation order
    # over K blocks); the library's own choice for the size may be a kernel that splits K
    # between waves, which regroups the fp32 additions
    auto = run_gpu(xq, wq, xs, ws)
    tile = run_gpu(xq, wq, xs, ws, kernel="tile_128x128")
    assert torch.equal(out.view(torch.int16), tile.view(torch.int16))
    assert (auto.view(torch.int16) != tile.view(torch.int16)).float().mean().item() < 0.02
    assert_close_to_f64(auto, xq, wq, xs, ws, f"auto {m}x{n}x{k}")


def test_one_hot_isolates_single_scale_product():
    # x has a single non-zero element (m0,k0), w a single non-zero element (n0,k0):
    # out[m0,n0] must be exactly bf16(x*w*xs*ws) and everything else exactly zero.
    m, n, k = 48, 384, 512
    xq = torch.zeros(m, k, dtype=torch.uint8)
    wq = torch.zeros(n, k, dtype=torch.uint8)
    g = torch.Generator().manual_seed(0)
    xs = torch.rand(m, k // 128, generator=g) + 0.5
    ws = torch.rand((n + 127) // 128, k // 128, generator=g) + 0.5
    cases = [(0, 0, 0), (47, 383, 511), (17, 200, 300), (31, 129, 127), (5, 255, 128)]
    for m0, n0, k0 in cases:
        xq.zero_(); wq.zero_()
        xq[m0, k0] = 0x40  # 2.0
        wq[n0, k0] = 0xB4  # -1.25 ... sign + exponent 6, mantissa 4 -> -(1.5)*2^-1 = -0.75
        out = run_gpu(xq.view(dtypes.fp8), wq.view(dtypes.fp8), xs, ws).cpu().float()
        a = torch.tensor([0x40], dtype=torch.uint8).view(dtypes.fp8).float().item()
        b = torch.tensor([0xB4], dtype=torch.uint8).view(dtypes.fp8).float().item()
        expect = np.float32(a * b) * (xs[m0, k0 // 128].numpy() * ws[n0 // 128, k0 // 128].numpy())
        assert out[m0, n0].item() == torch.tensor(float(expect)).bfloat16().float().item(), (m0, n0, k0)
        out[m0, n0] = 0
        assert torch.count_nonzero(out) == 0, (m0, n0, k0)


def test_identity_scales_reduce_to_plain_fp8_gemm():
    m, n, k = 64, 256, 512
    g = torch.Generator().manual_seed(3)
    xq = torch.randint(0, 256, (m, k), generator=g, dtype=torch.int32).to(torch.uint8)
    wq = torch.randint(0, 256, (n, k), generator=g, dtype=torch.int32).to(torch.uint8)
    xq[(xq & 0x7F) == 0x7F] = 0x10  # no NaN codes
    wq[(wq & 0x7F) == 0x7F] = 0x10
    xq[(xq & 0x78) > 0x50] &= 0x8F  # keep magnitudes small so fp32 sums stay exact-ish
    wq[(wq & 0x78) > 0x50] &= 0x8F
    xs = torch.ones(m, k // 128)
    ws = torch.ones(n // 128, k // 128)
    out = run_gpu(xq.view(dtypes.fp8), wq.view(dtypes.fp8), xs, ws).cpu().float()
    ref = (xq.view(dtypes.fp8).double() @ wq.view(dtypes.fp8).double().T)
    # bf16 rounding (2^-9) plus fp32 accumulation noise on sums of magnitude <= ~1e5
    assert torch.allclose(out.double(), ref, rtol=2**-8, atol=0.05)


def test_linear_in_x_scale():
    # doubling x_scale (exact in fp32) doubles every output bit-exactly (power-of-two scaling)
    xq, wq, xs, ws = make_problem(40, 384, 768, seed=5)
    a = run_gpu(xq, wq, xs, ws).cpu().float()
    b = run_gpu(xq, wq, xs * 2, ws).cpu().float()
    assert torch.equal(a * 2, b)


def test_fp16_output():
    xq, wq, xs, ws = make_problem(33, 256, 512, seed=8)
    out = run_gpu(xq, wq, xs, ws, dtype=torch.float16)
    assert out.dtype == torch.float16
    ref = tr.gemm_a8w8_blockscale_ref_f64(xq, wq, xs, ws)
    assert torch.allclose(out.cpu().double(), ref, rtol=RTOL, atol=ATOL)


def test_strided_operands_and_guard_bands():
    m, n, k = 24, 300, 512
    xq, wq, xs, ws = make_problem(m, n, k, seed=12)
    xbig = torch.zeros(m, k + 256, dtype=torch.uint8, device=DEV)
    wbig = torch.zeros(n, k + 128, dtype=torch.uint8, device=DEV)
    xbig[:, :k] = xq.view(torch.uint8).to(DEV)
    wbig[:, :k] = wq.view(torch.uint8).to(DEV)
    out, chk = guarded_empty((m, n), torch.bfloat16, DEV)
    aiter_amd.gemm_a8w8_blockscale_ck(
        xbig[:, :k].view(dtypes.fp8), wbig[:, :k].view(dtypes.fp8), xs.to(DEV), ws.to(DEV), out
    )
    torch.cuda.synchronize()
    chk()
    assert_close_to_f64(out, xq, wq, xs, ws, "strided")


@pytest.mark.parametrize("m,n,k,splitk", [(1, 64, 128, 0), (5, 200, 512, 0), (5, 200, 512, 2), (16, 2112, 1024, 3),
                                            (17, 384, 4096, -1), (33, 130, 2304, 1), (48, 1000, 7168, -1),
                                            (64, 256, 6144, 4), (64, 8192, 256, -1)])
def test_decode_stream_kernel(m, n, k, splitk):
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n + k + 1, outliers=0.01)
    out = run_gpu(xq, wq, xs, ws, kernel="decode_stream", splitK=splitk)
    assert_close_to_f64(out, xq, wq, xs, ws, f"decode_stream {m}x{n}x{k} splitK={splitk}")
    # K splitting only regroups the fp32 additions: still within a few fp32 ulps of one chunk,
    # and bit-identical from run to run (partials are added in a fixed order)
    again = run_gpu(xq, wq, xs, ws, kernel="decode_stream", splitK=splitk)
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))
    one = run_gpu(xq, wq, xs, ws, kernel="tile_16x256")
    assert (out.view(torch.int16) != one.view(torch.int16)).float().mean().item() < 0.02


@pytest.mark.parametrize("m,n,k,tuning", [
    (3, 4096, 1024, "r=2,g=7,p=2"),        # 128 row groups over 7 workgroups, partial tiles flushed every 2
    (20, 3000, 640, "r=1,g=5,p=3"),        # K not a multiple of 512, ragged N, two m tiles
    (64, 2112, 7168, "r=2,s=2,g=4"),       # K split across workgroups, several steps per wave, 17 groups each
    (40, 1536, 2048, "r=2,s=2,w=2,g=3"),   # two waves per workgroup
    (1, 24576, 1536, "g=16"),              # 48 row groups per workgroup, weights prefetched group by group
    (64, 512, 512, "w=1"),                 # one wave: nothing to add across waves
    (33, 1000, 896, "r=2,s=7"),            # one step per K range, last range short
])
def test_decode_work_split_overrides(m, n, k, tuning):
    # the work split is a launch-time choice; every split must give the same answer up to fp32
    # regrouping, and the same bits from run to run
    xq, wq, xs, ws = make_problem(m, n, k, seed=m * 7 + n + k, outliers=0.01)
    name = "decode_stream:" + tuning
    out = run_gpu(xq, wq, xs, ws, kernel=name, splitK=-1)
    assert_close_to_f64(out, xq, wq, xs, ws, f"{name} {m}x{n}x{k}")
    again = run_gpu(xq, wq, xs, ws, kernel=name, splitK=-1)
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))
    auto = run_gpu(xq, wq, xs, ws, kernel="decode_stream", splitK=-1)
    assert (out.view(torch.int16) != auto.view(torch.int16)).float().mean().item() < 0.02


@pytest.mark.parametrize("m,n,k,tuning", [
    (128, 7168, 2048, ""),              # weights resident, four chunks of 32 rows
    (65, 520, 512, ""),                 # ragged last chunk, ragged N
    (200, 2112, 7168, ""),              # long K: several steps per wave, chunks of 64 rows
    (130, 1024, 384, "r=2,g=3"),        # K not a multiple of 512, several row groups per workgroup
    (256, 1536, 1536, "r=2,s=3"),       # K split across workgroups, chunked
    (512, 256, 2048, "r=1"),            # the most rows the kernel takes
    (96, 24576, 1536, ""),              # three row groups per workgroup x three chunks
])
def test_decode_stream_more_than_64_rows(m, n, k, tuning):
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n + k, outliers=0.01)
    name = "decode_stream" + (":" + tuning if tuning else "")
    out = run_gpu(xq, wq, xs, ws, kernel=name, splitK=-1)
    assert_close_to_f64(out, xq, wq, xs, ws, f"{name} {m}x{n}x{k}")
    again = run_gpu(xq, wq, xs, ws, kernel=name, splitK=-1)
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))
    one = run_gpu(xq, wq, xs, ws, kernel="tile_128x128")
    assert (out.view(torch.int16) != one.view(torch.int16)).float().mean().item() < 0.02


@pytest.mark.parametrize("m,n,k,splitk", [(128, 128, 128, 0), (200, 520, 1024, -1), (512, 2112, 7168, -1), (300, 1000, 2304, 2),
                                            (1024, 4096, 1536, 0), (129, 130, 1024, 3), (256, 7168, 2048, -1)])
@pytest.mark.parametrize("kernel", ["mid_64x64", "mid_64x128", "mid_128x128", "mid_auto"])
def test_mid_kernel(kernel, m, n, k, splitk):
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n + k + 2, outliers=0.01)
    out = run_gpu(xq, wq, xs, ws, kernel=kernel, splitK=splitk)
    assert_close_to_f64(out, xq, wq, xs, ws, f"{kernel} {m}x{n}x{k} splitK={splitk}")
    again = run_gpu(xq, wq, xs, ws, kernel=kernel, splitK=splitk)
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))
    tile = run_gpu(xq, wq, xs, ws, kernel="tile_128x128")
    if splitk == 0:  # one K range: same products, same accumulation order as the generic tile kernel
        assert torch.equal(out.view(torch.int16), tile.view(torch.int16))
    else:
        assert (out.view(torch.int16) != tile.view(torch.int16)).float().mean().item() < 0.02


@pytest.mark.parametrize("kernel", ["mid_64x64:s=1", "mid_64x128:s=1", "mid_128x128:s=1"])
@pytest.mark.parametrize("m,n,dtype,shift", [
    (130, 520, torch.float16, 0),   # rows 16-byte aligned: the tile goes through LDS and all eight waves store it
    (130, 260, torch.bfloat16, 0),  # rows 8-byte aligned only: the multiplying waves store their fragments
    (70, 1002, torch.bfloat16, 0),  # rows 4-byte aligned: element-wise stores at the ragged edge
    (70, 520, torch.bfloat16, 4),   # 16-byte aligned rows behind a base that is not: fragment stores again
])
def test_mid_kernel_output_paths(kernel, m, n, dtype, shift):
    k = 384
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n)
    a = [t.to(DEV) for t in (xq, wq, xs, ws)]
    flat = torch.full((m * n + 64,), float("nan"), dtype=dtype, device=DEV)
    out = flat[shift : shift + m * n].view(m, n)
    aiter_amd.gemm_a8w8_blockscale_ck(*a, out, splitK=0, kernelName=kernel)
    torch.cuda.synchronize()
    assert_close_to_f64(out, xq, wq, xs, ws, f"{kernel} {m}x{n} {dtype} +{shift}")
    assert torch.isnan(flat[:shift]).all() and torch.isnan(flat[shift + m * n :]).all()  # nothing outside the matrix
    base = torch.empty(m, n, dtype=dtype, device=DEV)
    aiter_amd.gemm_a8w8_blockscale_ck(*a, base, splitK=0, kernelName="tile_128x128")
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))


@pytest.mark.parametrize("kblocks", [1, 2, 3, 4, 5, 6, 7, 8, 9, 11, 12, 13, 18])
def test_mid_64x64_lone_workgroups_every_k_length(kblocks):
    # no more workgroups than compute units: the 64x64 tile runs its six-stage ring, filled two K
    # blocks at a time; every K length up to and past two trips round the ring, odd and even
    m, n, k = 100, 200, 128 * kblocks
    xq, wq, xs, ws = make_problem(m, n, k, seed=900 + kblocks, outliers=0.01)
    out = run_gpu(xq, wq, xs, ws, kernel="mid_64x64", splitK=0)
    assert_close_to_f64(out, xq, wq, xs, ws, f"mid_64x64 {m}x{n}x{k}")
    tile = run_gpu(xq, wq, xs, ws, kernel="tile_128x128")
    assert torch.equal(out.view(torch.int16), tile.view(torch.int16))
    if kblocks >= 8:
        halves = run_gpu(xq, wq, xs, ws, kernel="mid_64x64:s=2", splitK=-1)
        assert_close_to_f64(halves, xq, wq, xs, ws, f"mid_64x64:s=2 {m}x{n}x{k}")


@pytest.mark.parametrize("name", ["mid_128x128:s=3", "mid_64x64:s=5", "mid_64x128:s=7", "mid_auto:s=2"])
@pytest.mark.parametrize("m,n,k,dtype", [(200, 520, 2304, torch.bfloat16), (128, 2112, 7168, torch.float16)])
def test_mid_kernel_pinned_k_ranges(name, m, n, k, dtype):
    # any number of K ranges, not only powers of two; partial tiles summed in range order by a second launch
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + k, outliers=0.01)
    out = run_gpu(xq, wq, xs, ws, dtype=dtype, kernel=name, splitK=-1)
    assert_close_to_f64(out, xq, wq, xs, ws, f"{name} {m}x{n}x{k}")
    again = run_gpu(xq, wq, xs, ws, dtype=dtype, kernel=name, splitK=-1)
    assert torch.equal(out.view(torch.int16), again.view(torch.int16))


def test_automatic_choice_on_random_shapes():
    # the kernel family, tile and number of K ranges all come from a cost model: whatever it picks must be right
    g = torch.Generator().manual_seed(2024)
    shapes = []
    while len(shapes) < 40:
        m = int(torch.randint(1, 700, (1,), generator=g))
        n = int(torch.randint(1, 2600, (1,), generator=g))
        k = 128 * int(torch.randint(1, 40, (1,), generator=g))
        if len(shapes) % 3 == 0:
            n = (n + 15) // 16 * 16      # the common case: N a multiple of 16
        if m * n * k > 6e8:              # keeps the fp64 oracle quick
            continue
        shapes.append((m, n, k))
    for (m, n, k) in shapes:
        xq, wq, xs, ws = make_problem(m, n, k, seed=m * 7 + n, outliers=0.01)
        out = run_gpu(xq, wq, xs, ws)
        assert_close_to_f64(out, xq, wq, xs, ws, f"auto {m}x{n}x{k}")
        again = run_gpu(xq, wq, xs, ws)
        assert torch.equal(out.view(torch.int16), again.view(torch.int16)), f"auto {m}x{n}x{k} not repeatable"


def test_mid_kernel_rejects_malformed_range_count():
    for name in ("mid_128x128:s=0", "mid_128x128:s=x", "mid_128x128:q=2", "mid_32x32"):
        with pytest.raises(RuntimeError, match="unknown kernelName"):
            run_gpu(*make_problem(128, 256, 256), kernel=name)


def test_decode_stream_rejects_more_than_512_rows():
    with pytest.raises(RuntimeError, match="decode_stream handles"):
        run_gpu(*make_problem(513, 256, 256), kernel="decode_stream")


def test_decode_split_k_repeated_calls_leave_tickets_clean():
    # the split-K tickets must return to zero after every call, also when shapes change
    for (m, n, k) in [(16, 2112, 7168), (1, 2112, 7168), (64, 2112, 7168), (16, 7168, 2048), (16, 2112, 7168)]:
        xq, wq, xs, ws = make_problem(m, n, k, seed=n + k)
        a = run_gpu(xq, wq, xs, ws)
        b = run_gpu(xq, wq, xs, ws)
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))
        assert_close_to_f64(a, xq, wq, xs, ws, f"repeat {m}x{n}x{k}")


@pytest.mark.parametrize("m", [1, 16, 64])
@pytest.mark.parametrize("n,k", [(7168, 2048), (24576, 1536), (2112, 7168)])
def test_decode_shapes(m, n, k):
    # benchmark config 3
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n)
    out = run_gpu(xq, wq, xs, ws)
    ref32 = tr.gemm_a8w8_blockscale_ref(xq, wq, xs, ws)
    assert tr.check_allclose_ratio(out.cpu(), ref32, RTOL, ATOL) == 0.0
    assert_close_to_f64(out, xq, wq, xs, ws, f"decode {m}x{n}x{k}")


@pytest.mark.parametrize("m,n,k", [(17, 24576, 1536), (40, 2112, 7168), (64, 576, 7168), (33, 32768, 512), (8, 32768, 512)])
def test_small_batches_that_the_library_sends_to_the_mid_tilings(m, n, k):
    # below 65 rows the choice between the weight-streaming kernel and the mid_* tilings is by modelled
    # duration; these go to the tilings (one 64-row tile, mostly padding rows that are never stored)
    assert _ffi.gemm_choice(m, n, k).startswith("mid_")
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n + k)
    out = run_gpu(xq, wq, xs, ws)
    assert_close_to_f64(out, xq, wq, xs, ws, f"small batch {m}x{n}x{k}")
    dev = [t.to(DEV) for t in (xq, wq, xs, ws)]
    stream = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    aiter_amd.gemm_a8w8_blockscale_ck(*dev, stream, splitK=-1, kernelName="decode_stream")
    # same products, fp32 sums grouped differently: a few results round to the neighbouring 16-bit value
    assert (out.to(DEV).view(torch.int16) != stream.view(torch.int16)).float().mean().item() < 0.05
    wsh = aiter_amd.shuffle_weight(dev[1].view(torch.uint8)).view(dev[1].dtype)
    assert _ffi.gemm_choice(m, n, k, True).startswith("mid_")
    pre = aiter_amd.gemm_a8w8_blockscale_bpreshuffle(dev[0], wsh, dev[2].t().contiguous().t(), dev[3])
    assert torch.equal(pre.view(torch.int16), out.to(DEV).view(torch.int16))


def test_fused_config_shape_sampled_rows():
    # benchmark config 5 GEMM: [2048,7168] x [4096,7168]^T; 64 sampled rows vs fp32 torch
    m, n, k = 2048, 4096, 7168
    xq, wq, xs, ws = make_problem(m, n, k, seed=0)
    out = run_gpu(xq, wq, xs, ws)
    rows = torch.randperm(m, generator=torch.Generator().manual_seed(2))[:64]
    ref = tr.gemm_a8w8_blockscale_ref(xq[rows], wq, xs[rows], ws)
    assert tr.check_allclose_ratio(out.cpu()[rows], ref, RTOL, ATOL) == 0.0


@pytest.mark.parametrize("m,n,k", [(8, 2112, 1024), (130, 4096, 7168), (1000, 2112, 2048), (2048, 4096, 1024)])
def test_kernel_choice_query_names_what_runs(m, n, k):
    # naming the kernel the query reports gives the bits the automatic choice gives
    xq, wq, xs, ws = (t.to(DEV) for t in make_problem(m, n, k, seed=17))
    cfg = aiter_amd.get_CKGEMM_config(m, n, k)
    auto = aiter_amd.gemm_a8w8_blockscale(xq, wq, xs, ws)
    named = torch.empty_like(auto)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, named, splitK=-1, kernelName=cfg["kernelName"])
    assert torch.equal(auto, named), cfg


def _gpu_problem(m, n, k, seed, outliers=False):
    """Operands made on the GPU (too big for the CPU helpers to be quick): x ~ N(0,1), optionally
    1 % of channels x50, quantised 1x128; w ~ N(0,0.02) quantised per 128x128 block.  Both
    quantisers are checked bit for bit against the oracle in their own tests."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.randn(m, k, generator=g, device=DEV)
    if outliers:
        x[:, torch.randperm(k, generator=g, device=DEV)[: max(1, k // 100)]] *= 50.0
    xq, xs = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(x.bfloat16(), quant_dtype=dtypes.fp8)
    del x
    w = (torch.randn(n, k, generator=g, device=DEV) * 0.02).bfloat16()
    wq, ws = aiter_amd.weight_per_128x128_quant(w, quant_dtype=dtypes.fp8)
    return xq, wq, xs, ws


def _check_rows_against_f64(out, xq, wq, xs, ws, rows, what):
    ref = tr.gemm_a8w8_blockscale_ref_f64(xq[rows].cpu(), wq.cpu(), xs[rows].cpu(), ws.cpu())
    o = out[rows].cpu().double()
    err = (o - ref).abs()
    bad = (err > ATOL + RTOL * ref.abs()).sum().item()
    assert bad == 0, f"{what}: {bad} of {o.numel()} outside rtol=atol=1e-2, max abs err {err.max().item():.4g}"


@pytest.mark.parametrize("m,n,k,expect", [
    (4096, 2112, 1024, "prefill_256x192"),       # eleven full 192-wide tiles per row of tiles, one round
    (2048, 2112, 7168, "prefill_256x192:s=2"),   # the same tiles with two K ranges each
    (8192, 2880, 512, "prefill_256x192"),        # 480 tiles on 256 workgroups: a second tile per workgroup
    (1536, 7168, 2048, "prefill_256x192"),       # 192 does not divide N: the last column of tiles is a third full
    (1024, 7168, 2048, "prefill_256x128"),       # half-width tiles where the wide ones cover 112 compute units
    (200, 24576, 1536, "prefill_256x128"),       # ... with a ragged row of tiles
])
def test_narrow_prefill_tiles_as_the_library_chooses_them(m, n, k, expect):
    assert _ffi.gemm_choice(m, n, k) == expect
    xq, wq, xs, ws = _gpu_problem(m, n, k, seed=m + n + k, outliers=True)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, out, splitK=-1)
    tile = torch.empty_like(out)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, tile, kernelName="tile_128x128")
    torch.cuda.synchronize()
    if ":s=" in expect:  # K ranges regroup the fp32 additions
        assert (out.view(torch.int16) != tile.view(torch.int16)).float().mean().item() < 0.02
    else:               # same products, same order over K blocks: same bits as the generic kernel
        assert torch.equal(out.view(torch.int16), tile.view(torch.int16))
    rows = torch.tensor(sorted({r for r in (0, 15, 16, 63, 64, 255, 256, m // 2, m - 1) if r < m}), device=DEV)
    _check_rows_against_f64(out, xq, wq, xs, ws, rows, f"{expect} {m}x{n}x{k}")
    # pre-shuffled weights: the same kernel on the other layout gives the same bits
    wsh = aiter_amd.shuffle_weight(wq.view(torch.uint8)).view(wq.dtype)
    pre = torch.empty_like(out)
    aiter_amd.gemm_a8w8_blockscale_bpreshuffle_ck(xq, wsh, xs.t().contiguous().view(*xs.shape), ws, pre,
                                                  kernelName=expect)
    named = torch.empty_like(out)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, named, splitK=-1, kernelName=expect)
    torch.cuda.synchronize()
    assert torch.equal(pre.view(torch.int16), named.view(torch.int16))


@pytest.mark.parametrize("m,n,k", [(4352, 4096, 256), (4352, 4352, 128), (4100, 4360, 256)])
def test_prefill_kernel_more_tiles_than_compute_units(m, n, k):
    # 272 / 289 / 306 tiles of 256x256 on 256 compute units: workgroups take a second tile (a
    # multiple of 8 tiles with the per-XCD renumbering, not a multiple, ragged edges)
    xq, wq, xs, ws = _gpu_problem(m, n, k, seed=m + n + k)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, out, kernelName="prefill_256x256")
    tile = torch.empty_like(out)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, tile, kernelName="tile_128x128")
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), tile.view(torch.int16))
    rows = torch.tensor([0, 255, 256, 2047, 4095, 4096, m - 1], device=DEV)
    _check_rows_against_f64(out, xq, wq, xs, ws, rows, f"prefill {m}x{n}x{k}")


@pytest.mark.parametrize("layout", ["plain", "preshuffled"])
def test_config4_full_size(layout):
    # benchmark config 4: M=8192, N=36864, K=7168 through the library's own kernel choice.  Every
    # output is compared bit for bit with the generic tile kernel (same products, same order of
    # additions), and 72 rows x all N with the fp64 reference on the CPU: two rows out of each of the
    # 32 tiles of 256 rows, 96 rows apart (another 64-row wave quarter and the other 32-row half of
    # it), at offsets that walk through all 16 lanes and 4 accumulator rows, plus the corners.
    m, n, k = 8192, 36864, 7168
    xq, wq, xs, ws = _gpu_problem(m, n, k, seed=4, outliers=True)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    if layout == "preshuffled":
        xs_t = xs.t().contiguous().t()  # column-major x_scale, as the quantiser's transpose_scale=True gives
        wsh = aiter_amd.shuffle_weight(wq.view(torch.uint8)).view(wq.dtype)
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle_ck(xq, wsh, xs_t, ws, out)
        del wsh
    else:
        aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, out, splitK=-1)
    tile = torch.empty_like(out)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, tile, kernelName="tile_128x128")
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), tile.view(torch.int16))
    del tile
    picked = {0, 1, 255, 256, 4095, 4096, 8190, 8191}
    for t in range(m // 256):
        r = (t * 37 + 5) % 256
        picked |= {t * 256 + r, t * 256 + (r + 96) % 256}
    assert len(picked) >= 64
    rows = torch.tensor(sorted(picked), device=DEV)
    _check_rows_against_f64(out, xq, wq, xs, ws, rows, f"config 4 {layout}")


@pytest.mark.parametrize("name", ["prefill_256x256", "prefill_256x192", "prefill_256x128", "prefill_256x256:s=3",
                                  "mid_128x128", "mid_64x128", "mid_64x64", "mid_128x128:s=3", "mid_64x64:s=3"])
@pytest.mark.parametrize("k", [2560, 1152])  # 20 K blocks (x_scale fetched four blocks at a time), 9 (one at a time)
def test_x_scale_in_windows_and_rows_not_16_byte_aligned(k, name):
    # Row-major x_scale reaches the mid_* and prefill_* kernels four K blocks per load where its rows are
    # 16-byte aligned.  The same values at an address 4 bytes past a 16-byte boundary must take the loads of
    # one block each and give the same bits; with three K ranges of 20 blocks (7 + 7 + 6) the ranges start
    # inside a window.
    m, n = 600, 1000
    xq, wq, xs, ws = _gpu_problem(m, n, k, seed=k, outliers=True)
    flat = torch.empty(xs.numel() + 1, dtype=torch.float32, device=DEV)
    shifted = flat[1:].view(xs.shape)
    shifted.copy_(xs)
    assert shifted.data_ptr() % 16 == 4 and shifted.is_contiguous()
    a = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    b = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, a, kernelName=name)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, shifted, ws, b, kernelName=name)
    tile = torch.empty_like(a)
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, tile, kernelName="tile_128x128")
    torch.cuda.synchronize()
    assert torch.equal(a.view(torch.int16), b.view(torch.int16))
    if ":s=" in name:  # K ranges regroup the fp32 additions
        assert (a.view(torch.int16) != tile.view(torch.int16)).float().mean().item() < 0.02
        rows = torch.tensor([0, 1, 255, 300, m - 1], device=DEV)
        _check_rows_against_f64(a, xq, wq, xs, ws, rows, f"{name} {m}x{n}x{k}")
    else:
        assert torch.equal(a.view(torch.int16), tile.view(torch.int16))


@pytest.mark.parametrize("m,n,k,name", [
    (512, 768, 2048, "prefill_256x256:s=2"),   # 6 tiles x 2 ranges of 8 K blocks
    (300, 1000, 1408, "prefill_256x256:s=3"),  # ragged tiles, 11 K blocks as 4 + 4 + 3
    (256, 256, 4096, "prefill_256x256:s=4"),   # one tile, four workgroups
    (512, 768, 2048, "prefill_256x128:s=2"),   # half-width tiles: 12 tiles x 2 ranges
    (300, 1000, 1408, "prefill_256x128:s=3"),
    (512, 2112, 2048, "prefill_256x192:s=2"),  # eleven full 192-wide tiles per row of tiles, two scale blocks per wave
    (300, 1000, 1408, "prefill_256x192:s=3"),
    (512, 768, 2560, "prefill_256x256:s=3"),   # 20 K blocks as 7 + 7 + 6: the ranges start inside a window of four x_scale blocks
    (2048, 4096, 7168, ""),                    # benchmark config 5's GEMM: the library's own choice (2 ranges)
])
def test_prefill_kernel_k_ranges_across_workgroups(m, n, k, name):
    xq, wq, xs, ws = _gpu_problem(m, n, k, seed=m + n + k, outliers=True)
    outs = []
    for _ in range(3):  # the tickets must be back at zero after every launch
        out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
        if name:
            aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, out, kernelName=name)
        else:
            aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, out, splitK=-1)
        outs.append(out)
    tile = torch.empty_like(outs[0])
    aiter_amd.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, tile, kernelName="tile_128x128")
    torch.cuda.synchronize()
    # the ranges are added in range order whichever workgroup finishes last: same bits every time
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    assert torch.equal(outs[0].view(torch.int16), outs[2].view(torch.int16))
    # against one workgroup per tile only the grouping of the fp32 additions differs
    assert (outs[0].view(torch.int16) != tile.view(torch.int16)).float().mean().item() < 0.02
    rows = torch.tensor(sorted({0, 1, 255, m // 2, m - 1}), device=DEV)
    _check_rows_against_f64(outs[0], xq, wq, xs, ws, rows, f"{name or 'auto'} {m}x{n}x{k}")
