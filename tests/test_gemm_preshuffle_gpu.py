"""GPU parity of the pre-shuffled-weight entry point (gemm_a8w8_blockscale_bpreshuffle) through
the C-ABI: same arithmetic as gemm_a8w8_blockscale, weights in shuffle_weight(…, (16,16)) order and
x_scale column-major (op_tests/test_gemm_a8w8_blockscale.py:100-125)."""

import pytest
import torch

import aiter_amd
from oracle import torch_ref as tr
from tests.test_gemm_gpu import DEV, assert_close_to_f64, make_problem

pytestmark = pytest.mark.gpu


def col_major(xs, form):
    """The two ways callers hand over column-major scales."""
    t = xs.transpose(0, 1).contiguous()
    if form == "buffer":  # transposed data behind a contiguous [M, K/128] shape
        return t.view(*xs.shape)
    return t.transpose(0, 1)  # [M, K/128] view with strides (1, M)


def run_preshuffled(xq, wq, xs, ws, dtype=torch.bfloat16, form="buffer", kernel=None):
    wsh = aiter_amd.shuffle_weight(wq.view(torch.uint8)).view(wq.dtype)
    a = [xq.to(DEV), wsh.to(DEV), col_major(xs.to(DEV), form), ws.to(DEV)]
    if kernel is None:
        out = aiter_amd.gemm_a8w8_blockscale_bpreshuffle(*a, dtype=dtype)
    else:
        out = torch.empty(xq.shape[0], wq.shape[0], dtype=dtype, device=DEV)
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle_ck(*a, out, kernelName=kernel)
    torch.cuda.synchronize()
    return out


SHAPES = [(1, 64, 128), (1, 7168, 2048), (16, 2112, 7168), (64, 24576, 1536), (5, 208, 640), (33, 1008, 896),
          (64, 512, 512), (100, 400, 384), (128, 2112, 1024), (256, 256, 128), (300, 1008, 384), (512, 768, 1024),
          (1024, 2112, 512)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("form", ["buffer", "view"])
def test_matches_oracle_and_plain_layout(m, n, k, form):
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + 3 * n + k, outliers=0.01)
    out = run_preshuffled(xq, wq, xs, ws, form=form)
    assert_close_to_f64(out, xq, wq, xs, ws, f"bpreshuffle {m}x{n}x{k} {form}")
    plain = aiter_amd.gemm_a8w8_blockscale(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV))
    # same products, same scales; at most the grouping of fp32 additions differs between kernels
    assert (out.view(torch.int16) != plain.view(torch.int16)).float().mean().item() < 0.02


@pytest.mark.parametrize("kernel", ["tile_16x256", "tile_64x128", "tile_128x128", "mid_64x64", "mid_64x128", "mid_128x128", "prefill_256x256",
                                    "prefill_256x192", "prefill_256x128", "decode_stream", "mid_128x128:s=2", "mid_64x64:s=2"])
@pytest.mark.parametrize("m", [48, 272])
def test_named_kernels(kernel, m):
    n, k = 1008, 1024
    xq, wq, xs, ws = make_problem(m, n, k, seed=11, outliers=0.01)
    out = run_preshuffled(xq, wq, xs, ws, kernel=kernel)
    assert_close_to_f64(out, xq, wq, xs, ws, f"bpreshuffle {kernel}")
    # the same kernel on the plain layout performs the same operations in the same order
    plain = torch.empty_like(out)
    aiter_amd.gemm_a8w8_blockscale_ck(xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV), plain, splitK=-1,
                                      kernelName=kernel)
    assert torch.equal(out.view(torch.int16), plain.view(torch.int16))


def test_fp16_output_and_out_argument():
    xq, wq, xs, ws = make_problem(32, 512, 768, seed=5)
    wsh = aiter_amd.shuffle_weight(wq.view(torch.uint8)).view(wq.dtype).to(DEV)
    out = torch.full((32, 512), 7.0, dtype=torch.float16, device=DEV)
    ret = aiter_amd.gemm_a8w8_blockscale_bpreshuffle(xq.to(DEV), wsh, col_major(xs.to(DEV), "view"), ws.to(DEV),
                                                     dtype=torch.float16, out=out)
    assert ret.data_ptr() == out.data_ptr()
    assert_close_to_f64(out, xq, wq, xs, ws, "bpreshuffle fp16")


def test_quant_kernel_feeds_it_directly():
    # the 1x128 quantiser with transpose_scale=True writes exactly the x_scale layout this entry reads
    m, n, k = 48, 1024, 2048
    x = tr.make_activation(m, k, seed=3)
    w = tr.make_weight(n, k, seed=4)
    wq, ws = tr.weight_per_128x128_quant(w)
    q = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)
    xq_t, xs_t = q(x.to(DEV), transpose_scale=True)
    xq_r, xs_r = q(x.to(DEV))
    wsh = aiter_amd.shuffle_weight(wq.view(torch.uint8)).view(wq.dtype).to(DEV)
    a = aiter_amd.gemm_a8w8_blockscale_bpreshuffle(xq_t, wsh, xs_t, ws.to(DEV))
    b = aiter_amd.gemm_a8w8_blockscale(xq_r, wq.to(DEV), xs_r, ws.to(DEV))
    assert (a.view(torch.int16) != b.view(torch.int16)).float().mean().item() < 0.02
    assert_close_to_f64(a, xq_r.cpu(), wq, xs_r.cpu(), ws, "quant -> bpreshuffle")


def test_rejects_what_the_layout_cannot_express():
    xq, wq, xs, ws = make_problem(4, 200, 256)  # N not a multiple of 16
    a = [xq.to(DEV), wq.to(DEV), xs.to(DEV), ws.to(DEV)]
    with pytest.raises(RuntimeError, match="N % 16"):
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle(*a)
    xq, wq, xs, ws = make_problem(4, 208, 256)
    bad = torch.empty(4, 3, device=DEV)  # wrong number of scales
    with pytest.raises(RuntimeError, match="column-major"):
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle(xq.to(DEV), wq.to(DEV), bad, ws.to(DEV))


@pytest.mark.parametrize("m,n,k", [(1, 7168, 2048), (16, 2112, 7168), (64, 512, 512), (300, 1008, 384), (1024, 2112, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_asm_spelling_with_and_without_bias(m, n, k, dtype):
    # aiter/ops/gemm_op_a8w8.py:404-430 (csrc/py_itfs_cu/asm_a8w8_blockscale_bpreshuffle.cu:253-266): same
    # operands, out third, optional fp32 bias per column; splitK and the reference's kernel names are its
    # own kernel's tuning and must not change anything here
    xq, wq, xs, ws = make_problem(m, n, k, seed=m + n + k, outliers=0.01)
    wsh = aiter_amd.shuffle_weight(wq.view(torch.uint8)).view(wq.dtype).to(DEV)
    a, b_scale = xq.to(DEV), ws.to(DEV)
    a_scale = col_major(xs.to(DEV), "view")
    base = aiter_amd.gemm_a8w8_blockscale_bpreshuffle(a, wsh, a_scale, b_scale, dtype=dtype)
    out = torch.full((m, n), 3.0, dtype=dtype, device=DEV)
    ret = aiter_amd.gemm_a8w8_blockscale_bpreshuffle_asm(a, wsh, out, a_scale, b_scale, splitK=2,
                                                         kernelName="_ZN5aiter42f8_block_scale_mi350_x128_splitk")
    assert ret.data_ptr() == out.data_ptr()
    assert torch.equal(out.view(torch.int16), base.view(torch.int16))
    g = torch.Generator().manual_seed(7)
    for shape in ((n,), (1, n)):
        bias = torch.randn(shape, generator=g).to(DEV)
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle_asm(a, wsh, out, a_scale, b_scale, bias=bias)
        torch.cuda.synchronize()
        # the definition: the stored result, widened, plus the bias, rounded once more
        want = (base.float() + bias.reshape(1, n)).to(dtype)
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))
        # and against the exact sum: the stored product was already rounded, so the bound follows the
        # product's magnitude, not the (possibly cancelled) sum's
        product, b64 = tr.gemm_a8w8_blockscale_ref_f64(xq, wq, xs, ws), bias.reshape(1, n).double().cpu()
        err = (out.double().cpu() - (product + b64)).abs()
        assert (err <= 1e-2 + 1e-2 * (product.abs() + b64.abs())).all(), f"{m}x{n}x{k}: max error {err.max().item():.3e}"
    with pytest.raises(RuntimeError, match="bias"):
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle_asm(a, wsh, out, a_scale, b_scale, bias=torch.zeros(n + 4, device=DEV))
    with pytest.raises(RuntimeError, match="bias"):
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle_asm(a, wsh, out, a_scale, b_scale,
                                                       bias=torch.zeros(n, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(NotImplementedError):
        aiter_amd.gemm_a8w8_blockscale_bpreshuffle_asm(a, wsh, out, a_scale, b_scale, bpreshuffle=False)
