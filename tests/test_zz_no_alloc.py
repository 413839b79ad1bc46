"""GPU: gemm_a8w8_blockscale_noalloc, the entry point that takes its split-K scratch from the
library's fixed device buffer and allocates nothing, gives what gemm_a8w8_blockscale gives, bit
for bit, on two calls in a row (the second with a smaller input: the buffer keeps the first call's
contents), and rejects a problem whose kernel needs more scratch than the buffer holds."""

import pytest
import torch

import aiter_amd
from aiter_amd import _ffi
from tests.test_gemm_gpu import assert_close_to_f64, make_problem

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def both(problem, m, n, split=-1, kernel=""):
    """(allocating entry point's result, no-alloc entry point's result); the no-alloc call goes first and
    the driver's count of free device memory must not move across it (torch's own statistics never see
    a hipMalloc made inside the library)."""
    a = [t.to(DEV) for t in problem]
    want = torch.empty(m, n, dtype=torch.bfloat16, device=DEV)
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    _ffi.call("gemm_a8w8_blockscale_noalloc", *a, got, split, kernel)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the no-alloc entry point changed the free device memory"
    _ffi.call("gemm_a8w8_blockscale", *a, want, split, kernel)
    return want, got


def test_two_calls_in_a_row_match_the_allocating_entry_point():
    # both shapes take the weight-streaming kernel with K split across workgroups: fp32 partial
    # tiles and tickets live in the scratch buffer
    first, second = (16, 1024, 7168), (8, 512, 4096)
    for m, n, k in (first, second):
        assert _ffi.gemm_choice(m, n, k) == "decode_stream"
    p1, p2 = make_problem(*first, seed=71), make_problem(*second, seed=72)
    w1, g1 = both(p1, first[0], first[1])
    w2, g2 = both(p2, second[0], second[1])
    torch.cuda.synchronize()
    assert torch.equal(g1.view(torch.int16), w1.view(torch.int16)), "first call differs"
    assert torch.equal(g2.view(torch.int16), w2.view(torch.int16)), "second (smaller) call differs"
    assert_close_to_f64(g1, *p1, "noalloc 16x1024x7168")
    assert_close_to_f64(g2, *p2, "noalloc 8x512x4096")


def test_two_launch_kernel_family_and_named_splits():
    # mid_* kernels: partial tiles by one launch, their sum by a second; then a smaller problem
    for (m, n, k), kernel in (((256, 2112, 7168), "mid_64x64:s=7"), ((96, 768, 1536), "mid_64x64:s=4"),
                              ((2048, 4096, 512), "mid_128x128:s=1"), ((200, 1024, 2048), "")):
        p = make_problem(m, n, k, seed=m + k)
        want, got = both(p, m, n, kernel=kernel)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (m, n, k, kernel)


def test_own_choice_of_k_ranges_fits_the_buffer():
    # the library's own choice for this shape is two K ranges per 256 x 192 tile: 96 tiles x 2 x 192 KiB of
    # parked accumulators, more than the fixed buffer's 32 MiB; the entry point that may not allocate then
    # keeps a tile in one workgroup (the named kernel's result, bit for bit) instead of failing
    m, n, k = 2048, 2304, 7168
    assert _ffi.gemm_choice(m, n, k) == "prefill_256x192:s=2"
    a = [t.to(DEV) for t in make_problem(m, n, k, seed=74)]
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    one = torch.empty_like(got)
    two = torch.empty_like(got)
    _ffi.call("gemm_a8w8_blockscale_noalloc", *a, got, -1, "")
    _ffi.call("gemm_a8w8_blockscale", *a, one, -1, "prefill_256x192")
    _ffi.call("gemm_a8w8_blockscale", *a, two, -1, "")
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), one.view(torch.int16))
    assert (got.view(torch.int16) != two.view(torch.int16)).float().mean().item() < 0.02
    with pytest.raises(RuntimeError, match="32 MiB"):  # asked for by name it is an error
        _ffi.call("gemm_a8w8_blockscale_noalloc", *a, got, -1, "prefill_256x192:s=2")


def test_own_choice_of_mid_tiling_fits_the_buffer():
    # the library's own plan for this shape is two K ranges of 128 x 128 tiles: 2 x 128 x 36864 fp32 = 36 MiB of
    # partial tiles, more than the fixed buffer holds; the entry point that may not allocate takes the best plan
    # that fits instead of failing, and gives that plan's result bit for bit
    m, n, k = 128, 36864, 7168
    assert _ffi.gemm_choice(m, n, k) == "mid_128x128:s=2"
    a = [t.to(DEV) for t in make_problem(m, n, k, seed=75)]
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=DEV)
    _ffi.call("gemm_a8w8_blockscale_noalloc", *a, got, -1, "")
    torch.cuda.synchronize()
    assert_close_to_f64(got, *[t.cpu() for t in a], "noalloc 128x36864x7168")
    same = []
    for kernel in ("mid_128x128:s=1", "mid_64x128:s=1", "mid_64x64:s=1", "mid_64x128:s=2", "mid_64x64:s=2"):
        one = torch.empty_like(got)
        _ffi.call("gemm_a8w8_blockscale", *a, one, -1, kernel)
        torch.cuda.synchronize()
        same.append(torch.equal(got.view(torch.int16), one.view(torch.int16)))
    assert any(same)
    with pytest.raises(RuntimeError, match="32 MiB"):  # asked for by name it is an error
        _ffi.call("gemm_a8w8_blockscale_noalloc", *a, got, -1, "mid_128x128:s=2")


def test_rejects_what_the_buffer_cannot_hold():
    m, n, k = 2048, 8192, 1280   # 5 K ranges x 2048 x 8192 fp32 = 320 MiB of partial tiles
    a = [t.to(DEV) for t in make_problem(m, n, k, seed=73)]
    out = torch.zeros(m, n, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="32 MiB"):
        _ffi.call("gemm_a8w8_blockscale_noalloc", *a, out, -1, "mid_128x128:s=5")
    torch.cuda.synchronize()
    assert not out.any()          # nothing was launched
    _ffi.call("gemm_a8w8_blockscale_noalloc", *a, out, -1, "mid_128x128:s=1")  # no scratch needed: served
    torch.cuda.synchronize()
    assert_close_to_f64(out, *[t.cpu() for t in a], "noalloc mid_128x128:s=1")
