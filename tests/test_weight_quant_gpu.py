"""GPU parity of the weight-side 128x128 block quantiser through the C-ABI: codes and scales
bit-exact against the C oracle (pinned against the torch restatement of
op_tests/multigpu_tests/test_dispatch_combine.py:180-204 in tests/test_oracle_pins.py)."""

import numpy as np
import pytest
import torch

import aiter_amd
from aiter_amd import dtypes
from oracle import c_oracle as co
from oracle import torch_ref as tr
from tests.helpers import codes8, codes16, guarded_empty

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def check(w, what):
    wq, ws = aiter_amd.weight_per_128x128_quant(w.to(DEV))
    torch.cuda.synchronize()
    if w.dtype == torch.bfloat16:   # the C oracle's weight quantiser reads bf16
        oq, os_ = co.weight_block_quant(codes16(w))
    else:
        tq, ts = tr.weight_per_128x128_quant(w)
        oq, os_ = tq.view(torch.uint8).numpy(), ts.numpy()
    assert wq.shape == w.shape and ws.shape == ((w.shape[0] + 127) // 128, w.shape[1] // 128)
    assert np.array_equal(ws.cpu().numpy().view(np.uint32), os_.view(np.uint32)), f"{what}: scales differ"
    got = codes8(wq)
    bad = np.argwhere(got != oq)
    assert bad.size == 0, f"{what}: {len(bad)} codes differ, first at {bad[0]}: {got[tuple(bad[0])]} vs {oq[tuple(bad[0])]}"
    return wq, ws


@pytest.mark.parametrize("n,k", [(128, 128), (512, 1024), (2112, 7168), (64, 256), (130, 384), (4096, 512)])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_matches_oracle(n, k, dtype):
    w = tr.make_weight(n, k, seed=n + k).to(dtype)
    wq, ws = check(w, f"[{n},{k}] {dtype}")
    # and the torch restatement of the reference's offline recipe agrees as well
    tq, ts = tr.weight_per_128x128_quant(w)
    assert torch.equal(ws.cpu(), ts) and torch.equal(wq.cpu().view(torch.uint8), tq.view(torch.uint8))


def test_special_blocks():
    w = tr.make_weight(256, 512, seed=9)
    w[:128, :128] = 0                      # zero block: scale 1, codes +-0
    w[5, 130] = float("inf")               # block with an inf
    w[130, 5] = float("nan")               # block with a NaN
    w[140, 300] = -0.0
    w[128:, 384:] *= 1e-30                 # amax below the fast-path window
    w[200, 400] = 3e38                     # ... and one far above it
    wq, ws = check(w, "special blocks")
    assert ws[0, 0].item() == 1.0


def test_strided_rows_and_guard_bands():
    n, k = 200, 256
    full = tr.make_weight(n, k + 128, seed=3)
    w = full[:, :k]
    wd = full.to(DEV)[:, :k]                                # row stride k + 128
    assert not wd.is_contiguous()
    out, chk_out = guarded_empty((n, k), dtypes.fp8, DEV)
    sc, chk_sc = guarded_empty((2, 2), torch.float32, DEV)
    aiter_amd._ffi.call("weight_per_128x128_quant", out, wd, sc)
    torch.cuda.synchronize()
    chk_out()
    chk_sc()
    oq, os_ = co.weight_block_quant(codes16(w.contiguous()))
    assert np.array_equal(codes8(out), oq) and np.array_equal(sc.cpu().numpy().view(np.uint32), os_.view(np.uint32))


def test_feeds_the_gemm():
    m, n, k = 32, 1024, 1024
    x = tr.make_activation(m, k, seed=1)
    w = tr.make_weight(n, k, seed=2)
    wq, ws = aiter_amd.weight_per_128x128_quant(w.to(DEV))
    xq, xs = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(x.to(DEV))
    out = aiter_amd.gemm_a8w8_blockscale(xq, wq, xs, ws)
    ref = tr.gemm_a8w8_blockscale_ref(xq.cpu(), wq.cpu(), xs.cpu(), ws.cpu())
    assert tr.check_allclose_ratio(out.cpu(), ref, 1e-2, 1e-2) == 0.0


def test_rejects_bad_operands():
    w = torch.zeros(128, 192, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 128"):
        aiter_amd.weight_per_128x128_quant(w)
    with pytest.raises(RuntimeError, match="bf16 or fp16"):
        aiter_amd.weight_per_128x128_quant(torch.zeros(128, 128, device=DEV))
