"""torch.ops.aiter.* on the GPU: the registered ops and a compiled graph give exactly what the
eager entry points give (the reference's bindings are reachable the same way,
aiter/jit/utils/torch_guard.py:292-300)."""

import pytest
import torch

import aiter_amd
from aiter_amd import dtypes

from tests.test_torch_ops_host import decoder_step, expert_layer

pytestmark = pytest.mark.gpu


def same(a, b):
    return torch.equal(a.view(torch.uint8) if a.dtype == dtypes.fp8 else a, b.view(torch.uint8) if b.dtype == dtypes.fp8 else b)


def operands(dev, M=96, N=512, K=1024):
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn(M, K, generator=g, device=dev).bfloat16()
    w = (torch.randn(N, K, generator=g, device=dev) * 0.05).bfloat16()
    wq, ws = aiter_amd.weight_per_128x128_quant(w)
    return x, wq, ws


def test_ops_equal_entry_points():
    dev = torch.device("cuda:0")
    x, wq, ws = operands(dev)
    q, s = aiter_amd.per_group_quant_hip(x)
    q2, s2 = torch.ops.aiter.per_group_quant_hip(x)
    assert same(q, q2) and torch.equal(s, s2)
    y = aiter_amd.gemm_a8w8_blockscale(q, wq, s, ws)
    assert torch.equal(y, torch.ops.aiter.gemm_a8w8_blockscale(q, wq, s, ws))
    out = torch.empty_like(y)
    assert torch.ops.aiter.gemm_a8w8_blockscale_ck(q, wq, s, ws, out, -1, "") is None
    assert torch.equal(y, out)

    # the three spellings of the pre-shuffled call
    wsh = aiter_amd.shuffle_weight(wq, layout=(16, 16))
    qt, st = aiter_amd.per_group_quant_hip(x, transpose_scale=True)
    ref = aiter_amd.gemm_a8w8_blockscale_bpreshuffle(qt, wsh, st, ws)
    assert torch.equal(ref, aiter_amd.gemm_a8w8_blockscale(qt, wsh, st, ws, isBpreshuffled=True))
    out = torch.empty_like(ref)
    assert aiter_amd.gemm_a8w8_blockscale_bpreshuffle_asm(qt, wsh, out, st, ws) is out
    assert torch.equal(ref, out)
    out2 = torch.empty_like(ref)
    assert torch.ops.aiter.gemm_a8w8_blockscale_bpreshuffle(qt, wsh, st, ws, torch.bfloat16, out2) is out2
    assert torch.equal(ref, out2)
    # a zero bias changes nothing
    aiter_amd.gemm_a8w8_blockscale_bpreshuffle_asm(qt, wsh, out, st, ws, bias=torch.zeros(ref.shape[1], device=dev))
    assert torch.equal(ref, out)


def test_compiled_decoder_step_equals_eager():
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(6)
    x = torch.randn(64, 1024, generator=g, device=dev).bfloat16()
    res = torch.randn(64, 1024, generator=g, device=dev).bfloat16()
    w = (torch.rand(1024, generator=g, device=dev) + 0.5).bfloat16()
    wq, ws = aiter_amd.weight_per_128x128_quant((torch.randn(512, 1024, generator=g, device=dev) * 0.05).bfloat16())
    wq2, ws2 = aiter_amd.weight_per_128x128_quant((torch.randn(256, 512, generator=g, device=dev) * 0.05).bfloat16())
    wsh = aiter_amd.shuffle_weight(wq2, layout=(16, 16))
    eager = decoder_step(x, res, w, wq, ws, wsh, ws2, torch.empty(64, 256, dtype=torch.bfloat16, device=dev))
    compiled = torch.compile(decoder_step, backend="aot_eager", fullgraph=True)
    for _ in range(2):
        got = compiled(x, res, w, wq, ws, wsh, ws2, torch.zeros(64, 256, dtype=torch.bfloat16, device=dev))
        for a, b in zip(eager, got):
            assert torch.equal(a, b)


def test_compiled_expert_layer_equals_eager():
    dev = torch.device("cuda:0")
    g = torch.Generator(device=dev).manual_seed(7)
    E, dim, inter, tokens = 8, 512, 256, 16
    x = torch.randn(tokens, dim, generator=g, device=dev).bfloat16()
    w1q, w1s = aiter_amd.weight_per_128x128_quant((torch.randn(E * 2 * inter, dim, generator=g, device=dev) * 0.1).bfloat16())
    w2q, w2s = aiter_amd.weight_per_128x128_quant((torch.randn(E * dim, inter, generator=g, device=dev) * 0.1).bfloat16())
    w1 = aiter_amd.shuffle_weight(w1q.view(E, 2 * inter, dim).view(torch.uint8)).view(dtypes.fp8)
    w2 = aiter_amd.shuffle_weight(w2q.view(E, dim, inter).view(torch.uint8)).view(dtypes.fp8)
    gating = torch.randn(tokens, E, generator=g, device=dev).bfloat16()
    args = (x, w1, w2, w1s.view(E, -1), w2s.view(E, -1), gating)
    eager = expert_layer(*args)
    got = torch.compile(expert_layer, backend="aot_eager", fullgraph=True)(*args)
    assert torch.equal(eager, got)
