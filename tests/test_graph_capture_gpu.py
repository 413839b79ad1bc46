"""The entry points only enqueue work on the caller's stream: captured into a HIP graph (after one
eager call has sized the library's scratch), every replay must give what the eager call gives, also
with eager work and synchronisations between the replays and with new input contents each time."""

import pytest
import torch

import aiter_amd
from aiter_amd import dtypes
from oracle import torch_ref as tr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def replay_and_compare(build_inputs, refill, run):
    """build_inputs() -> static tensors; refill(inputs, i) overwrites them in place; run(inputs) -> outputs"""
    inputs = build_inputs()
    refill(inputs, 0)
    run(inputs)                      # eager: sizes scratch buffers
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            captured = run(inputs)
    for i in range(1, 4):
        refill(inputs, i)
        eager = [t.clone() for t in run(inputs)]
        torch.cuda.synchronize()
        for t in captured:
            t.fill_(0) if t.dtype in (torch.float32, torch.bfloat16, torch.float16) else t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for a, b in zip(eager, captured):
            assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)), f"replay {i} differs from the eager call"


def test_quant_norm_gemm_chain_under_graph_replay():
    m, k, n = 96, 2048, 2112        # the GEMM picks a K split here: workspace + second launch inside the graph
    w = tr.make_weight(n, k, seed=3).to(DEV)
    wq, ws = aiter_amd.weight_per_128x128_quant(w)
    gamma = (torch.rand(k, device=DEV) + 0.5).bfloat16()

    def build():
        return dict(x=torch.empty(m, k, device=DEV, dtype=torch.bfloat16),
                    y8=torch.empty(m, k, device=DEV, dtype=dtypes.fp8),
                    ys=torch.empty(m, k // 128, device=DEV, dtype=torch.float32),
                    out=torch.empty(m, n, device=DEV, dtype=torch.bfloat16),
                    out2=torch.empty(m, n, device=DEV, dtype=torch.bfloat16))

    def refill(t, i):
        g = torch.Generator(device=DEV).manual_seed(100 + i)
        t["x"].copy_(torch.randn(m, k, generator=g, device=DEV).bfloat16())

    quant = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)

    def run(t):
        aiter_amd.rmsnorm2d_fwd_with_dynamicquant(t["y8"], t["x"], t["ys"], gamma, 1e-6, 0, group_size=128)
        aiter_amd.gemm_a8w8_blockscale_ck(t["y8"], wq, t["ys"], ws, t["out"], splitK=-1)
        q, s = quant(t["x"], quant_dtype=dtypes.fp8)          # allocates from the graph's pool under capture
        aiter_amd.gemm_a8w8_blockscale_ck(q, wq, s, ws, t["out2"], splitK=2, kernelName="mid_64x64")
        return [t["y8"], t["ys"], t["out"], t["out2"]]

    replay_and_compare(build, refill, run)


def test_moe_under_graph_replay_with_changing_routing():
    tokens, dim, inter, experts, topk = 24, 512, 128, 16, 4
    g = torch.Generator(device=DEV).manual_seed(5)
    w1 = (torch.randn(experts * 2 * inter, dim, generator=g, device=DEV) * 0.1).bfloat16()
    w2 = (torch.randn(experts * dim, inter, generator=g, device=DEV) * 0.1).bfloat16()
    w1q, w1s = aiter_amd.weight_per_128x128_quant(w1)
    w2q, w2s = aiter_amd.weight_per_128x128_quant(w2)
    w1q = aiter_amd.shuffle_weight(w1q.view(experts, 2 * inter, dim).view(torch.uint8)).view(dtypes.fp8)
    w2q = aiter_amd.shuffle_weight(w2q.view(experts, dim, inter).view(torch.uint8)).view(dtypes.fp8)
    w1s, w2s = w1s.view(experts, -1).contiguous(), w2s.view(experts, -1).contiguous()
    mask = torch.ones(experts, dtype=torch.int32, device=DEV)
    mask[[2, 7, 11]] = 0             # pairs routed there are absent: their table entries must not go stale
    local = mask.bool()
    w1l, w2l, s1l, s2l = w1q[local].contiguous(), w2q[local].contiguous(), w1s[local].contiguous(), w2s[local].contiguous()

    def build():
        return dict(x=torch.empty(tokens, dim, device=DEV, dtype=torch.bfloat16),
                    score=torch.empty(tokens, experts, device=DEV))

    def refill(t, i):
        gg = torch.Generator(device=DEV).manual_seed(200 + i)
        t["x"].copy_(torch.randn(tokens, dim, generator=gg, device=DEV).bfloat16())
        t["score"].copy_(torch.randn(tokens, experts, generator=gg, device=DEV))

    def run(t):
        tw, ti = aiter_amd.fused_topk(t["x"], t["score"], topk, True)
        out = aiter_amd.fused_moe(t["x"], w1l, w2l, tw, ti, expert_mask=mask,
                                  quant_type=aiter_amd.QuantType.per_1x128, w1_scale=s1l, w2_scale=s2l)
        return [tw, ti, out]

    replay_and_compare(build, refill, run)


def test_moe_with_many_rows_per_expert_under_graph_replay():
    # 200 rows per expert: pairs of blocks (the first GEMM's LDS ring, 128 KiB of dynamic LDS), the second GEMM
    # by rows (16-bit rows through LDS) and the separate per-token sum, with the routing redrawn per replay
    tokens, dim, inter, experts, topk = 400, 7168, 256, 4, 2
    g = torch.Generator(device=DEV).manual_seed(6)
    w1 = (torch.randn(experts * 2 * inter, dim, generator=g, device=DEV) * 0.1).bfloat16()
    w2 = (torch.randn(experts * dim, inter, generator=g, device=DEV) * 0.1).bfloat16()
    w1q, w1s = aiter_amd.weight_per_128x128_quant(w1)
    w2q, w2s = aiter_amd.weight_per_128x128_quant(w2)
    w1q = aiter_amd.shuffle_weight(w1q.view(experts, 2 * inter, dim).view(torch.uint8)).view(dtypes.fp8)
    w2q = aiter_amd.shuffle_weight(w2q.view(experts, dim, inter).view(torch.uint8)).view(dtypes.fp8)
    w1s, w2s = w1s.view(experts, -1).contiguous(), w2s.view(experts, -1).contiguous()

    def build():
        return dict(x=torch.empty(tokens, dim, device=DEV, dtype=torch.bfloat16),
                    score=torch.empty(tokens, experts, device=DEV))

    def refill(t, i):
        gg = torch.Generator(device=DEV).manual_seed(300 + i)
        t["x"].copy_(torch.randn(tokens, dim, generator=gg, device=DEV).bfloat16())
        t["score"].copy_(torch.randn(tokens, experts, generator=gg, device=DEV))

    def run(t):
        tw, ti = aiter_amd.fused_topk(t["x"], t["score"], topk, True)
        out = aiter_amd.fused_moe(t["x"], w1q, w2q, tw, ti, quant_type=aiter_amd.QuantType.per_1x128,
                                  w1_scale=w1s, w2_scale=w2s)
        return [tw, ti, out]

    replay_and_compare(build, refill, run)
