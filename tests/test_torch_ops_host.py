"""torch.ops.aiter.* registration: schemas, fake implementations and graph tracing, without a GPU.

The reference registers its bindings the same way (aiter/jit/utils/torch_guard.py:200-357) so that
torch.compile sees each of them as one opaque call; fakes of the GEMMs at
aiter/ops/gemm_op_a8w8.py:790-801,893-905."""

import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

import aiter_amd
from aiter_amd import dtypes, torch_ops

EXPECTED = {
    "dynamic_per_token_scaled_quant", "per_group_quant_hip", "gemm_a8w8_blockscale", "gemm_a8w8_blockscale_ck",
    "gemm_a8w8_blockscale_bpreshuffle", "gemm_a8w8_blockscale_bpreshuffle_ck", "rmsnorm", "rmsnorm_quant",
    "add_rmsnorm", "add_rmsnorm_quant", "rms_norm", "topk_softmax", "moe_sorting_fwd", "fmoe_fp8_blockscale_g1u1",
}


def test_every_entry_point_is_a_torch_op():
    assert set(torch_ops.REGISTERED) == EXPECTED
    for name in EXPECTED:
        op = getattr(torch.ops.aiter, name)
        schema = op.default._schema
        assert schema.name == f"aiter::{name}"
        # ops that write into arguments return nothing; nothing returns an alias of an input
        assert all(r.alias_info is None for r in schema.returns), name
        if any(a.alias_info is not None and a.alias_info.is_write for a in schema.arguments):
            if name != "gemm_a8w8_blockscale_bpreshuffle":  # optional out=, as the reference declares it
                assert len(schema.returns) == 0, name


def test_fakes_give_the_shapes_and_dtypes_of_the_real_calls():
    with FakeTensorMode():
        dev = "cuda"
        xq = torch.empty(48, 1024, dtype=dtypes.fp8, device=dev)
        wq = torch.empty(512, 1024, dtype=dtypes.fp8, device=dev)
        xs, ws = torch.empty(48, 8, device=dev), torch.empty(4, 8, device=dev)
        y = torch.ops.aiter.gemm_a8w8_blockscale(xq, wq, xs, ws)
        assert y.shape == (48, 512) and y.dtype == torch.bfloat16 and y.device.type == "cuda"
        y = torch.ops.aiter.gemm_a8w8_blockscale(xq, wq, xs, ws, torch.float16, True)
        assert y.shape == (48, 512) and y.dtype == torch.float16
        y = torch.ops.aiter.gemm_a8w8_blockscale_bpreshuffle(xq, wq, xs, ws, torch.float16)
        assert y.shape == (48, 512) and y.dtype == torch.float16
        x = torch.empty(3, 5, 256, dtype=torch.float16, device=dev)
        q, s = torch.ops.aiter.per_group_quant_hip(x, group_size=64)
        assert q.shape == x.shape and q.dtype == dtypes.fp8 and s.shape == (3, 5, 4) and s.dtype == torch.float32
        out = torch.empty(48, 512, dtype=torch.bfloat16, device=dev)
        assert torch.ops.aiter.gemm_a8w8_blockscale_ck(xq, wq, xs, ws, out, 0, "") is None
        assert torch.ops.aiter.rmsnorm_quant(xq, torch.empty(48, 1024, dtype=torch.bfloat16, device=dev), xs,
                                             torch.empty(1024, dtype=torch.bfloat16, device=dev), 1e-6, 128) is None


def test_meta_tensors_dispatch_to_the_fakes():
    xq = torch.empty(8, 256, dtype=dtypes.fp8, device="meta")
    wq = torch.empty(32, 256, dtype=dtypes.fp8, device="meta")
    y = torch.ops.aiter.gemm_a8w8_blockscale(xq, wq, torch.empty(8, 2, device="meta"), torch.empty(1, 2, device="meta"))
    assert y.shape == (8, 32) and y.device.type == "meta"


def test_cpu_tensors_reach_the_librarys_own_error():
    z = torch.zeros(2, 128, dtype=torch.uint8).view(dtypes.fp8)
    with pytest.raises(RuntimeError, match="must live in GPU memory"):
        torch.ops.aiter.gemm_a8w8_blockscale(z, torch.zeros(16, 128, dtype=torch.uint8).view(dtypes.fp8),
                                             torch.ones(2, 1), torch.ones(1, 1))


def decoder_step(x, res, w, wq, ws, wq_sh, ws2, out2):
    q = torch.empty(x.shape, dtype=dtypes.fp8, device=x.device)
    s = torch.empty(x.shape[0], x.shape[1] // 128, dtype=torch.float32, device=x.device)
    res_out = torch.empty_like(x)
    aiter_amd.rmsnorm2d_fwd_with_add_dynamicquant(q, x, res, res_out, s, w, 1e-6, 0, group_size=128)
    y = aiter_amd.gemm_a8w8_blockscale(q, wq, s, ws)
    q2, s2 = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(y, quant_dtype=dtypes.fp8, transpose_scale=True)
    aiter_amd.gemm_a8w8_blockscale_bpreshuffle(q2, wq_sh, s2, ws2, out=out2)
    return y, res_out, out2


def expert_layer(x, w1, w2, w1s, w2s, gating):
    tw, ti = aiter_amd.fused_topk(x, gating, 4, True)
    return aiter_amd.fused_moe(x, w1, w2, tw, ti, quant_type=aiter_amd.QuantType.per_1x128, w1_scale=w1s, w2_scale=w2s)


def test_whole_graph_tracing_without_breaks():
    """Dynamo traces the Python entry points into one graph of aiter ops (no graph break, no ctypes call)."""
    with FakeTensorMode():
        dev = "cuda"
        x = torch.empty(64, 1024, dtype=torch.bfloat16, device=dev)
        args = (x, torch.empty_like(x), torch.empty(1024, dtype=torch.bfloat16, device=dev),
                torch.empty(512, 1024, dtype=dtypes.fp8, device=dev), torch.empty(4, 8, device=dev),
                torch.empty(256, 512, dtype=dtypes.fp8, device=dev), torch.empty(2, 4, device=dev),
                torch.empty(64, 256, dtype=torch.bfloat16, device=dev))
        gm, _ = torch._dynamo.export(decoder_step)(*args)
        called = [n.target for n in gm.graph.nodes if n.op == "call_function" and "aiter" in str(n.target)]
        assert [str(t) for t in called] == ["aiter.add_rmsnorm_quant", "aiter.gemm_a8w8_blockscale",
                                            "aiter.per_group_quant_hip", "aiter.gemm_a8w8_blockscale_bpreshuffle_ck"]

        E, dim, inter = 8, 512, 256
        margs = (torch.empty(16, dim, dtype=torch.bfloat16, device=dev),
                 torch.empty(E, 2 * inter, dim, dtype=dtypes.fp8, device=dev),
                 torch.empty(E, dim, inter, dtype=dtypes.fp8, device=dev),
                 torch.empty(E, 4, 4, device=dev), torch.empty(E, 4, 2, device=dev),
                 torch.empty(16, E, dtype=torch.bfloat16, device=dev))
        gm, _ = torch._dynamo.export(expert_layer)(*margs)
        called = [str(n.target) for n in gm.graph.nodes if n.op == "call_function" and "aiter" in str(n.target)]
        assert called == ["aiter.topk_softmax", "aiter.moe_sorting_fwd", "aiter.fmoe_fp8_blockscale_g1u1"]
