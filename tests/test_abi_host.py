"""CPU: the C-ABI library loads without a GPU, exports every symbol the header declares, keeps
the descriptor layout, and turns bad arguments into status -1 + message (never an abort).
No compute call is made here."""

import ctypes
import os
import re

import pytest
import torch

import aiter_amd
from aiter_amd import _ffi, dtypes
from aiter_amd.dtypes import aiter_tensor_t, torch_to_aiter

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "aiter_fp8bs.h")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_ffi.LIB_PATH):
        from aiter_amd.build import build_library

        build_library()
    return _ffi.load_library()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b([a-z_0-9]+)\s*\([^;{}]*\)\s*;", text)))


def test_every_declared_symbol_is_exported(lib):
    names = declared_functions()
    assert "gemm_a8w8_blockscale" in names and "dynamic_per_token_scaled_quant" in names
    assert "rmsnorm_quant" in names and "aiter_get_last_error" in names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/aiter_fp8bs.h but not exported"
    assert sorted(_ffi.EXPORTED_SYMBOLS) == names


def test_abi_version_and_descriptor_layout(lib):
    assert lib.aiter_ctypes_abi_version() == 2
    assert ctypes.sizeof(aiter_tensor_t) == 160
    off = {f[0]: getattr(aiter_tensor_t, f[0]).offset for f in aiter_tensor_t._fields_}
    assert off == {"ptr": 0, "numel_": 8, "ndim": 16, "shape": 24, "strides": 88, "dtype_": 152, "device_id": 156}
    t = torch.zeros(3, 5, 7, dtype=torch.bfloat16)[:, ::2]
    d = torch_to_aiter(t)
    assert (d.ndim, d.numel_, d.dtype_, d.device_id) == (3, 63, 3, -1)
    assert list(d.shape[:3]) == [3, 3, 7] and list(d.strides[:3]) == [35, 14, 1]
    assert dtypes.AITER_DTYPE["fp8"] == 0 and dtypes.AITER_DTYPE["fp32"] == 4 and dtypes.AITER_DTYPE["u64"] == 13


def test_kernel_name_list(lib):
    names = aiter_amd.gemm_kernel_names()
    assert len(names) >= 1 and all(n for n in names)


def fake_gpu(t: torch.Tensor, ptr=0x7F0000000000):
    """Descriptor that claims device memory; only ever used on paths that fail validation."""
    d = torch_to_aiter(t)
    d.device_id = 0
    d.ptr = ptr
    return d


def call_raw(lib, name, *args):
    lib.aiter_clear_last_error()
    rc = getattr(lib, name)(*args)
    msg = lib.aiter_get_last_error()
    return rc, (msg.decode() if msg else None)


def test_error_paths_return_status_and_message(lib):
    x = torch.zeros(4, 256, dtype=torch.bfloat16)
    y = torch.zeros(4, 256, dtype=torch.uint8).view(dtypes.fp8)
    s = torch.zeros(4, 2, dtype=torch.float32)
    xv = x.view(-1, 128)
    R = ctypes.byref

    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", None, None, None, None, 0, None, 1, None)
    assert rc == -1 and "out must not be null" in msg
    # host memory is rejected before anything touches HIP
    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", R(torch_to_aiter(y)), R(torch_to_aiter(xv)),
                       R(torch_to_aiter(s)), None, 0, None, 1, None)
    assert rc == -1 and "GPU memory" in msg
    # wrong dtypes / shapes with descriptors that claim to be on the GPU
    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", R(fake_gpu(y)), R(fake_gpu(x.float().view(-1, 128))),
                       R(fake_gpu(s)), None, 0, None, 1, None)
    assert rc == -1 and "bf16 or fp16" in msg
    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", R(fake_gpu(y)), R(fake_gpu(x)), R(fake_gpu(s)),
                       None, 0, None, 1, None)
    assert rc == -1 and "group in {32, 64, 128}" in msg
    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", R(fake_gpu(y)), R(fake_gpu(xv)),
                       R(fake_gpu(torch.zeros(4, 3))), None, 0, None, 1, None)
    assert rc == -1 and "one element per group" in msg
    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", R(fake_gpu(y)), R(fake_gpu(xv)), R(fake_gpu(s)),
                       R(fake_gpu(s)), 0, None, 1, None)
    assert rc == -1 and "scale_ub" in msg
    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", R(fake_gpu(y)), R(fake_gpu(xv, ptr=0x7F0000000004)),
                       R(fake_gpu(s)), None, 0, None, 1, None)
    assert rc == -1 and "aligned" in msg
    # a successful validation of an empty problem needs no device at all
    e_y = torch.zeros(0, 256, dtype=torch.uint8).view(dtypes.fp8)
    e_x = torch.zeros(0, 128, dtype=torch.bfloat16)
    e_s = torch.zeros(0, 2)
    rc, msg = call_raw(lib, "dynamic_per_token_scaled_quant", R(fake_gpu(e_y)), R(fake_gpu(e_x)), R(fake_gpu(e_s)),
                       None, 0, None, 1, None)
    assert rc == 0 and msg is None


def test_gemm_validation(lib):
    R = ctypes.byref
    f8 = lambda *sh: torch.zeros(*sh, dtype=torch.uint8).view(dtypes.fp8)
    xq, wq = f8(8, 256), f8(64, 256)
    xs, ws = torch.zeros(8, 2), torch.zeros(1, 2)
    out = torch.zeros(8, 64, dtype=torch.bfloat16)

    def go(*a, splitk=0, name=b""):
        return call_raw(lib, "gemm_a8w8_blockscale", *[R(fake_gpu(t)) for t in a], splitk, name, None)

    rc, msg = go(xq, f8(64, 128), xs, ws, out)
    assert rc == -1 and "WQ is [64,128]" in msg
    rc, msg = go(f8(8, 192), f8(64, 192), xs, ws, out)
    assert rc == -1 and "multiple of the 128" in msg
    rc, msg = go(xq, wq, xs, torch.zeros(2, 2), out)
    assert rc == -1 and "w_scale must be contiguous [1,2]" in msg
    rc, msg = go(xq, wq, xs, ws, out.float())
    assert rc == -1 and "bf16 or fp16" in msg
    rc, msg = go(xq, wq, xs.half(), ws.half(), out)
    assert rc == -1 and "scales must be fp32" in msg
    rc, msg = go(xq, wq, xs, ws, out, splitk=31)  # the reference takes 0..30 (gemm_a8w8_blockscale.cu:82-114)
    assert rc == -1 and "splitK" in msg
    rc, msg = go(xq.view(torch.uint8), wq, xs, ws, out)
    assert rc == -1 and "same dtype" in msg  # csrc/ck_gemm_a8w8_blockscale/gemm_a8w8_blockscale.cu:90-93
    rc, msg = go(f8(0, 256), wq, torch.zeros(0, 2), ws, torch.zeros(0, 64, dtype=torch.bfloat16))
    assert rc == 0 and msg is None


def test_moe_validation(lib):
    R = ctypes.byref
    g = lambda t: R(fake_gpu(t))
    f8 = lambda *sh: torch.zeros(*sh, dtype=torch.uint8).view(dtypes.fp8)
    i32 = lambda *sh: torch.zeros(*sh, dtype=torch.int32)
    # routing
    rc, msg = call_raw(lib, "topk_softmax", g(torch.zeros(4, 2)), g(i32(4, 2)), None, g(torch.zeros(4, 2000)), 1, None)
    assert rc == -1 and "experts = 2000" in msg
    rc, msg = call_raw(lib, "topk_softmax", g(torch.zeros(4, 9)), g(i32(4, 9)), None, g(torch.zeros(4, 8)), 1, None)
    assert rc == -1 and "topk = 9" in msg
    rc, msg = call_raw(lib, "topk_softmax", g(torch.zeros(4, 2)), g(i32(4, 2).long()), None, g(torch.zeros(4, 8)), 1, None)
    assert rc == -1 and "int32" in msg
    # sorting: buffers sized as aiter/fused_moe.py:209-215 sizes them
    ids, w = i32(4, 2), torch.zeros(4, 2)
    padded = 4 * 2 + 8 * 32 - 2
    ok = (g(ids), g(w), g(i32(padded)), g(torch.zeros(padded)), g(i32((padded + 31) // 32)), g(i32(2)))
    rc, msg = call_raw(lib, "moe_sorting_fwd", *ok[:2], g(i32(padded - 1)), *ok[3:], None, 8, 32, None, None, 0, None)
    assert rc == -1 and "sorted_token_ids" in msg and str(padded) in msg
    rc, msg = call_raw(lib, "moe_sorting_fwd", *ok, None, 2000, 32, None, None, 0, None)
    assert rc == -1 and "num_experts" in msg
    rc, msg = call_raw(lib, "moe_sorting_fwd", *ok, None, 8, 32, g(i32(7)), None, 0, None)
    assert rc == -1 and "local_expert_mask" in msg
    # experts
    E, dim, inter, M = 4, 256, 128, 4
    args = dict(out=torch.zeros(M, dim, dtype=torch.bfloat16), inp=f8(M, dim), gate=f8(E, 2 * inter, dim),
                down=f8(E, dim, inter), sids=i32(padded), sw=torch.zeros(padded), se=i32((padded + 31) // 32),
                nv=i32(2), xs=torch.zeros(dim // 128, M), s1=torch.zeros(E, 2 * inter // 128 * dim // 128),
                s2=torch.zeros(E, dim // 128 * inter // 128))

    def fmoe(topk=2, blkn=128, blkk=128, act=0, block_m=32, **over):
        a = dict(args, **over)
        opt = lambda t: g(t) if t is not None else None
        return call_raw(lib, "fmoe_fp8_blockscale_g1u1", g(a["out"]), g(a["inp"]), g(a["gate"]), g(a["down"]),
                        g(a["sids"]), g(a["sw"]), g(a["se"]), g(a["nv"]), topk, opt(a["xs"]), g(a["s1"]), g(a["s2"]),
                        b"", blkn, blkk, None, act, block_m, None)

    rc, msg = fmoe(gate=f8(E, inter, dim))
    assert rc == -1 and "gate must be [experts, 2*inter_dim, dim]" in msg
    rc, msg = fmoe(blkn=64)
    assert rc == -1 and "128 x 128" in msg
    rc, msg = fmoe(block_m=48)
    assert rc == -1 and "block_size_M" in msg
    rc, msg = fmoe(act=7)
    assert rc == -1 and "activation" in msg
    rc, msg = fmoe(xs=None)
    assert rc == -1 and "input_scale" in msg
    rc, msg = fmoe(xs=torch.zeros(M, dim // 128))
    assert rc == -1 and "[dim/128, tokens]" in msg
    rc, msg = fmoe(s2=torch.zeros(E, 3))
    assert rc == -1 and "fc2_scale" in msg
    rc, msg = fmoe(out=torch.zeros(M, dim))
    assert rc == -1 and "bf16 or fp16" in msg
    rc, msg = fmoe(inp=f8(0, dim), out=torch.zeros(0, dim, dtype=torch.bfloat16), xs=torch.zeros(dim // 128, 0))
    assert rc == 0 and msg is None  # nothing to do: returns before any HIP call


def test_rmsnorm_validation(lib):
    R = ctypes.byref
    x = torch.zeros(4, 1024, dtype=torch.bfloat16)
    w = torch.zeros(1024, dtype=torch.bfloat16)
    y = torch.zeros(4, 1024, dtype=torch.uint8).view(dtypes.fp8)
    s = torch.zeros(4, 8)
    g = lambda t: R(fake_gpu(t))
    rc, msg = call_raw(lib, "rmsnorm_quant", g(y), g(x), g(s), g(w), ctypes.c_float(1e-6), 0, 0, 0, None)
    assert rc == -1 and "group_size 0" in msg
    rc, msg = call_raw(lib, "rmsnorm_quant", g(y), g(x), g(s), g(w.half()), ctypes.c_float(1e-6), 128, 0, 0, None)
    assert rc == -1 and "weight dtype" in msg
    big = torch.zeros(1, 16384, dtype=torch.bfloat16)
    rc, msg = call_raw(lib, "rmsnorm", g(big), g(big), g(torch.zeros(16384, dtype=torch.bfloat16)),
                       ctypes.c_float(1e-6), 0, None)
    assert rc == -1 and "8192" in msg
    rc, msg = call_raw(lib, "rmsnorm_quant", g(y), g(x), g(torch.zeros(4, 7)), g(w), ctypes.c_float(1e-6), 128, 0, 0, None)
    assert rc == -1 and "scale must be contiguous" in msg


def test_python_facade_raises_runtime_error_on_cpu_tensors():
    x = torch.zeros(4, 256, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="dynamic_per_token_scaled_quant failed: .*GPU memory"):
        aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)(x)
    with pytest.raises(RuntimeError, match="gemm_a8w8_blockscale failed"):
        aiter_amd.gemm_a8w8_blockscale(
            torch.zeros(2, 128, dtype=torch.uint8).view(dtypes.fp8),
            torch.zeros(4, 128, dtype=torch.uint8).view(dtypes.fp8),
            torch.zeros(2, 1), torch.zeros(1, 1),
        )
    with pytest.raises(NotImplementedError):
        aiter_amd.get_hip_quant(aiter_amd.QuantType.per_Token)(x)
    with pytest.raises(ValueError, match="static per token quant"):
        aiter_amd.per_group_quant_hip(x, scale=torch.zeros(4, 2))
    with pytest.raises(NotImplementedError):
        aiter_amd.rmsnorm2d_fwd_with_dynamicquant(x, x, torch.zeros(4, 2), x[0], 1e-6, 0, group_size=0)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_ffi, "_lib", None)
    monkeypatch.setattr(_ffi, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _ffi.load_library()


def test_shuffle_weight_closed_form():
    # independent statement of the (16,16) layout: byte b of half h of 32-wide chunk c of row r of
    # tile t sits at t*16*K + c*512 + h*256 + r*16 + b
    import aiter_amd

    n, k = 48, 160
    w = torch.arange(n * k, dtype=torch.int32).remainder(251).to(torch.uint8).view(n, k)
    flat = aiter_amd.shuffle_weight(w).flatten()
    for t, c, h, r, b in [(0, 0, 0, 0, 0), (2, 4, 1, 15, 15), (1, 3, 0, 7, 9), (2, 0, 1, 3, 0), (0, 4, 1, 0, 15)]:
        assert flat[t * 16 * k + c * 512 + h * 256 + r * 16 + b] == w[t * 16 + r, c * 32 + h * 16 + b]
    # it is a permutation, and leading dimensions are shuffled matrix by matrix
    assert torch.equal(flat.sort().values, w.flatten().sort().values)
    w3 = torch.stack([w, w.flip(0)])
    s3 = aiter_amd.shuffle_weight(w3)
    assert torch.equal(s3[0], aiter_amd.shuffle_weight(w)) and torch.equal(s3[1], aiter_amd.shuffle_weight(w.flip(0)))
    with pytest.raises(ValueError):
        aiter_amd.shuffle_weight(w[:40])
