"""ctypes binding of the scalar C oracle (``libfp8bs_oracle.so``).  TEST INFRASTRUCTURE ONLY.

Arrays cross as numpy buffers; 16-bit floats cross as raw ``uint16`` codes and fp8 as raw
``uint8`` codes so that no conversion happens on the Python side.
"""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libfp8bs_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it (gcc, seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, i64, ci, cf = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
        L.oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_bf16_to_f32.restype = cf
        L.oracle_f32_to_bf16.argtypes = [cf]
        L.oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.oracle_f16_to_f32.restype = cf
        L.oracle_f32_to_e4m3fn.argtypes = [cf]
        L.oracle_f32_to_e4m3fn.restype = ctypes.c_uint8
        L.oracle_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3fn_to_f32.restype = cf
        L.oracle_f32_to_e4m3fn_n.argtypes = [vp, vp, i64]
        L.oracle_e4m3fn_to_f32_n.argtypes = [vp, vp, i64]
        L.oracle_group_quant.argtypes = [vp, ci, i64, ci, vp, vp]
        L.oracle_weight_block_quant.argtypes = [vp, i64, i64, ci, ci, vp, vp]
        L.oracle_rmsnorm_bf16.argtypes = [vp, vp, cf, i64, i64, ci, vp]
        L.oracle_add_rmsnorm_bf16.argtypes = [vp, vp, vp, cf, i64, i64, ci, vp, vp]
        L.oracle_gemm_blockscale.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, ci, vp, vp]
        for name in (
            "oracle_f32_to_e4m3fn_n",
            "oracle_e4m3fn_to_f32_n",
            "oracle_group_quant",
            "oracle_weight_block_quant",
            "oracle_rmsnorm_bf16",
            "oracle_add_rmsnorm_bf16",
            "oracle_gemm_blockscale",
        ):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _p(a: np.ndarray):
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.c_void_p)


_DT = {"bf16": 0, "fp16": 1, "fp32": 2}


def f32_to_e4m3fn(f: np.ndarray) -> np.ndarray:
    f = np.ascontiguousarray(f, dtype=np.float32)
    out = np.empty(f.shape, dtype=np.uint8)
    lib().oracle_f32_to_e4m3fn_n(_p(f), _p(out), f.size)
    return out


def e4m3fn_to_f32(c: np.ndarray) -> np.ndarray:
    c = np.ascontiguousarray(c, dtype=np.uint8)
    out = np.empty(c.shape, dtype=np.float32)
    lib().oracle_e4m3fn_to_f32_n(_p(c), _p(out), c.size)
    return out


def group_quant(x_codes: np.ndarray, in_dtype: str = "bf16", group: int = 128):
    """x_codes: uint16 raw codes (bf16/fp16) or float32 values, last dim % group == 0.
    Returns (uint8 codes with x's shape, float32 scales [..., K/group])."""
    x_codes = np.ascontiguousarray(x_codes)
    assert x_codes.shape[-1] % group == 0
    assert x_codes.dtype == (np.float32 if in_dtype == "fp32" else np.uint16)
    n_groups = x_codes.size // group
    y = np.empty(x_codes.shape, dtype=np.uint8)
    s = np.empty(x_codes.shape[:-1] + (x_codes.shape[-1] // group,), dtype=np.float32)
    lib().oracle_group_quant(_p(x_codes), _DT[in_dtype], n_groups, group, _p(y), _p(s))
    return y, s


def weight_block_quant(w_codes: np.ndarray, block=(128, 128)):
    w_codes = np.ascontiguousarray(w_codes, dtype=np.uint16)
    n, k = w_codes.shape
    nb, kb = (n + block[0] - 1) // block[0], (k + block[1] - 1) // block[1]
    wq = np.empty((n, k), dtype=np.uint8)
    s = np.empty((nb, kb), dtype=np.float32)
    lib().oracle_weight_block_quant(_p(w_codes), n, k, block[0], block[1], _p(wq), _p(s))
    return wq, s


def rmsnorm_bf16(x_codes, w_codes, eps: float, gemma_norm: bool = False):
    x_codes = np.ascontiguousarray(x_codes, dtype=np.uint16)
    w_codes = np.ascontiguousarray(w_codes, dtype=np.uint16)
    rows, cols = x_codes.shape
    out = np.empty((rows, cols), dtype=np.uint16)
    lib().oracle_rmsnorm_bf16(_p(x_codes), _p(w_codes), eps, rows, cols, int(gemma_norm), _p(out))
    return out


def add_rmsnorm_bf16(x_codes, res_codes, w_codes, eps: float, gemma_norm: bool = False):
    x_codes = np.ascontiguousarray(x_codes, dtype=np.uint16)
    res_codes = np.ascontiguousarray(res_codes, dtype=np.uint16)
    w_codes = np.ascontiguousarray(w_codes, dtype=np.uint16)
    rows, cols = x_codes.shape
    res_out = np.empty((rows, cols), dtype=np.uint16)
    out = np.empty((rows, cols), dtype=np.uint16)
    lib().oracle_add_rmsnorm_bf16(
        _p(x_codes), _p(res_codes), _p(w_codes), eps, rows, cols, int(gemma_norm), _p(res_out), _p(out)
    )
    return out, res_out


def gemm_blockscale(xq, wq, xs, ws, accumulate: str = "f64"):
    """xq [M,K] uint8, wq [N,K] uint8, xs [M,K/128] f32, ws [ceil(N/128),K/128] f32.
    Returns (float32 [M,N], bf16 codes uint16 [M,N])."""
    xq = np.ascontiguousarray(xq, dtype=np.uint8)
    wq = np.ascontiguousarray(wq, dtype=np.uint8)
    xs = np.ascontiguousarray(xs, dtype=np.float32)
    ws = np.ascontiguousarray(ws, dtype=np.float32)
    m, k = xq.shape
    n = wq.shape[0]
    out = np.empty((m, n), dtype=np.float32)
    outb = np.empty((m, n), dtype=np.uint16)
    lib().oracle_gemm_blockscale(
        _p(xq), _p(wq), _p(xs), _p(ws), m, n, k, k, k, 0 if accumulate == "f64" else 1, _p(out), _p(outb)
    )
    return out, outb


# torch <-> raw-code helpers (torch is only used for the views; no arithmetic)
def codes16(t):
    """bf16/fp16 torch tensor -> numpy uint16 raw codes."""
    import torch

    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def codes8(t):
    import torch

    return t.contiguous().view(torch.uint8).numpy()
