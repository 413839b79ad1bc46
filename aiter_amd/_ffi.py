"""Loader and call bridge for ``libaiter_fp8bs.so`` (the only compute backend).

Mirrors the reference's ctypes bridge, aiter/jit/core.py:1306-1323 and :1580-1612: tensors go
as borrowed ``aiter_tensor_t*`` (None -> NULL), the caller's current HIP stream is appended,
a non-zero status raises ``RuntimeError("<fn> failed: <message>")``.

There is no fallback: if the library is missing or cannot be loaded every op raises.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch

from .dtypes import aiter_tensor_t, shared_descriptor

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG_DIR, "libaiter_fp8bs.so")

_lock = threading.Lock()
_lib = None

_TP = ctypes.POINTER(aiter_tensor_t)
_SIGNATURES = {
    # name: argtypes before the trailing stream
    "dynamic_per_token_scaled_quant": [_TP, _TP, _TP, _TP, ctypes.c_int, _TP, ctypes.c_int64],
    "rmsnorm": [_TP, _TP, _TP, ctypes.c_float, ctypes.c_int],
    "rmsnorm_quant": [_TP, _TP, _TP, _TP, ctypes.c_float, ctypes.c_int64, ctypes.c_int, ctypes.c_int],
    "add_rmsnorm": [_TP, _TP, _TP, _TP, _TP, ctypes.c_float, ctypes.c_int],
    "add_rmsnorm_quant": [
        _TP, _TP, _TP, _TP, _TP, _TP, ctypes.c_float, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
    ],
    "weight_per_128x128_quant": [_TP, _TP, _TP],
    "gemm_a8w8_blockscale": [_TP, _TP, _TP, _TP, _TP, ctypes.c_int64, ctypes.c_char_p],
    "gemm_a8w8_blockscale_noalloc": [_TP, _TP, _TP, _TP, _TP, ctypes.c_int64, ctypes.c_char_p],
    "gemm_a8w8_blockscale_bpreshuffle": [_TP, _TP, _TP, _TP, _TP, ctypes.c_char_p],
    "gemm_a8w8_blockscale_bpreshuffle_asm": [_TP, _TP, _TP, _TP, _TP, _TP, ctypes.c_int, ctypes.c_char_p, ctypes.c_int,
                                             _TP],
    "topk_softmax": [_TP, _TP, _TP, _TP, ctypes.c_int],
    "moe_sorting_fwd": [_TP, _TP, _TP, _TP, _TP, _TP, _TP, ctypes.c_int64, ctypes.c_int64, _TP, _TP, ctypes.c_int64],
    "fmoe_fp8_blockscale_g1u1": [
        _TP, _TP, _TP, _TP, _TP, _TP, _TP, _TP, ctypes.c_int64, _TP, _TP, _TP, ctypes.c_char_p,
        ctypes.c_int64, ctypes.c_int64, _TP, ctypes.c_int64, ctypes.c_int64,
    ],
}
EXPORTED_SYMBOLS = sorted(
    list(_SIGNATURES)
    + [
        "aiter_ctypes_abi_version",
        "aiter_get_last_error",
        "aiter_clear_last_error",
        "aiter_fp8bs_gemm_kernel_names",
        "aiter_fp8bs_gemm_choice",
        "aiter_fp8bs_gemm_resolve",
    ]
)


def load_library():
    """Load (once) and return the ctypes handle; raises if the library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m aiter_amd.build` "
                "(there is no fallback implementation)"
            )
        lib = ctypes.CDLL(LIB_PATH)
        lib.aiter_ctypes_abi_version.restype = ctypes.c_int
        if lib.aiter_ctypes_abi_version() != 2:
            raise RuntimeError("libaiter_fp8bs.so reports an unexpected ABI version")
        lib.aiter_get_last_error.restype = ctypes.c_char_p
        lib.aiter_clear_last_error.restype = None
        lib.aiter_fp8bs_gemm_kernel_names.restype = ctypes.c_char_p
        lib.aiter_fp8bs_gemm_choice.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                                ctypes.c_char_p, ctypes.c_int64]
        lib.aiter_fp8bs_gemm_choice.restype = ctypes.c_int
        lib.aiter_fp8bs_gemm_resolve.argtypes = [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                                                 ctypes.c_int64, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_int64]
        lib.aiter_fp8bs_gemm_resolve.restype = ctypes.c_int
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes + [ctypes.c_void_p]
            fn.restype = ctypes.c_int
        _lib = lib
    return _lib


# the raw handle of the current stream without building a torch.cuda.Stream object (2 us less per call)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _current_stream(device_index):
    if device_index is None or device_index < 0:
        return None
    if _raw_stream is not None:
        return _raw_stream(device_index)
    return torch.cuda.current_stream(device_index).cuda_stream


def call(name: str, *args):
    """Call entry point ``name``.  torch tensors become descriptors, None stays NULL, str is
    encoded; the current stream of the first GPU tensor's device is appended."""
    lib = load_library()
    fn = getattr(lib, name)
    c_args, keep, device = [], [], None
    for a in args:
        if isinstance(a, torch.Tensor):
            if device is None and a.is_cuda:
                device = a.device.index
            at = shared_descriptor(a)
            keep.append(at)
            c_args.append(ctypes.byref(at))
        elif isinstance(a, str):
            c_args.append(a.encode())
        elif isinstance(a, bool):
            c_args.append(1 if a else 0)
        else:
            c_args.append(a)
    c_args.append(ctypes.c_void_p(_current_stream(device)))
    lib.aiter_clear_last_error()
    status = fn(*c_args)
    if status != 0:
        raw = lib.aiter_get_last_error()
        msg = raw.decode(errors="replace") if raw else f"ctypes status={status}"
        lib.aiter_clear_last_error()
        raise RuntimeError(f"{name} failed: {msg}")
    return None


def gemm_kernel_names():
    return load_library().aiter_fp8bs_gemm_kernel_names().decode().split(",")


def gemm_choice(m: int, n: int, k: int, preshuffled: bool = False) -> str:
    lib = load_library()
    buf = ctypes.create_string_buffer(64)
    if lib.aiter_fp8bs_gemm_choice(int(m), int(n), int(k), 1 if preshuffled else 0, buf, 64) != 0:
        raw = lib.aiter_get_last_error()
        raise RuntimeError(f"aiter_fp8bs_gemm_choice failed: {raw.decode(errors='replace') if raw else '?'}")
    return buf.value.decode()


def gemm_resolve(m: int, n: int, k: int, split_k: int = 0, kernel_name: str = "", preshuffled: bool = False):
    """(kernel, splitK) that a call with this (kernelName, splitK) pair runs; host-only."""
    lib = load_library()
    buf = ctypes.create_string_buffer(96)
    if lib.aiter_fp8bs_gemm_resolve(int(m), int(n), int(k), 1 if preshuffled else 0, int(split_k),
                                    (kernel_name or "").encode(), buf, 96) != 0:
        raw = lib.aiter_get_last_error()
        raise RuntimeError(f"aiter_fp8bs_gemm_resolve failed: {raw.decode(errors='replace') if raw else '?'}")
    name, _, tail = buf.value.decode().partition(";splitK=")
    return name, int(tail)
