"""dtype aliases and the ctypes mirror of ``aiter_tensor_t``.

Mirrors aiter/utility/dtypes.py:11-60 (aliases; on gfx950 ``fp8`` is OCP e4m3fn) and
aiter/utility/aiter_types.py:55-87 + aiter/utility/dtypes.py:101-129 (descriptor and
``torch_to_aiter``) of the reference.
"""

from __future__ import annotations

import ctypes

import torch

fp8 = torch.float8_e4m3fn  # gfx950: OCP format (aiter/utility/dtypes.py:11-13)
fp8_e8m0 = getattr(torch, "float8_e8m0fnu", None)
fp16 = torch.float16
bf16 = torch.bfloat16
fp32 = torch.float32
i8 = torch.int8
u8 = torch.uint8
i16 = torch.int16
i32 = torch.int32
u32 = getattr(torch, "uint32", None)
i64 = torch.int64
u64 = getattr(torch, "uint64", None)

# csrc/include/aiter_enum.h:34-51
AITER_DTYPE = {
    "fp8": 0,
    "fp8_e8m0": 1,
    "fp16": 2,
    "bf16": 3,
    "fp32": 4,
    "i4x2": 5,
    "fp4x2": 6,
    "u32": 7,
    "i32": 8,
    "i16": 9,
    "i8": 10,
    "u8": 11,
    "i64": 12,
    "u64": 13,
}

_TORCH_TO_ID = {
    fp8: AITER_DTYPE["fp8"],
    fp16: AITER_DTYPE["fp16"],
    bf16: AITER_DTYPE["bf16"],
    fp32: AITER_DTYPE["fp32"],
    i32: AITER_DTYPE["i32"],
    i16: AITER_DTYPE["i16"],
    i8: AITER_DTYPE["i8"],
    u8: AITER_DTYPE["u8"],
    i64: AITER_DTYPE["i64"],
}
for _t, _n in ((fp8_e8m0, "fp8_e8m0"), (u32, "u32"), (u64, "u64")):
    if _t is not None:
        _TORCH_TO_ID[_t] = AITER_DTYPE[_n]


class aiter_tensor_t(ctypes.Structure):
    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("numel_", ctypes.c_size_t),
        ("ndim", ctypes.c_int),
        ("shape", ctypes.c_int64 * 8),
        ("strides", ctypes.c_int64 * 8),
        ("dtype_", ctypes.c_int),
        ("device_id", ctypes.c_int),
    ]


assert ctypes.sizeof(aiter_tensor_t) == 160, "aiter_tensor_t must be 160 bytes (include/aiter_fp8bs.h)"


def torch_to_aiter(tensor: torch.Tensor) -> aiter_tensor_t:
    """Zero-copy descriptor of a torch tensor (borrowed: keep the tensor alive)."""
    shape = tuple(tensor.shape)
    ndim = len(shape)
    if ndim > 8:
        raise ValueError(f"aiter_tensor_t supports at most 8 dims, got {ndim}")
    try:
        dtype_id = _TORCH_TO_ID[tensor.dtype]
    except KeyError:
        raise TypeError(f"unsupported tensor dtype {tensor.dtype}") from None
    at = aiter_tensor_t()
    at.ptr = tensor.data_ptr()
    at.numel_ = tensor.numel()
    at.ndim = ndim
    at.shape[:ndim] = shape
    at.strides[:ndim] = tuple(tensor.stride())
    at.dtype_ = dtype_id
    index = tensor.device.index
    at.device_id = -1 if (tensor.device.type == "cpu" or index is None) else index
    return at


_DESCRIPTORS: dict = {}
_DESCRIPTORS_MAX = 4096


def shared_descriptor(tensor: torch.Tensor) -> aiter_tensor_t:
    """``torch_to_aiter`` through a cache, for the call bridge.  A descriptor is a pure function of
    (address, shape, strides, dtype, device) and the library only reads it, so one structure can serve
    every call that passes the same buffer the same way: building one costs 2 us, finding one 0.7 us,
    and a decode step passes the same weights and buffers again and again.  Never modify what this
    returns."""
    key = (tensor.data_ptr(), tensor.shape, tensor.stride(), tensor.dtype, tensor.device)
    at = _DESCRIPTORS.get(key)
    if at is None:
        at = torch_to_aiter(tensor)
        if len(_DESCRIPTORS) >= _DESCRIPTORS_MAX:
            _DESCRIPTORS.clear()
        _DESCRIPTORS[key] = at
    return at
