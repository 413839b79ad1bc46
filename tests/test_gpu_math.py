"""The short arithmetic forms of aiter_amd/csrc/fp8bs_math.h against the operations they stand for, on the GPU:
the test-only library tests/gpu_math/libgpu_math_check.so (built by __graft_entry__.build()) includes the
header the kernels include."""
import ctypes
import os

import pytest

LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpu_math", "libgpu_math_check.so")


def load():
    if not os.path.exists(LIB):  # a fresh checkout: build it as __graft_entry__.build() does (hipcc cross-compiles)
        import sys

        sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
        import __graft_entry__

        __graft_entry__.build_gpu_math_check()
    lib = ctypes.CDLL(LIB)
    for name in ("gpu_math_recip_sweep", "gpu_math_mean_sweep"):
        fn = getattr(lib, name)
        fn.argtypes = [ctypes.c_uint32, ctypes.c_uint32, ctypes.POINTER(ctypes.c_ulonglong),
                       ctypes.POINTER(ctypes.c_uint32)]
        fn.restype = ctypes.c_int
    lib.gpu_math_recip_min_bits.restype = ctypes.c_uint32
    lib.gpu_math_recip_max_bits.restype = ctypes.c_uint32
    return lib


def test_check_library_is_built_and_exports_its_entry_points():
    lib = load()
    assert lib.gpu_math_recip_min_bits() == (127 - 100) << 23 and lib.gpu_math_recip_max_bits() == (127 + 100) << 23


@pytest.mark.gpu
def test_short_reciprocal_equals_the_division_for_every_float_in_its_range():
    lib = load()
    bad, example = ctypes.c_ulonglong(0), ctypes.c_uint32(0)
    lo, hi = lib.gpu_math_recip_min_bits(), lib.gpu_math_recip_max_bits() + 1  # 2^-100 ... 2^100 inclusive
    assert lib.gpu_math_recip_sweep(lo, hi, ctypes.byref(bad), ctypes.byref(example)) == 0
    assert bad.value == 0, f"{bad.value} of {2 * (hi - lo)} reciprocals differ, e.g. for bits {example.value:#010x}"


@pytest.mark.gpu
def test_quotient_by_the_row_length_equals_the_fp64_division():
    lib = load()
    bad, example = ctypes.c_ulonglong(0), ctypes.c_uint32(0)
    # row lengths 1 .. 16384 (the kernels take up to 8192), 4096 sums each plus 0, inf and the length itself
    assert lib.gpu_math_mean_sweep(16384, 4096, ctypes.byref(bad), ctypes.byref(example)) == 0
    assert bad.value == 0, f"{bad.value} quotients differ, e.g. for row length {example.value}"
