"""Shared helpers for the parity tests (oracle = checker only)."""

import numpy as np
import torch

from oracle import c_oracle as co
from oracle import torch_ref as tr

GUARD = 0xA5  # canary byte written around outputs, as the reference's fused-norm test does
              # (op_tests/test_rmsnorm2dFusedAddQuant.py:20,264-271)


def bits32(t):
    """fp32 tensor/array -> uint32 numpy view."""
    if isinstance(t, torch.Tensor):
        t = t.detach().cpu().contiguous().numpy()
    return np.ascontiguousarray(t, dtype=np.float32).view(np.uint32)


def codes8(t):
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def codes16(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_codes16(a, dtype=torch.bfloat16):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(dtype)


def guarded_empty(shape, dtype, device, pad_bytes=512):
    """Uninitialised-looking tensor carved out of a byte buffer filled with the guard pattern,
    with pad_bytes of guard on either side.  Returns (tensor, check) where check() asserts
    the guard bands are intact."""
    numel = int(np.prod(shape)) if len(shape) else 1
    nbytes = numel * torch.empty((), dtype=dtype).element_size()
    # keep 256-byte alignment of the payload
    pad = (pad_bytes + 255) // 256 * 256
    raw = torch.full((pad + nbytes + pad,), GUARD, dtype=torch.uint8, device=device)
    t = raw[pad : pad + nbytes].view(dtype).view(*shape)

    def check():
        assert bool((raw[:pad] == GUARD).all()), "guard band before the output was overwritten"
        assert bool((raw[pad + nbytes :] == GUARD).all()), "guard band after the output was overwritten"

    return t, check


def assert_quant_bit_exact(y, s, x_cpu, group=128, in_dtype="bf16", what=""):
    """y/s from the GPU vs the C oracle on the same 16-bit inputs: codes and scales bit-exact."""
    yo, so = co.group_quant(codes16(x_cpu), in_dtype=in_dtype, group=group)
    yg = codes8(y).reshape(yo.shape)
    sg = bits32(s).reshape(so.shape)
    bad_c = int((yg != yo).sum())
    bad_s = int((sg != so.view(np.uint32)).sum())
    detail = ""
    if bad_c:
        xc = codes16(x_cpu).reshape(yo.shape)
        idx = np.argwhere(yg != yo)[:8]
        detail = "; first mismatches (x code, got, want, scale bits): " + ", ".join(
            f"{xc[tuple(i)]:#06x}:{yg[tuple(i)]:#04x}!={yo[tuple(i)]:#04x}@{so.view(np.uint32).reshape(-1)[np.ravel_multi_index(tuple(i), yo.shape) // group]:#010x}"
            for i in idx
        )
    assert bad_c == 0 and bad_s == 0, f"{what}: {bad_c} code mismatches, {bad_s} scale mismatches{detail}"
