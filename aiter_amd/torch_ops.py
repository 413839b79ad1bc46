"""``torch.ops.aiter.*`` registration of this path's entry points, with fake (shape-only)
implementations so that ``torch.compile`` / FakeTensor tracing sees them as single opaque calls.

The reference wraps its bindings the same way (aiter/jit/utils/torch_guard.py:200-357: a
``Library("aiter", "FRAGMENT")``, one op per function name, real kernels for the CUDA and CPU
keys, a fake for tracing; fakes for the GEMMs at aiter/ops/gemm_op_a8w8.py:790-801,893-905).
Here the schemas are written out (the set of ops is small and fixed) and two rules keep the ops
usable under functionalisation, which the reference's generic wrapper does not guarantee:

* an op that writes into an argument declares it ``Tensor(a!)`` and returns nothing; where the
  reference's Python function hands the written tensor back, the Python entry point returns it
  itself;
* an op never returns one of its inputs.

Eager calls bypass the dispatcher (one ctypes call, no schema matching): only while a compiler is
tracing does an entry point go through ``torch.ops.aiter``.
"""

from __future__ import annotations

import functools
from typing import Callable, Optional

import torch

_lib: Optional[torch.library.Library] = None
REGISTERED: dict = {}  # op name -> schema, for the ops this module defined


def _library() -> torch.library.Library:
    global _lib
    if _lib is None:
        _lib = torch.library.Library("aiter", "FRAGMENT")
    return _lib


def _defined(name: str) -> bool:
    try:
        getattr(torch.ops.aiter, name)
        return True
    except (AttributeError, RuntimeError):
        return False


def torch_op(schema: str, fake: Callable):
    """Register ``fn`` as ``torch.ops.aiter.<name>`` with ``schema`` (name included) and return
    the entry point: ``fn`` itself in eager mode, the registered op while compiling.  If another
    library has already defined an op of that name in this process, nothing is registered and
    ``fn`` is returned unchanged."""

    def deco(fn):
        name = schema[: schema.index("(")]
        if _defined(name):
            return fn
        lib = _library()
        lib.define(schema)
        lib.impl(name, fn, "CUDA")
        lib.impl(name, fn, "CPU")  # CPU tensors reach the library's own "must live in GPU memory" error
        torch.library.register_fake(f"aiter::{name}", fake, lib=lib)
        REGISTERED[name] = schema
        op = getattr(torch.ops.aiter, name)

        @functools.wraps(fn)
        def entry(*args, **kwargs):
            if torch.compiler.is_compiling():
                return op(*args, **kwargs)
            return fn(*args, **kwargs)

        entry.op = op
        entry.eager = fn
        return entry

    return deco


def fake_none(*args, **kwargs) -> None:
    """Fake of an op that only writes into its ``Tensor(a!)`` arguments."""
    return None
