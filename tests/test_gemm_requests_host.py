"""CPU: what the reference's callers forward as (splitK, kernelName) never makes the GEMM entry
points fail.  Every row of the reference's tuned table
(aiter/configs/model_configs/a8w8_blockscale_tuned_gemm_ds_v3.csv; its four integer columns and its
kernel names are kept as data in tests/golden/tuned_gemm_requests.npz) goes through the library's
own resolution of such a request, host-only: aiter_fp8bs_gemm_resolve runs the code the GEMM entry
points run to turn (shape, kernelName, splitK) into a kernel."""

import os

import numpy as np
import pytest

import aiter_amd
from aiter_amd import _ffi

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tuned_gemm_requests.npz")


@pytest.fixture(scope="module")
def table():
    z = np.load(GOLDEN)
    return z["mnk_splitk"], [str(n) for n in z["kernel_names"]]


def family(name):
    return name.split(":")[0]


def test_every_tuned_row_resolves(table):
    rows, names = table
    own = set(aiter_amd.gemm_kernel_names())
    assert len(rows) > 7000 and set(rows[:, 3].tolist()) == {0, 1, 2, 3}
    assert all(n.startswith("a8w8_blockscale_") for n in names)
    for i, (m, n, k, s) in enumerate(rows.tolist()):
        foreign = names[i % len(names)]
        # with the table's kernel name: the name and the splitK tuned for it are both dropped
        kern, split = _ffi.gemm_resolve(m, n, k, s, foreign)
        assert family(kern) in own and split == -1, (m, n, k, s, kern, split)
        assert kern == _ffi.gemm_choice(m, n, k), (m, n, k)
        # with no name: splitK > 0 is a hint for the kernel the library chooses, 0 means choose
        kern2, split2 = _ffi.gemm_resolve(m, n, k, s, "")
        assert family(kern2) in own and family(kern2) == family(kern)
        assert split2 == (s if s > 0 else -1)


def test_split_hint_range_and_names():
    for s in (-1, 0, 1, 4, 5, 17, 30):
        for shape in ((1, 7168, 2048), (128, 7168, 2048), (8192, 36864, 7168), (3258, 128, 7168)):
            kern, split = _ffi.gemm_resolve(*shape, s, "")
            assert split == (s if s > 0 else -1) and family(kern) in aiter_amd.gemm_kernel_names()
            for name in aiter_amd.gemm_kernel_names():
                assert _ffi.gemm_resolve(*shape, s, name) == (name, s)
    for s in (-2, 31, 1000):
        with pytest.raises(RuntimeError, match="splitK"):
            _ffi.gemm_resolve(16, 256, 512, s, "")
    with pytest.raises(RuntimeError, match="unknown kernelName"):
        _ffi.gemm_resolve(16, 256, 512, 0, "no_such_kernel")
    with pytest.raises(RuntimeError, match="unknown kernelName"):
        _ffi.gemm_resolve(16, 256, 512, 0, "mid_128x128:s=0")
    assert _ffi.gemm_resolve(16, 256, 512, 2, "decode_stream:r=2,s=4") == ("decode_stream:r=2,s=4", 2)
    assert _ffi.gemm_resolve(300, 256, 512, 1, "prefill_256x256:s=2") == ("prefill_256x256:s=2", 1)


def test_choice_below_65_rows_against_measured_durations():
    """The automatic choice between the weight-streaming kernel and the mid_* tilings, held against
    durations of both measured on an MI355X (tests/golden/choice_grid_m1_to_64.json, written by
    tests/golden/measure_choice_grid.py: 1 ... 64 rows x fourteen weight shapes): what the choice
    loses against the faster family is 1 % at most on average and 10 % at worst, and where one
    family is ahead by a quarter the choice takes it."""
    import json

    with open(os.path.join(os.path.dirname(__file__), "golden", "choice_grid_m1_to_64.json")) as f:
        rows = json.load(f)["rows"]
    assert len(rows) == 98
    losses = []
    for r in rows:
        chosen = "decode_stream" if _ffi.gemm_choice(r["M"], r["N"], r["K"]).startswith("decode_stream") else "mid_auto"
        other = "mid_auto" if chosen == "decode_stream" else "decode_stream"
        losses.append(r[chosen] / min(r["decode_stream"], r["mid_auto"]) - 1.0)
        assert r[chosen] <= 1.10 * r[other], (r, chosen)
        if r[other] > 1.25 * r[chosen] or r[chosen] > 1.25 * r[other]:
            assert r[chosen] < r[other], (r, chosen)
    assert sum(losses) / len(losses) <= 0.01, sum(losses) / len(losses)
