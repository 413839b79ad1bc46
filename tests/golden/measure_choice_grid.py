"""Measures, on an MI355X, both kernel families that serve small batches -- the weight-streaming
kernel (`decode_stream`) and the library's best `mid_*` tiling (`mid_auto`) -- over 1 ... 64 rows on
fourteen weight shapes (0.5 ... 117 MB), weights cycled through 700 MB so that every launch streams
them from HBM, and writes the durations (us per launch of a replayed graph) to
tests/golden/choice_grid_m1_to_64.json.  tests/test_gemm_requests_host.py holds the library's
automatic choice against these figures.

    python tests/golden/measure_choice_grid.py        (needs the GPU; about a minute)
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import torch

import aiter_amd
from aiter_amd import dtypes
from bench import quant_weight_gpu, time_launches

SHAPES = [(24576, 1536), (7168, 2048), (2112, 7168), (4096, 7168), (1536, 7168), (576, 7168), (32768, 512),
          (7168, 16384), (3072, 1536), (4608, 7168), (7168, 256), (16384, 4096), (1024, 2048), (8192, 1024)]
ROWS = (1, 8, 16, 24, 32, 48, 64)


def main():
    dev = "cuda:0"
    quant = aiter_amd.get_hip_quant(aiter_amd.QuantType.per_1x128)
    out_rows = []
    for n, k in SHAPES:
        copies = max(8, 700_000_000 // (n * k) + 1)
        wq0, ws = quant_weight_gpu(torch, dtypes.fp8, n, k, 1, dev)
        wqs = [wq0] + [wq0.clone() for _ in range(copies - 1)]
        for m in ROWS:
            xq, xs = quant(torch.randn(m, k, device=dev).bfloat16())
            out = torch.empty(m, n, dtype=torch.bfloat16, device=dev)

            def timed(kernel):
                i = [0]

                def call():
                    i[0] = (i[0] + 1) % copies
                    aiter_amd.gemm_a8w8_blockscale_ck(xq, wqs[i[0]], xs, ws, out, splitK=-1, kernelName=kernel)

                return round(time_launches(torch, call, copies, 3) * 1e6, 3)

            row = {"M": m, "N": n, "K": k, "decode_stream": timed("decode_stream"), "mid_auto": timed("mid_auto")}
            out_rows.append(row)
            print(row, flush=True)
        del wqs
        torch.cuda.empty_cache()
    path = os.path.join(ROOT, "tests", "golden", "choice_grid_m1_to_64.json")
    with open(path, "w") as f:
        json.dump({"device": torch.cuda.get_device_name(0), "unit": "us per launch, graph replay, weights from HBM",
                   "rows": out_rows}, f, indent=0)
    print("wrote", path)


if __name__ == "__main__":
    main()
