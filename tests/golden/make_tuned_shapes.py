"""Writes tests/golden/tuned_gemm_requests.npz: the (M, N, K, splitK) columns of the reference's
tuned block-scale GEMM table, aiter/configs/model_configs/a8w8_blockscale_tuned_gemm_ds_v3.csv,
plus one representative kernel name of its zoo.  Data only: what callers of the reference forward
to gemm_a8w8_blockscale_ck as (splitK, kernelName).  Run in the development container, where the
reference checkout is mounted:  python tests/golden/make_tuned_shapes.py
"""

import csv
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = "/root/reference/aiter/configs/model_configs/a8w8_blockscale_tuned_gemm_ds_v3.csv"


def main():
    if not os.path.exists(SRC):
        sys.exit(f"{SRC} not found")
    rows = list(csv.DictReader(open(SRC)))
    table = np.array([[int(r["M"]), int(r["N"]), int(r["K"]), int(r["splitK"])] for r in rows], dtype=np.int32)
    names = sorted({r["kernelName"] for r in rows})
    out = os.path.join(HERE, "tuned_gemm_requests.npz")
    np.savez_compressed(out, mnk_splitk=table, kernel_names=np.array(names))
    print(f"{out}: {len(table)} rows, {len(names)} kernel names, splitK in {sorted(set(table[:, 3].tolist()))}")


if __name__ == "__main__":
    main()
