"""Writes tests/golden/spmm_reference_op_vectors.npz: inputs and outputs of the
REFERENCE's own compiled operator (oracle/_ref, built by oracle/build_ref.sh from the
reference sources in place) on small seeded cases, so that parity with the reference can
be checked on machines where that build is not available.

Cases straddle the reference's 16-float vector and 64-float main-block edges
(self_benchmark/a64fx/model/ops/src/spmm.cpp:452-479), start from a non-zero ``out``
(accumulate semantics, :32-35) and include empty rows and repeated column indices.

Run from the repository root:  python tests/golden/make_spmm_reference_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import spmm as ospmm  # noqa: E402


def main():
    import torch

    ref = ospmm.load_reference_op()
    if ref is None:
        raise SystemExit("oracle/_ref is not built (run oracle/build_ref.sh on an AVX-512 host)")
    out = {}
    for case, (rows, cols, feat, mean_deg) in enumerate([(60, 50, 47, 5), (50, 80, 100, 9), (48, 40, 130, 14),
                                                          (40, 50, 16, 3), (16, 20, 602, 6)]):
        rng = np.random.default_rng(1000 + case)
        deg = rng.poisson(mean_deg, rows)
        deg[::5] = 0
        deg[3] = 300  # one long row
        rowptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int64)
        col = rng.integers(0, cols, rowptr[-1]).astype(np.int64)
        for r in range(rows):
            col[rowptr[r]:rowptr[r + 1]].sort()
        val = rng.standard_normal(rowptr[-1]).astype(np.float32)
        x = rng.standard_normal((cols, feat)).astype(np.float32)
        out0 = rng.standard_normal((rows, feat)).astype(np.float32)
        threads = torch.get_num_threads()
        res = torch.from_numpy(out0.copy())
        ref.spmm(torch.from_numpy(rowptr), torch.from_numpy(col), torch.from_numpy(val), torch.from_numpy(x), res, rows,
                 torch.from_numpy(ospmm.divide_work(rows, threads)), torch.tensor([0, feat], dtype=torch.int32))
        for name, arr in (("rowptr", rowptr), ("col", col), ("val", val), ("x", x), ("out0", out0), ("out", res.numpy())):
            out[f"c{case}_{name}"] = arr
    path = os.path.join(ROOT, "tests", "golden", "spmm_reference_op_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
