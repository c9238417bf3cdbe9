"""Writes tests/golden/quantization_reference_op_vectors.npz: inputs and outputs of the
REFERENCE's own compiled quantisation kernels (oracle/_ref, built by oracle/build_ref.sh
from the reference sources in place; the x86 variants,
self_benchmark/a64fx/model/ops/src/quantization_x86.cpp:17-305) on small seeded cases, so
that the oracle can be checked against them on machines where that build is not available.

Cases: row-packed ``quantize_tensor`` / ``dequantize_tensor`` for 2, 4 and 8 bits with row
counts that are and are not multiples of the rows per byte and widths around the 16-float
vector edge (:55-60, :82-96); mixed-bits ``quantize_tensor_v1`` / ``dequantize_tensor_v1``
with every width per row, a constant row (scale 0 -> 1, :203-204) and odd feature counts.

Run from the repository root:  python tests/golden/make_quantization_reference_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import quantization as oq  # noqa: E402
from oracle import spmm as ospmm  # noqa: E402


def main():
    import torch

    ref = ospmm.load_reference_op()
    if ref is None:
        raise SystemExit("oracle/_ref is not built (run oracle/build_ref.sh on an AVX-512 host)")
    out = {}
    case = 0
    for bits in (2, 4, 8):
        epb = 8 // bits
        for rows, feat in ((8, 16), (7, 5), (13, 47), (1, 33), (64, 130)):
            rng = np.random.default_rng(5000 + case)
            x = (rng.standard_normal((rows, feat)) * rng.uniform(0.1, 30.0, (rows, 1))).astype(np.float32)
            if rows > 2:
                x[2] = 0.75  # constant row
            params = oq.row_params(x, bits)
            packed = torch.zeros((-(-rows // epb), feat), dtype=torch.uint8)
            ref.quantize_tensor(torch.from_numpy(x), packed, torch.from_numpy(params[:, 0].copy()),
                                torch.from_numpy(params[:, 1].copy()), bits)
            back = torch.zeros((rows, feat), dtype=torch.float32)
            ref.dequantize_tensor(packed, back, torch.from_numpy(params[:, 0].copy()),
                                  torch.from_numpy(params[:, 1].copy()), bits)
            for name, arr in (("x", x), ("params", params), ("packed", packed.numpy()), ("back", back.numpy())):
                out[f"rows{case}_{name}"] = arr
            out[f"rows{case}_bits"] = np.int64(bits)
            case += 1
    out["rows_cases"] = np.int64(case)

    case = 0
    for rows, feat in ((5, 3), (9, 16), (12, 47), (6, 130), (3, 1)):
        rng = np.random.default_rng(7000 + case)
        x = (rng.standard_normal((rows, feat)) * rng.uniform(0.1, 30.0, (rows, 1))).astype(np.float32)
        x[1] = -2.5
        node_bits = rng.choice([8, 4, 2], rows).astype(np.float32)
        node_bits[:3] = (8, 4, 2)
        feat_range = oq.get_quantized_nodes_feat_range(rows, feat, node_bits)
        params = torch.zeros((rows, 3), dtype=torch.float32)
        params[:, 0] = torch.from_numpy(node_bits)
        data = torch.zeros(int(feat_range[-1]), dtype=torch.uint8)
        ref.quantize_tensor_v1(torch.from_numpy(x), data, torch.from_numpy(feat_range), params)
        back = torch.zeros((rows, feat), dtype=torch.float32)
        ref.dequantize_tensor_v1(data, back, torch.from_numpy(feat_range), params)
        for name, arr in (("x", x), ("bits", node_bits), ("range", feat_range), ("params", params.numpy()),
                          ("data", data.numpy()), ("back", back.numpy())):
            out[f"mixed{case}_{name}"] = arr
        case += 1
    out["mixed_cases"] = np.int64(case)

    path = os.path.join(ROOT, "tests", "golden", "quantization_reference_op_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
