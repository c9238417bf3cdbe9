"""Pins the codec oracle (oracle/quantization.py) to the reference: its own golden bytes
(self_benchmark/a64fx/tests/test_quantizer.py), committed outputs of its compiled x86
kernels, the live compiled kernels where oracle/_ref is built, and brute force."""
import os

import numpy as np

from oracle import quantization as oq

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "quantization_reference_op_vectors.npz")

# tests/test_quantizer.py:58-84 and :87-114 of the reference
REF_X = np.array([[0.2, 0.1, 0.3], [0.4, 0.5, 0.6], [0.7, 0.8, 0.9], [1.0, 1.1, 1.2], [0.3, 0.1, 0.7]], dtype=np.float32)
REF_BITS = [8, 4, 2, 4, 4]
REF_BYTES = [127, 0, 255, 7, 240, 44, 8, 240, 80, 240]


def test_mixed_bits_golden_bytes_of_the_reference():
    data, params = oq.quantize_mixed(REF_X, REF_BITS)
    assert data.tolist() == REF_BYTES
    assert oq.get_quantized_nodes_feat_range(5, 3, REF_BITS).tolist() == [0, 3, 5, 6, 8, 10]
    want = np.empty((5, 3), dtype=np.float32)
    want[:, 0] = REF_BITS
    want[:, 1] = REF_X.min(axis=1)
    want[:, 2] = (REF_X.max(axis=1) - want[:, 1]) / (2.0 ** want[:, 0] - 1)
    np.testing.assert_allclose(params, want, rtol=1e-5, atol=1e-8)  # torch.allclose defaults, test_quantizer.py:83


def test_mixed_bits_dequantise_golden_of_the_reference():
    params = np.array([[8, 0.1, 7.8431e-04], [4, 0.4, 1.3333e-02], [2, 0.7, 6.6667e-02], [4, 1.0, 1.3333e-02],
                       [4, 0.1, 4.0000e-02]], dtype=np.float32)
    back = oq.dequantize_mixed(np.array(REF_BYTES, dtype=np.uint8), params, 3)
    # The reference asserts allclose(back, original) (test_quantizer.py:114), which no 2..8-bit code
    # can meet (0.2 -> byte 127 -> 0.19961); its compiled kernel returns exactly what the oracle
    # does (see the compiled-reference tests below).  What holds is half a step per element.
    # (the vector's scales are printed to five digits, hence the slack)
    assert (np.abs(back - REF_X) <= params[:, 2:3] * 0.5 * 1.001 + 1e-5).all()
    want_row0 = np.float32(0.1) + np.array([127, 0, 255], dtype=np.float32) * np.float32(7.8431e-04)
    np.testing.assert_allclose(back[0], want_row0, rtol=1e-6)


def test_feat_range_vectors_of_the_reference():
    # test_quantizer.py:29-56
    assert oq.get_quantized_nodes_feat_range(6, 4, [8, 4, 2, 8, 4, 2]).tolist() == [0, 4, 6, 7, 11, 13, 14]
    assert oq.get_quantized_nodes_feat_range(3, 1, [2, 2, 2]).tolist() == [0, 1, 2, 3]
    assert oq.get_quantized_nodes_feat_range(3, 3, [4, 4, 2]).tolist() == [0, 2, 4, 5]


def test_splits_for_quantised_exchange_vector_of_the_reference():
    # test_quantizer.py:10-27
    recv, send = oq.get_splits_for_comm_quantized_data([2, 0, 4, 1], [0, 3, 0, 3], [0, 2, 4, 6, 8, 12, 13, 19],
                                                       [0, 1, 2, 5, 7, 11, 30])
    assert recv == [4, 0, 9, 6] and send == [0, 5, 0, 25]


def _check_rows_case(z, c, quantize, dequantize):
    x, p, bits = z[f"rows{c}_x"], z[f"rows{c}_params"], int(z[f"rows{c}_bits"])
    packed = quantize(x, p[:, 0], p[:, 1], bits)
    assert np.array_equal(packed, z[f"rows{c}_packed"]), (c, bits)
    back = dequantize(packed, p[:, 0], p[:, 1], x.shape[0], bits)
    assert np.array_equal(back, z[f"rows{c}_back"]), (c, bits)


def test_row_packed_oracle_equals_committed_outputs_of_the_compiled_reference():
    z = np.load(GOLDEN)
    for c in range(int(z["rows_cases"])):
        _check_rows_case(z, c, oq.quantize_rows, oq.dequantize_rows)


def test_mixed_oracle_equals_committed_outputs_of_the_compiled_reference():
    z = np.load(GOLDEN)
    for c in range(int(z["mixed_cases"])):
        x, bits = z[f"mixed{c}_x"], z[f"mixed{c}_bits"]
        data, params = oq.quantize_mixed(x, bits)
        assert np.array_equal(data, z[f"mixed{c}_data"])
        assert np.array_equal(params, z[f"mixed{c}_params"])
        assert np.array_equal(oq.get_quantized_nodes_feat_range(x.shape[0], x.shape[1], bits), z[f"mixed{c}_range"])
        assert np.array_equal(oq.dequantize_mixed(data, params, x.shape[1]), z[f"mixed{c}_back"])


def test_oracle_equals_live_compiled_reference(reference_op):
    import torch

    rng = np.random.default_rng(11)
    for bits in (2, 4, 8):
        epb = 8 // bits
        for rows, feat in ((37, 100), (4, 16), (5, 602)):
            x = (rng.standard_normal((rows, feat)) * 7).astype(np.float32)
            p = oq.row_params(x, bits)
            packed = torch.zeros((-(-rows // epb), feat), dtype=torch.uint8)
            reference_op.quantize_tensor(torch.from_numpy(x), packed, torch.from_numpy(p[:, 0].copy()),
                                         torch.from_numpy(p[:, 1].copy()), bits)
            assert np.array_equal(packed.numpy(), oq.quantize_rows(x, p[:, 0], p[:, 1], bits))
            back = torch.zeros((rows, feat))
            reference_op.dequantize_tensor(packed, back, torch.from_numpy(p[:, 0].copy()),
                                           torch.from_numpy(p[:, 1].copy()), bits)
            assert np.array_equal(back.numpy(), oq.dequantize_rows(packed.numpy(), p[:, 0], p[:, 1], rows, bits))


def test_segments_are_packed_one_by_one_brute_force():
    """Scalar loops over (segment, row, column): each rank's rows start a new byte group,
    row k of a group sits at bit (epb-k-1)*bits, params are the row's own min and range."""
    rng = np.random.default_rng(3)
    for bits in (2, 4, 8):
        epb = 8 // bits
        splits = [3, 0, 6, 1, 5]
        x = (rng.standard_normal((sum(splits), 7)) * 3).astype(np.float32)
        x[4] = 1.25
        packed, params = oq.quantize_segments(x, splits, bits)
        assert packed.shape == (sum(-(-s // epb) for s in splits), 7)
        row, prow = 0, 0
        for s in splits:
            for local in range(s):
                lo, hi = x[row].min(), x[row].max()
                scale = np.float32(np.float32(hi - lo) / np.float32((1 << bits) - 1)) or np.float32(1.0)
                assert params[row, 0] == lo and params[row, 1] == scale
                for j in range(7):
                    q = int(np.rint(np.float32(np.float32(x[row, j] - lo) / scale)))
                    assert 0 <= q < (1 << bits)
                    byte = int(packed[prow + local // epb, j])
                    assert (byte >> ((epb - local % epb - 1) * bits)) & ((1 << bits) - 1) == q
                row += 1
            # bits of rows a partial group lacks stay 0
            if s % epb:
                used = s % epb
                assert not (packed[prow + s // epb] & ((1 << ((epb - used) * bits)) - 1)).any()
            prow += -(-s // epb)
        back = oq.dequantize_segments(packed, params, splits, bits)
        # half a quantisation step per element, plus rounding
        assert (np.abs(back - x) <= params[:, 1:2] * 0.5 * (1 + 1e-5) + 1e-6).all()
        # a constant row survives exactly
        assert np.array_equal(back[4], x[4])
        # composition: a segment alone gives the same bytes
        a = splits[0] + splits[1]
        alone, _ = oq.quantize_segments(x[a:a + splits[2]], [splits[2]], bits)
        begin = sum(-(-s // epb) for s in splits[:2])
        assert np.array_equal(alone, packed[begin:begin + alone.shape[0]])


def test_bf16_round_trip_matches_torch():
    import torch

    rng = np.random.default_rng(5)
    x = np.concatenate([(rng.standard_normal(5000) * 10.0 ** rng.integers(-20, 20, 5000)).astype(np.float32),
                        np.array([0.0, -0.0, 1.00390625, 1.01171875, np.inf, -np.inf, 3.3895314e38, 1e-40], dtype=np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    assert np.array_equal(oq.to_bf16_and_back(x).view(np.uint32), want.view(np.uint32))
    # NaN stays NaN; which NaN differs between torch's own scalar and vector code, so only that much is pinned
    assert np.isnan(oq.to_bf16_and_back(np.array([np.nan, -np.nan], dtype=np.float32))).all()
