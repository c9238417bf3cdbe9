"""GPU parity of the boundary-buffer codec against the oracle (oracle/quantization.py,
itself pinned to the reference's golden bytes and compiled kernels): packed bytes and
parameters bit-exact, dequantised rows bit-exact (one fused multiply-add per element)."""
import os

import numpy as np
import pytest
import torch

from oracle import quantization as oq

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "quantization_reference_op_vectors.npz")


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _rows(rng, rows, feat):
    x = (rng.standard_normal((rows, feat)) * rng.uniform(0.01, 50.0, (rows, 1))).astype(np.float32)
    if rows > 3:
        x[3] = -4.5  # constant row: scale 0 -> 1
    return x


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("feat", [1, 3, 16, 47, 64, 100, 128, 130, 256, 260, 602, 1024, 1028, 2052])
def test_segments_codec_matches_oracle(bits, feat):
    from gnn_benchmark_amd import computation_ops as ops

    rng = np.random.default_rng(1000 * bits + feat)
    splits = [5, 0, 13, 1, 8, 0, 4, 7]
    rows = sum(splits)
    x = _rows(rng, rows, feat)
    want_packed, want_params = oq.quantize_segments(x, splits, bits)
    work_range = torch.tensor(np.concatenate(([0], np.cumsum(splits))), dtype=torch.int32)
    packed = torch.full(want_packed.shape, 0xAB, dtype=torch.uint8, device="cuda")
    params = torch.full((rows, 2), -7.0, device="cuda")
    ops.quantize_tensor_for_all_procs(dev(x), packed, params, work_range, len(splits), bits)
    assert np.array_equal(params.cpu().numpy(), want_params)
    assert np.array_equal(packed.cpu().numpy(), want_packed)

    wire = oq.params_over_the_wire(want_params)  # the receiver sees bf16-rounded parameters
    for p in (want_params, wire):
        want_back = oq.dequantize_segments(want_packed, p, splits, bits)
        back = torch.full((rows, feat), 9.0, device="cuda")
        ops.dequantize_tensor_for_all_procs(packed, back, dev(p), work_range.cuda(), len(splits), bits)
        assert np.array_equal(back.cpu().numpy().view(np.uint32), want_back.view(np.uint32))


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_whole_buffer_as_one_segment_and_ragged_tail(bits):
    from gnn_benchmark_amd.quantizer import QuantizerForPureBits

    epb = 8 // bits
    rng = np.random.default_rng(bits)
    for rows in (1, epb, epb + 1, 4 * epb - 1, 1001):
        x = _rows(rng, rows, 100)
        want_packed, want_params = oq.quantize_segments(x, [rows], bits)
        packed = torch.zeros(want_packed.shape, dtype=torch.uint8, device="cuda")
        assert packed.numel() == QuantizerForPureBits.get_quantized_buffer_size(rows, bits, 100)
        params = torch.zeros((rows, 2), device="cuda")
        QuantizerForPureBits.quantize_fp32_to_intX(dev(x), packed, params, bits)
        assert np.array_equal(packed.cpu().numpy(), want_packed)
        assert np.array_equal(params.cpu().numpy(), want_params)
        back = torch.zeros((rows, 100), device="cuda")
        QuantizerForPureBits.dequantize_intX_to_fp32(packed, back, params, bits)
        assert np.array_equal(back.cpu().numpy(), oq.dequantize_segments(want_packed, want_params, [rows], bits))


def test_committed_outputs_of_the_reference_kernels_bit_for_bit():
    """Row-packed cases: the reference's x86 kernel takes the parameters as inputs; they are
    the row's own min / range here, so the bytes must agree.  Mixed-bits cases as they are."""
    from gnn_benchmark_amd import computation_ops as ops

    z = np.load(GOLDEN)
    for c in range(int(z["rows_cases"])):
        x, bits = z[f"rows{c}_x"], int(z[f"rows{c}_bits"])
        packed = torch.zeros(z[f"rows{c}_packed"].shape, dtype=torch.uint8, device="cuda")
        params = torch.zeros((x.shape[0], 2), device="cuda")
        ops.quantize_tensor(dev(x), packed, params, bits)
        assert np.array_equal(params.cpu().numpy(), z[f"rows{c}_params"])
        assert np.array_equal(packed.cpu().numpy(), z[f"rows{c}_packed"]), c
        back = torch.zeros(x.shape, device="cuda")
        ops.dequantize_tensor(packed, back, params, bits)
        assert np.array_equal(back.cpu().numpy(), z[f"rows{c}_back"]), c
    for c in range(int(z["mixed_cases"])):
        x = z[f"mixed{c}_x"]
        params = torch.zeros((x.shape[0], 3), device="cuda")
        params[:, 0] = dev(z[f"mixed{c}_bits"])
        feat_range = dev(z[f"mixed{c}_range"])
        data = torch.zeros(int(z[f"mixed{c}_range"][-1]), dtype=torch.uint8, device="cuda")
        ops.quantize_tensor_v1(dev(x), data, feat_range, params)
        assert np.array_equal(data.cpu().numpy(), z[f"mixed{c}_data"]), c
        assert np.array_equal(params.cpu().numpy(), z[f"mixed{c}_params"]), c
        back = torch.zeros(x.shape, device="cuda")
        ops.dequantize_tensor_v1(data, back, feat_range, params)
        assert np.array_equal(back.cpu().numpy(), z[f"mixed{c}_back"]), c


def test_mixed_bits_golden_bytes_of_the_reference():
    """self_benchmark/a64fx/tests/test_quantizer.py:58-84 through the reference's class names."""
    from gnn_benchmark_amd.quantizer import QuantizerForMixedBits

    x = torch.tensor([[0.2, 0.1, 0.3], [0.4, 0.5, 0.6], [0.7, 0.8, 0.9], [1.0, 1.1, 1.2], [0.3, 0.1, 0.7]],
                     device="cuda")
    bits = torch.tensor([8, 4, 2, 4, 4], device="cuda")
    params = torch.empty((5, 3), device="cuda")
    params[:, 0] = bits
    feat_range = QuantizerForMixedBits.get_quantized_nodes_feat_range(5, 3, bits)
    assert feat_range.tolist() == [0, 3, 5, 6, 8, 10]
    data = torch.empty(int(feat_range[-1]), dtype=torch.uint8, device="cuda")
    QuantizerForMixedBits.quantize_fp32_to_intX(x, data, feat_range, params)
    assert data.tolist() == [127, 0, 255, 7, 240, 44, 8, 240, 80, 240]
    lo = x.min(dim=1)[0]
    assert torch.allclose(params[:, 1], lo) and torch.allclose(params[:, 2], (x.max(dim=1)[0] - lo) / (2.0 ** bits - 1))
    back = torch.empty_like(x)
    QuantizerForMixedBits.dequantize_intX_to_fp32(data, back, feat_range, params)
    assert bool(((back - x).abs() <= params[:, 2:3] * 0.5 + 1e-6).all())


def test_mixed_bits_wide_rows_match_oracle():
    from gnn_benchmark_amd import computation_ops as ops

    rng = np.random.default_rng(77)
    for rows, feat in ((300, 100), (64, 602), (17, 1)):
        x = _rows(rng, rows, feat)
        bits = rng.choice([2, 4, 8], rows).astype(np.float32)
        want_data, want_params = oq.quantize_mixed(x, bits)
        feat_range = oq.get_quantized_nodes_feat_range(rows, feat, bits)
        params = torch.zeros((rows, 3), device="cuda")
        params[:, 0] = dev(bits)
        data = torch.zeros(int(feat_range[-1]), dtype=torch.uint8, device="cuda")
        ops.quantize_tensor_v1(dev(x), data, dev(feat_range), params)
        assert np.array_equal(data.cpu().numpy(), want_data)
        assert np.array_equal(params.cpu().numpy(), want_params)
        back = torch.zeros((rows, feat), device="cuda")
        ops.dequantize_tensor_v1(data, back, dev(feat_range), params)
        assert np.array_equal(back.cpu().numpy(), oq.dequantize_mixed(want_data, want_params, feat))


def test_error_behaviour():
    from gnn_benchmark_amd import computation_ops as ops

    x = torch.zeros((8, 16), device="cuda")
    packed = torch.zeros((2, 16), dtype=torch.uint8, device="cuda")
    params = torch.zeros((8, 2), device="cuda")
    with pytest.raises(RuntimeError, match="bits"):
        ops.quantize_tensor(x, packed, params, 3)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.quantize_tensor(x.cpu(), packed, params, 2)
    with pytest.raises(RuntimeError, match="too small"):
        ops.quantize_tensor(x, packed[:1], params, 2)
    with pytest.raises(RuntimeError, match="work range"):
        ops.quantize_tensor_for_all_procs(x, packed, params, torch.tensor([0, 4, 7], dtype=torch.int32), 2, 2)
    p3 = torch.zeros((8, 3), device="cuda")
    p3[:, 0] = 3
    with pytest.raises(RuntimeError, match="bit width"):
        ops.quantize_tensor_v1(x, torch.zeros(64, dtype=torch.uint8, device="cuda"),
                               torch.arange(9, dtype=torch.int64, device="cuda") * 6, p3)
    # empty buffers are fine
    ops.quantize_tensor(x[:0], packed[:0], params[:0], 2)
    ops.dequantize_tensor(packed[:0], x[:0], params[:0], 2)


@pytest.mark.parametrize("rows,feat,bits", [(3_000_003, 128, 2), (9_000_001, 256, 4)])
def test_full_size_round_trip_properties(rows, feat, bits):
    """3 M boundary rows x 128 (config 4's receive buffer), and 9 M x 256 (element offsets past
    2^31): idempotence of the codec -- what was dequantised quantises back to the same bytes --
    and the half-step error bound."""
    from gnn_benchmark_amd import computation_ops as ops

    gen = torch.Generator(device="cuda").manual_seed(1)
    x = torch.randn(rows, feat, device="cuda", generator=gen)
    splits = [rows // 15] * 15
    splits[-1] += rows - sum(splits)
    splits.insert(3, 0)
    work_range = torch.tensor(np.concatenate(([0], np.cumsum(splits))), dtype=torch.int32)
    packed_rows = sum(-(-s // (8 // bits)) for s in splits)
    packed = torch.zeros((packed_rows, feat), dtype=torch.uint8, device="cuda")
    params = torch.zeros((rows, 2), device="cuda")
    ops.quantize_tensor_for_all_procs(x, packed, params, work_range, 16, bits)
    back = torch.empty_like(x)
    ops.dequantize_tensor_for_all_procs(packed, back, params, work_range, 16, bits)
    assert bool(((back - x).abs() <= params[:, 1:2] * 0.5 * (1 + 1e-5) + 1e-6).all())
    assert torch.equal(params[:, 0], x.min(dim=1)[0])
    packed2 = torch.zeros_like(packed)
    params2 = torch.zeros_like(params)
    ops.quantize_tensor_for_all_procs(back, packed2, params2, work_range, 16, bits)
    assert torch.equal(packed2, packed)
    # a sample of rows against the oracle
    sel = slice(splits[0] - 5, splits[0] + 9)  # straddles the first segment boundary
    xs = x[sel].cpu().numpy()
    want = oq.row_params(xs, bits)
    assert np.array_equal(params[sel].cpu().numpy(), want)


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("feat", [4, 48, 100, 128, 256, 600, 2052])
def test_aggregation_straight_from_packed_bytes_equals_dequantise_then_aggregate(bits, feat):
    """SPMM_forward_quantized / SPMM_backward_quantized against the two-step path, bit for bit, on a
    ragged matrix with long and empty rows and a boundary buffer cut into per-rank segments."""
    from gnn_benchmark_amd import SPMM_backward, SPMM_forward
    from gnn_benchmark_amd import computation_ops as ops
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits
    from gnn_benchmark_amd.sparse_tensor import SparseTensor
    from gnn_benchmark_amd.spmm_kernel import SPMM_backward_quantized, SPMM_forward_quantized
    from tests.gpu_util import skewed_csr

    rng = np.random.default_rng(100 * bits + feat)
    rows_a, halo = 700, 450
    rowptr, col, val = skewed_csr(rows_a, halo, seed=feat + bits)
    adj = SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(rows_a, halo), is_sorted=True)
    splits = [120, 0, 77, 253]                       # halo rows per peer rank
    cs = CommSplits(splits, [5, 5, 5, 5], 4, bits)
    qbuf = CommBufferForQuantization(cs, feat, bits, device="cuda")
    recv = dev(_rows(rng, halo, feat))
    ops.quantize_tensor_for_all_procs(recv, qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32,
                                      qbuf.dequantized_work_range_per_proc, 4, bits)
    deq = torch.empty_like(recv)
    ops.dequantize_tensor_for_all_procs(qbuf.quantized_recv_data_buf, deq, qbuf.quantized_recv_params_buf_fp32,
                                        qbuf.dequantized_work_range_per_proc, 4, bits)
    out0 = dev(rng.standard_normal((rows_a, feat)).astype(np.float32))
    want, got = out0.clone(), out0.clone()
    SPMM_forward(adj, deq, want)
    SPMM_forward_quantized(adj, qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32, qbuf.recv_row_code,
                           got, bits)
    assert torch.equal(got, want)
    want2, got2 = torch.empty_like(out0), torch.empty_like(out0)
    SPMM_forward(adj, deq, want2, accumulate=False)
    SPMM_forward_quantized(adj, qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32, qbuf.recv_row_code,
                           got2, bits, accumulate=False)
    assert torch.equal(got2, want2)
    # the same product looking each row's code up per gather (row codes not translated per element beforehand)
    from gnn_benchmark_amd.spmm_kernel import _spmm_quantized

    got2b = torch.empty_like(out0)
    _spmm_quantized(adj.get_plan(), adj.csr()[2], qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32,
                    qbuf.recv_row_code, got2b, bits, False, halo)
    assert torch.equal(got2b, want2)
    # transposed: the operand has one row per ROW of the matrix
    adj_t = SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(rows_a, halo), is_sorted=True)
    cs_t = CommSplits([1, 1, 1, 1], [300, 0, 399, 1], 4, bits)
    qt = CommBufferForQuantization(cs_t, feat, bits, device="cuda")
    send = dev(_rows(rng, rows_a, feat))
    ops.quantize_tensor_for_all_procs(send, qt.quantized_send_data_buf, qt.quantized_send_params_buf_fp32,
                                      qt.quantized_work_range_per_proc, 4, bits)
    deq_t = torch.empty_like(send)
    ops.dequantize_tensor_for_all_procs(qt.quantized_send_data_buf, deq_t, qt.quantized_send_params_buf_fp32,
                                        qt.quantized_work_range_per_proc, 4, bits)
    dx0 = dev(rng.standard_normal((halo, feat)).astype(np.float32))
    want3, got3 = dx0.clone(), dx0.clone()
    SPMM_backward(adj_t, deq_t, want3)
    SPMM_backward_quantized(adj_t, qt.quantized_send_data_buf, qt.quantized_send_params_buf_fp32, qt.send_row_code, got3,
                            bits)
    assert torch.equal(got3, want3)


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("feat", [4, 48, 64, 100, 128, 132, 256, 260, 512])
def test_product_with_quantised_result_rows_equals_product_then_quantise(bits, feat):
    """``spmm_quantize_for_all_procs`` (the pre-aggregation writing the packed bytes itself) against ``SPMM_forward``
    followed by ``quantize_tensor_for_all_procs``: bytes and parameters bit for bit -- ragged matrix with long rows
    (several index chunks) and empty rows, segments whose heights are no multiples of the rows a byte holds, an empty
    segment, a dense operand that is a column block of a wider array -- and against the oracle's bytes."""
    from gnn_benchmark_amd import SPMM_forward
    from gnn_benchmark_amd import computation_ops as ops
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits
    from gnn_benchmark_amd.sparse_tensor import SparseTensor
    from tests.gpu_util import skewed_csr

    rng = np.random.default_rng(1000 * bits + feat)
    send_rows, local = 703, 450
    rowptr, col, val = skewed_csr(send_rows, local, seed=feat + bits)
    adj = SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(send_rows, local), is_sorted=True)
    splits = [121, 0, 78, 504]
    cs = CommSplits([5, 5, 5, 5], splits, 4, bits)
    for strided in (False, True):
        wide = dev(_rows(rng, local, feat + 8))
        x = wide[:, 4:4 + feat] if strided else wide[:, :feat].contiguous()
        two = CommBufferForQuantization(cs, feat, bits, device="cuda")
        one = CommBufferForQuantization(cs, feat, bits, device="cuda")
        for q in (one, two):   # whatever neither path writes stays equal
            q.quantized_send_data_buf.fill_(0xAB)
            q.quantized_send_params_buf_fp32.fill_(-7.0)
        send = torch.empty(send_rows, feat, device="cuda")
        SPMM_forward(adj, x, send, accumulate=False)
        ops.quantize_tensor_for_all_procs(send, two.quantized_send_data_buf, two.quantized_send_params_buf_fp32,
                                          two.quantized_work_range_per_proc, 4, bits)
        rp, c, v = adj.csr()
        done = ops.spmm_quantize_for_all_procs(rp, c, v, x, one.quantized_send_data_buf,
                                               one.quantized_send_params_buf_fp32, one.quantized_work_range_per_proc, 4,
                                               bits)
        assert done
        assert torch.equal(one.quantized_send_params_buf_fp32, two.quantized_send_params_buf_fp32)
        assert torch.equal(one.quantized_send_data_buf, two.quantized_send_data_buf)
        o_bytes, o_params = oq.quantize_segments(send.cpu().numpy(), splits, bits)
        assert np.array_equal(one.quantized_send_data_buf.cpu().numpy().reshape(-1)[:o_bytes.size], o_bytes.reshape(-1))
        assert np.array_equal(one.quantized_send_params_buf_fp32.cpu().numpy(), o_params)


def test_product_with_quantised_result_rows_leaves_other_widths_to_the_two_calls():
    from gnn_benchmark_amd import computation_ops as ops
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits

    cs = CommSplits([1], [3], 1, 2)
    rp = torch.tensor([0, 1, 2, 2], device="cuda")
    c = torch.tensor([0, 1], device="cuda")
    v = torch.ones(2, device="cuda")
    for feat in (6, 516):
        q = CommBufferForQuantization(cs, feat, 2, device="cuda")
        before = q.quantized_send_data_buf.clone()
        assert not ops.spmm_quantize_for_all_procs(rp, c, v, torch.ones(2, feat, device="cuda"), q.quantized_send_data_buf,
                                                   q.quantized_send_params_buf_fp32, q.quantized_work_range_per_proc, 1, 2)
        assert torch.equal(q.quantized_send_data_buf, before)
    q = CommBufferForQuantization(cs, 8, 2, device="cuda")
    none = torch.zeros(0, dtype=torch.int64, device="cuda")   # a matrix without stored elements
    assert not ops.spmm_quantize_for_all_procs(torch.zeros(4, dtype=torch.int64, device="cuda"), none, v[:0],
                                               torch.ones(2, 8, device="cuda"), q.quantized_send_data_buf,
                                               q.quantized_send_params_buf_fp32, q.quantized_work_range_per_proc, 1, 2)
    with pytest.raises(RuntimeError, match="outside"):   # a column index beyond the dense operand's rows
        ops.spmm_quantize_for_all_procs(rp, torch.tensor([0, 2], device="cuda"), v, torch.ones(2, 8, device="cuda"),
                                        q.quantized_send_data_buf, q.quantized_send_params_buf_fp32,
                                        q.quantized_work_range_per_proc, 1, 2)


@pytest.mark.parametrize("bits", [2, 4, 8])
@pytest.mark.parametrize("feat", [1, 3, 16, 47, 128, 130, 256, 602, 1028, 2052])
def test_gather_folded_into_the_quantise_pass_equals_gather_then_quantise(bits, feat):
    """``gather_quantize_for_all_procs`` (raw boundary rows quantised as they are gathered) against
    ``src[index]`` followed by ``quantize_tensor_for_all_procs``: bytes and parameters bit for bit, repeated and
    unsorted indices, ragged segments, every width class of the quantise kernel."""
    from gnn_benchmark_amd import computation_ops as ops
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits

    rng = np.random.default_rng(10 * feat + bits)
    src = dev(_rows(rng, 333, feat))
    splits = [121, 0, 78, 504]
    index = torch.from_numpy(rng.integers(0, 333, sum(splits))).cuda()
    cs = CommSplits([5, 5, 5, 5], splits, 4, bits)
    one = CommBufferForQuantization(cs, feat, bits, device="cuda")
    two = CommBufferForQuantization(cs, feat, bits, device="cuda")
    for q in (one, two):
        q.quantized_send_data_buf.fill_(0xAB)
        q.quantized_send_params_buf_fp32.fill_(-7.0)
    ops.quantize_tensor_for_all_procs(src[index].contiguous(), two.quantized_send_data_buf,
                                      two.quantized_send_params_buf_fp32, two.quantized_work_range_per_proc, 4, bits)
    ops.gather_quantize_for_all_procs(src, index, one.quantized_send_data_buf, one.quantized_send_params_buf_fp32,
                                      one.quantized_work_range_per_proc, 4, bits)
    assert torch.equal(one.quantized_send_params_buf_fp32, two.quantized_send_params_buf_fp32)
    assert torch.equal(one.quantized_send_data_buf, two.quantized_send_data_buf)
    with pytest.raises(RuntimeError, match="outside"):
        bad = index.clone()
        bad[5] = 333
        ops.gather_quantize_for_all_procs(src, bad, one.quantized_send_data_buf, one.quantized_send_params_buf_fp32,
                                          one.quantized_work_range_per_proc, 4, bits)


def test_quantised_aggregation_error_behaviour():
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits
    from gnn_benchmark_amd.sparse_tensor import SparseTensor
    from gnn_benchmark_amd.spmm_kernel import SPMM_forward_quantized

    adj = SparseTensor(rowptr=torch.arange(9, device="cuda"), col=torch.arange(8, device="cuda"),
                       value=torch.ones(8, device="cuda"), sparse_sizes=(8, 8), is_sorted=True)
    q = CommBufferForQuantization(CommSplits([8], [8], 1, 2), 6, 2, device="cuda")
    out = torch.zeros(8, 6, device="cuda")
    with pytest.raises(RuntimeError, match="multiple of 4"):
        SPMM_forward_quantized(adj, q.quantized_recv_data_buf, q.quantized_recv_params_buf_fp32, q.recv_row_code, out, 2)
    q = CommBufferForQuantization(CommSplits([8], [8], 1, 2), 8, 2, device="cuda")
    out = torch.zeros(8, 8, device="cuda")
    with pytest.raises(RuntimeError, match="bits"):
        SPMM_forward_quantized(adj, q.quantized_recv_data_buf, q.quantized_recv_params_buf_fp32, q.recv_row_code, out, 3)
    with pytest.raises(RuntimeError, match="Input mismatch"):
        SPMM_forward_quantized(adj, q.quantized_recv_data_buf, q.quantized_recv_params_buf_fp32[:4], q.recv_row_code, out, 2)


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_reference_recipe_all_procs_against_per_segment_loop_and_torch(bits):
    """The reference's own check (tests/test_quantization_ops.py:128-151, :217-235): 256 rows x 233
    features cut into 256 random segments (most of them a row or two, many empty);
    quantize_tensor_for_all_procs must give the bytes of quantize_tensor run segment by segment,
    and the same values back.  For 8 and 4 bits it also compares with torch.quantize_per_channel
    (:23-35, :156-158), which rounds x * (1/scale) + zero_point instead of (x - min) / scale: equal
    but for ties and last-bit cases, so that comparison allows one step on a fraction of the values."""
    from gnn_benchmark_amd import computation_ops as ops

    num_nodes, feat_len, num_procs = 256, 233, 256
    gen = torch.Generator().manual_seed(bits)
    data = torch.randn((num_nodes, feat_len), generator=gen)
    work_range = torch.randint(0, num_nodes, (num_procs + 1,), generator=gen, dtype=torch.int32).sort()[0]
    work_range[0], work_range[-1] = 0, num_nodes
    per = 8 // bits
    sizes = [int(work_range[i + 1] - work_range[i]) for i in range(num_procs)]
    packed_rows = sum(-(-s // per) for s in sizes)
    x = data.cuda()

    packed = torch.zeros((packed_rows, feat_len), dtype=torch.uint8, device="cuda")
    params = torch.zeros((num_nodes, 2), device="cuda")
    ops.quantize_tensor_for_all_procs(x, packed, params, work_range, num_procs, bits)

    pieces, piece_params = [], []
    for i, s in enumerate(sizes):
        if s == 0:
            continue
        seg = x[int(work_range[i]):int(work_range[i + 1])].contiguous()
        out = torch.zeros((-(-s // per), feat_len), dtype=torch.uint8, device="cuda")
        prm = torch.zeros((s, 2), device="cuda")
        ops.quantize_tensor(seg, out, prm, bits)
        pieces.append(out)
        piece_params.append(prm)
    assert torch.equal(packed, torch.cat(pieces))
    assert torch.equal(params, torch.cat(piece_params))

    back = torch.zeros((num_nodes, feat_len), device="cuda")
    ops.dequantize_tensor_for_all_procs(packed, back, params, work_range, num_procs, bits)
    scale = params[:, 1:2]
    assert bool(((back - x).abs() <= scale * 0.5 * (1 + 1e-5) + 1e-6).all())

    if bits in (8, 4):
        s_cpu = ((data.max(dim=1)[0] - data.min(dim=1)[0] + 10e-20) / (2 ** bits - 1))
        zp_cpu = data.min(dim=1)[0] / s_cpu * (-1)
        ref = torch.dequantize(torch.quantize_per_channel(data, s_cpu, zp_cpu, 0,
                                                          torch.quint8 if bits == 8 else torch.quint4x2))
        diff = (back.cpu() - ref).abs()
        assert bool((diff <= s_cpu.view(-1, 1) * (1 + 1e-4) + 1e-6).all())
        assert float((diff > 1e-6 + 1e-5 * ref.abs()).float().mean()) < 0.02


@pytest.mark.parametrize("feat", [4, 48, 128, 256, 604])
@pytest.mark.parametrize("kind", ["bf16", 2, 8])
def test_one_launch_over_dense_rows_and_rows_in_their_exchange_format(kind, feat):
    """``SpmmPlan.spmm_dense_then``: a plan over [L | R], the first elements of every row gathering fp32 rows, the
    others bf16 rows or packed int2 / int8 rows -- bit-equal to the product with L followed by the product with R
    from the exchange format (accumulating and overwriting), for local parts that end before, at and behind the
    boundaries of the 32- / 64-element index chunks, rows with only local or only received elements and empty rows."""
    from gnn_benchmark_amd import SPMM_forward
    from gnn_benchmark_amd import computation_ops as ops
    from gnn_benchmark_amd.data_manager import CommBufferForQuantization, CommSplits
    from gnn_benchmark_amd.sparse_tensor import SparseTensor, side_by_side
    from gnn_benchmark_amd.spmm_kernel import SPMM_forward_quantized

    rng = np.random.default_rng(7 * feat + (0 if kind == "bf16" else kind))
    rows, local_cols, halo = 600, 500, 333

    def ragged(cols, lens):
        rowptr = np.concatenate(([0], np.cumsum(lens))).astype(np.int64)
        col = np.concatenate([np.sort(rng.integers(0, cols, n)) for n in lens] + [np.zeros(0, np.int64)]).astype(np.int64)
        val = rng.standard_normal(rowptr[-1]).astype(np.float32)
        return SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(rows, cols), is_sorted=True)

    len_l = rng.poisson(6, rows)
    len_r = rng.poisson(3, rows)
    edges = [0, 1, 7, 8, 9, 31, 32, 33, 63, 64, 65, 96, 127, 128, 129, 300]
    for i, n in enumerate(edges):       # local lengths around the chunk boundaries, with and without received elements
        len_l[3 * i], len_r[3 * i] = n, 5
        len_l[3 * i + 1], len_r[3 * i + 1] = n, 0
        len_l[3 * i + 2], len_r[3 * i + 2] = n, 70
    len_l[100:110], len_r[100:110] = 0, 0
    left, right = ragged(local_cols, len_l), ragged(halo, len_r)
    both = side_by_side(left, right)
    assert np.array_equal(both.first_counts.cpu().numpy(), len_l)
    x = dev(_rows(rng, local_cols, feat))
    recv = dev(_rows(rng, halo, feat))
    if kind == "bf16":
        second = recv.to(torch.bfloat16)

        def from_format(out):
            SPMM_forward(right, second, out)
    else:
        cs = CommSplits([100, 0, 33, 200], [5, 5, 5, 5], 4, kind)
        qbuf = CommBufferForQuantization(cs, feat, kind, device="cuda")
        ops.quantize_tensor_for_all_procs(recv, qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32,
                                          qbuf.dequantized_work_range_per_proc, 4, kind)
        second = (qbuf.quantized_recv_data_buf, qbuf.quantized_recv_params_buf_fp32, qbuf.recv_row_code, kind)

        def from_format(out):
            SPMM_forward_quantized(right, second[0], second[1], second[2], out, kind)
    out0 = dev(rng.standard_normal((rows, feat)).astype(np.float32))
    for accumulate in (True, False):
        want, got = out0.clone(), out0.clone()
        SPMM_forward(left, x, want, accumulate=accumulate)
        from_format(want)
        both.get_plan().spmm_dense_then(both.csr()[2], both.first_counts, x, second, got, accumulate)
        assert torch.equal(got, want), (kind, feat, accumulate)
    # operands that are column blocks of wider arrays
    wide_x = torch.zeros(local_cols, feat + 8, device="cuda")
    wide_x[:, 4:4 + feat] = x
    wide_out = torch.zeros(rows, 2 * feat, device="cuda")
    both.get_plan().spmm_dense_then(both.csr()[2], both.first_counts, wide_x[:, 4:4 + feat], second, wide_out[:, feat:], False)
    assert torch.equal(wide_out[:, feat:], want) and not wide_out[:, :feat].any()
    with pytest.raises(RuntimeError, match="Input mismatch"):
        both.get_plan().spmm_dense_then(both.csr()[2], both.first_counts[:-1], x, second, got, False)


@pytest.mark.parametrize("bits", [2, 4, 8])
def test_compiled_module_codec_functions_match_oracle_and_golden_bytes(bits):
    """The codec functions of the compiled pybind11 module ``computation_ops`` (gnn_benchmark_amd/ext), called with the
    reference's positional arguments (self_benchmark/a64fx/model/ops/src/quantization_arm.h; quantizer.py:18-90):
    the oracle's bytes and parameters for ragged segments, the whole-buffer form, and the mixed-width golden bytes of
    self_benchmark/a64fx/tests/test_quantizer.py:81."""
    from gnn_benchmark_amd import ext

    mod = ext.load()
    rng = np.random.default_rng(77 + bits)
    feat = 130
    splits = [5, 0, 13, 1, 8, 0, 4, 7]
    rows = sum(splits)
    x = _rows(rng, rows, feat)
    want_packed, want_params = oq.quantize_segments(x, splits, bits)
    work_range = torch.tensor(np.concatenate(([0], np.cumsum(splits))), dtype=torch.int32)
    packed = torch.full(want_packed.shape, 0xAB, dtype=torch.uint8, device="cuda")
    params = torch.full((rows, 2), -7.0, device="cuda")
    for _ in range(2):  # the second call finds the range's device copies again
        assert mod.quantize_tensor_for_all_procs(dev(x), packed, params, work_range, len(splits), bits) is None
    assert np.array_equal(params.cpu().numpy(), want_params) and np.array_equal(packed.cpu().numpy(), want_packed)
    back = torch.full((rows, feat), 9.0, device="cuda")
    mod.dequantize_tensor_for_all_procs(packed, back, params, work_range, len(splits), bits)
    want_back = oq.dequantize_segments(want_packed, want_params, splits, bits)
    assert np.array_equal(back.cpu().numpy().view(np.uint32), want_back.view(np.uint32))
    work_range[2] += 1  # changed in place: a new prefix, no stale copy
    work_range[2] -= 1
    mod.dequantize_tensor_for_all_procs(packed, back, params, work_range, len(splits), bits)
    assert np.array_equal(back.cpu().numpy().view(np.uint32), want_back.view(np.uint32))

    one_packed, one_params = oq.quantize_segments(x, [rows], bits)
    packed1 = torch.zeros(one_packed.shape, dtype=torch.uint8, device="cuda")
    params1 = torch.zeros((rows, 2), device="cuda")
    mod.quantize_tensor(dev(x), packed1, params1, bits)
    assert np.array_equal(packed1.cpu().numpy(), one_packed) and np.array_equal(params1.cpu().numpy(), one_params)
    back1 = torch.zeros((rows, feat), device="cuda")
    mod.dequantize_tensor(packed1, back1, params1, bits)
    assert np.array_equal(back1.cpu().numpy().view(np.uint32),
                          oq.dequantize_segments(one_packed, one_params, [rows], bits).view(np.uint32))

    with pytest.raises(RuntimeError, match="GPU"):
        mod.quantize_tensor(torch.zeros(4, 8), packed1, params1, bits)
    with pytest.raises(RuntimeError, match="bits"):
        mod.quantize_tensor(dev(x), packed1, params1, 3)
    with pytest.raises(RuntimeError, match="work range"):
        mod.quantize_tensor_for_all_procs(dev(x), packed, params, work_range[:-1], len(splits), bits)


def test_compiled_module_mixed_width_functions_on_the_reference_golden_bytes():
    from gnn_benchmark_amd import ext
    from gnn_benchmark_amd.quantizer import QuantizerForMixedBits

    mod = ext.load()
    x = torch.tensor([[0.2, 0.1, 0.3], [0.4, 0.5, 0.6], [0.7, 0.8, 0.9], [1.0, 1.1, 1.2], [0.3, 0.1, 0.7]],
                     device="cuda")
    bits = torch.tensor([8, 4, 2, 4, 4], device="cuda")
    params = torch.empty((5, 3), device="cuda")
    params[:, 0] = bits
    feat_range = QuantizerForMixedBits.get_quantized_nodes_feat_range(5, 3, bits)
    data = torch.empty(int(feat_range[-1]), dtype=torch.uint8, device="cuda")
    mod.quantize_tensor_v1(x, data, feat_range, params)
    assert data.tolist() == [127, 0, 255, 7, 240, 44, 8, 240, 80, 240]   # tests/test_quantizer.py:81
    back = torch.empty_like(x)
    mod.dequantize_tensor_v1(data, back, feat_range, params)
    assert bool(((back - x).abs() <= params[:, 2:3] * 0.5 + 1e-6).all())
    params[2, 0] = 3.0
    with pytest.raises(RuntimeError, match="bit width"):
        mod.quantize_tensor_v1(x, data, feat_range, params)
