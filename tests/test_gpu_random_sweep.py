"""Seeded random sweep over shapes the hand-picked cases do not name: every SpMM path
(plan, plan-less, transposed), the row-packed codec and the producers that write it themselves, bit for bit against the
oracle; packed and strided operands bit for bit against the dense / contiguous product; the fused LayerNorm pass against
torch's fp64 ops (5e-5 absolute on outputs, 2e-4 relative on gradients)."""
import numpy as np
import pytest
import torch

from gnn_benchmark_amd import SPMM_backward, SPMM_forward, gcn, packed
from gnn_benchmark_amd import computation_ops as ops
from gnn_benchmark_amd.sparse_tensor import SparseTensor
from oracle import quantization as oq
from oracle import spmm as ospmm

pytestmark = pytest.mark.gpu

WIDTHS = [1, 2, 3, 4, 5, 8, 12, 16, 31, 32, 33, 48, 64, 66, 100, 127, 128, 129, 172, 200, 256, 257, 300, 512, 513, 602,
          700, 1024, 1100]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _degrees(rng, rows):
    kind = int(rng.integers(0, 4))
    if kind == 0:
        deg = rng.poisson(rng.uniform(0.2, 12), rows)
    elif kind == 1:
        deg = (rng.pareto(1.2, rows) * 3).astype(np.int64)
    elif kind == 2:  # one very long row (block-per-row kernel above 2048)
        deg = rng.poisson(2, rows)
        deg[rng.integers(0, rows)] = int(rng.choice([300, 2000, 9000, 20000]))
    else:            # mostly empty
        deg = np.zeros(rows, np.int64)
        deg[rng.integers(0, rows, max(1, rows // 10))] = rng.integers(1, 50)
    return np.minimum(deg, 30000).astype(np.int64)


@pytest.mark.parametrize("seed", range(6))
def test_random_shapes_match_oracle_bit_for_bit(seed):
    rng = np.random.default_rng(9000 + seed)
    for case in range(25):
        rows = int(rng.choice([1, 2, 7, 63, 64, 65, 300, 1000, 5000]))
        cols = int(rng.choice([1, 3, 64, 500, 4000]))
        feat = int(rng.choice(WIDTHS))
        deg = _degrees(rng, rows)
        rowptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int64)
        nnz = int(rowptr[-1])
        col = rng.integers(0, cols, nnz).astype(np.int64)
        val = rng.standard_normal(nnz).astype(np.float32)
        x = rng.standard_normal((cols, feat)).astype(np.float32)
        out0 = rng.standard_normal((rows, feat)).astype(np.float32)
        g = rng.standard_normal((rows, feat)).astype(np.float32)
        dx0 = rng.standard_normal((cols, feat)).astype(np.float32)
        acc = bool(rng.integers(0, 2))
        what = dict(seed=seed, case=case, rows=rows, cols=cols, feat=feat, nnz=nnz, longest=int(deg.max()), acc=acc)

        want = ospmm.spmm(rowptr, col, val, x, out0.copy() if acc else np.zeros_like(out0))
        src = SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(rows, cols), is_sorted=True)
        got = dev(out0)
        SPMM_forward(src, dev(x), got, accumulate=acc)
        assert np.array_equal(got.cpu().numpy(), want), ("plan", what)
        got = dev(out0 if acc else np.zeros_like(out0))
        ops.spmm(dev(rowptr), dev(col), dev(val), dev(x), got, rows, None, None)
        assert np.array_equal(got.cpu().numpy(), want), ("plan-less", what)
        want_t = ospmm.spmm_transposed(rowptr, col, val, g, dx0.copy() if acc else np.zeros_like(dx0), cols)
        got = dev(dx0)
        SPMM_backward(src, dev(g), got, accumulate=acc)
        assert np.array_equal(got.cpu().numpy(), want_t), ("transposed", what)

        bits = int(rng.choice([2, 4, 8]))
        nseg = int(rng.integers(1, 9))
        splits = rng.multinomial(rows, np.ones(nseg) / nseg).tolist()
        xq = (rng.standard_normal((rows, feat)) * rng.uniform(1e-3, 1e3, (rows, 1))).astype(np.float32)
        want_packed, want_params = oq.quantize_segments(xq, splits, bits)
        work_range = torch.tensor(np.concatenate(([0], np.cumsum(splits))), dtype=torch.int32)
        packed = torch.zeros(want_packed.shape, dtype=torch.uint8, device="cuda")
        params = torch.zeros((rows, 2), device="cuda")
        ops.quantize_tensor_for_all_procs(dev(xq), packed, params, work_range, nseg, bits)
        assert np.array_equal(packed.cpu().numpy(), want_packed), ("packed bytes", what, bits, splits)
        assert np.array_equal(params.cpu().numpy(), want_params), ("parameters", what, bits, splits)
        wire = oq.params_over_the_wire(want_params)
        back = torch.zeros((rows, feat), device="cuda")
        ops.dequantize_tensor_for_all_procs(packed, back, dev(wire), work_range, nseg, bits)
        want_back = oq.dequantize_segments(want_packed, wire, splits, bits)
        assert np.array_equal(back.cpu().numpy().view(np.uint32), want_back.view(np.uint32)), ("dequantised", what, bits)


@pytest.mark.parametrize("seed", range(4))
def test_random_products_and_gathers_that_write_the_exchange_format(seed):
    """The pre-aggregation writing packed int2 / int4 / int8 rows itself and the gather folded into the quantise pass:
    bytes and parameters equal the oracle codec over the oracle product (over the gathered rows), bit for bit --
    ragged segments, empty and several-chunk rows, strided operands, every lane-group shape of the kernels."""
    rng = np.random.default_rng(7000 + seed)
    for case in range(20):
        bits = int(rng.choice([2, 4, 8]))
        feat = int(rng.choice([4, 8, 36, 64, 68, 100, 128, 132, 256, 260, 512]))
        rows = int(rng.choice([1, 2, 3, 5, 17, 64, 255, 1000]))
        cols = int(rng.choice([1, 7, 300, 5000]))
        kind = rng.random(rows)
        deg = np.where(kind < 0.2, 0, np.where(kind < 0.9, rng.integers(1, 12, rows), rng.integers(30, 300, rows)))
        rowptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int64)
        nnz = int(rowptr[-1])
        col = rng.integers(0, cols, nnz).astype(np.int64)
        val = rng.standard_normal(nnz).astype(np.float32)
        nseg = int(rng.choice([1, 2, 4, 9]))
        splits = np.diff(np.concatenate(([0], np.sort(rng.integers(0, rows + 1, nseg - 1)), [rows]))).tolist()
        work_range = torch.tensor(np.concatenate(([0], np.cumsum(splits))).astype(np.int32))
        wide = (rng.standard_normal((cols, feat + 8)) * rng.uniform(0.01, 30, (cols, 1))).astype(np.float32)
        strided = bool(rng.integers(0, 2))
        x_host = np.ascontiguousarray(wide[:, 4:4 + feat] if strided else wide[:, :feat])
        wide_d = dev(wide)
        x = wide_d[:, 4:4 + feat] if strided else wide_d[:, :feat].contiguous()
        what = dict(seed=seed, case=case, bits=bits, feat=feat, rows=rows, cols=cols, nnz=nnz, nseg=nseg, strided=strided)
        per = 8 // bits
        packed_rows = sum(-(-int(v) // per) for v in splits)
        if nnz:
            send = ospmm.spmm(rowptr, col, val, x_host, np.zeros((rows, feat), np.float32))
            o_bytes, o_params = oq.quantize_segments(send, splits, bits)
            got = torch.full((packed_rows, feat), 0xAB, dtype=torch.uint8, device="cuda")
            params = torch.full((rows, 2), -7.0, device="cuda")
            assert ops.spmm_quantize_for_all_procs(dev(rowptr), dev(col), dev(val), x, got, params, work_range, nseg, bits), what
            assert np.array_equal(got.cpu().numpy(), o_bytes), what
            assert np.array_equal(params.cpu().numpy().view(np.uint32), o_params.view(np.uint32)), what
        index = rng.integers(0, cols, rows).astype(np.int64)
        o_bytes, o_params = oq.quantize_segments(x_host[index], splits, bits)
        got = torch.full((packed_rows, feat), 0xAB, dtype=torch.uint8, device="cuda")
        params = torch.full((rows, 2), -7.0, device="cuda")
        ops.gather_quantize_for_all_procs(dev(x_host), dev(index), got, params, work_range, nseg, bits)
        assert np.array_equal(got.cpu().numpy(), o_bytes), what
        assert np.array_equal(params.cpu().numpy().view(np.uint32), o_params.view(np.uint32)), what


@pytest.mark.parametrize("seed", range(4))
def test_random_packed_operands_match_the_dense_product(seed):
    """Packed activations of random sparsity (all-zero and full rows included) through random
    matrices: the packed-source product equals the dense one bit for bit."""
    rng = np.random.default_rng(12000 + seed)
    for case in range(20):
        rows = int(rng.choice([1, 5, 64, 300, 2000]))
        cols = int(rng.choice([1, 3, 64, 500, 3000]))
        feat = int(rng.choice([32, 64, 128, 256]))
        deg = _degrees(rng, rows)
        rowptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int64)
        nnz = int(rowptr[-1])
        col = rng.integers(0, cols, nnz).astype(np.int64)
        val = rng.standard_normal(nnz).astype(np.float32)
        z = rng.standard_normal((cols, feat)).astype(np.float32)
        keep_p = float(rng.choice([0.0, 0.1, 0.5, 0.9, 1.0]))
        keep = (rng.random((cols, feat)) < keep_p)
        if cols > 2:
            z[0] = -1.0          # a row of zeros after the ReLU
            z[1] = 2.0           # a full row where kept
            keep[1] = True
        src = SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(rows, cols), is_sorted=True)
        bias = torch.zeros(feat, device="cuda")
        dense = gcn._BiasReluDropout.apply(dev(z), bias, dev(keep), 1.5, None)
        values, header = gcn._BiasReluDropoutPacked.apply(dev(z), bias, dev(keep), 1.5, None)
        assert torch.equal(packed.unpack(values, header), dense)
        acc = bool(rng.integers(0, 2))
        out0 = dev(rng.standard_normal((rows, feat)).astype(np.float32))
        want, got = out0.clone(), out0.clone()
        SPMM_forward(src, dense, want, accumulate=acc)
        packed.spmm(src, values, header, got, accumulate=acc)
        assert torch.equal(got, want), dict(seed=seed, case=case, rows=rows, cols=cols, feat=feat, keep=keep_p, acc=acc)


@pytest.mark.parametrize("seed", range(4))
def test_random_column_blocks_match_contiguous_operands(seed):
    """SpMM (both directions) and the weight gradient on column blocks of wider arrays at random
    offsets and strides: the same bits as on contiguous copies, nothing outside the block written."""
    rng = np.random.default_rng(15000 + seed)
    for case in range(20):
        rows = int(rng.choice([1, 7, 64, 300, 3000]))
        cols = int(rng.choice([1, 3, 64, 500, 3000]))
        feat = int(rng.choice(WIDTHS))
        deg = _degrees(rng, rows)
        rowptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int64)
        nnz = int(rowptr[-1])
        col = rng.integers(0, cols, nnz).astype(np.int64)
        val = rng.standard_normal(nnz).astype(np.float32)
        src = SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(rows, cols), is_sorted=True)
        lead_x, tail_x, lead_o, tail_o = (int(v) for v in rng.integers(0, 9, 4))
        wide_x = dev(rng.standard_normal((max(rows, cols), lead_x + feat + tail_x)).astype(np.float32))
        wide_o = dev(rng.standard_normal((max(rows, cols), lead_o + feat + tail_o)).astype(np.float32))
        acc = bool(rng.integers(0, 2))
        what = dict(seed=seed, case=case, rows=rows, cols=cols, feat=feat, longest=int(deg.max()), acc=acc,
                    offsets=(lead_x, tail_x, lead_o, tail_o))
        for op, n_in, n_out in ((SPMM_forward, cols, rows), (SPMM_backward, rows, cols)):
            x_view = wide_x[:n_in, lead_x:lead_x + feat]
            before = wide_o.clone()
            o_view = wide_o[:n_out, lead_o:lead_o + feat]
            want = o_view.contiguous()
            op(src, x_view.contiguous(), want, accumulate=acc)
            op(src, x_view, o_view, accumulate=acc)
            assert torch.equal(o_view, want), (op.__name__, what)
            untouched = torch.ones_like(wide_o, dtype=torch.bool)
            untouched[:n_out, lead_o:lead_o + feat] = False
            assert torch.equal(wide_o[untouched], before[untouched]), (op.__name__, what)
        fo = int(rng.choice([1, 5, 47, 64, 172, 256]))
        if feat <= 256:
            g = dev(rng.standard_normal((rows, fo + 3)).astype(np.float32))[:, 3:]
            x_view = wide_x[:rows, lead_x:lead_x + feat]
            assert torch.equal(gcn.weight_gradient(x_view, g),
                               gcn.weight_gradient(x_view.contiguous(), g.contiguous())), ("weight gradient", what, fo)


@pytest.mark.parametrize("seed", range(3))
def test_random_fused_layernorm_passes_match_torch(seed):
    from gnn_benchmark_amd import sage

    rng = np.random.default_rng(17000 + seed)
    for case in range(15):
        rows = int(rng.choice([1, 3, 64, 257, 4000]))
        feat = 4 * int(rng.integers(1, 257))
        z = dev((rng.standard_normal((rows, feat)) * rng.uniform(0.1, 10) + rng.uniform(-2, 2)).astype(np.float32))
        with_mask = bool(rng.integers(0, 2))
        p = float(rng.choice([0.1, 0.5, 0.8]))
        keep = dev(rng.random((rows, feat)) >= p) if with_mask else None
        scale = 1.0 / (1.0 - p) if with_mask else 1.0
        gamma = dev(rng.uniform(0.5, 1.5, feat).astype(np.float32))
        beta = dev(rng.uniform(-0.5, 0.5, feat).astype(np.float32))
        grad = dev(rng.standard_normal((rows, 2 * feat)).astype(np.float32))
        what = dict(seed=seed, case=case, rows=rows, feat=feat, mask=with_mask, p=p)

        z_ref = z.double().cpu().requires_grad_()
        g_ref, b_ref = gamma.double().cpu().requires_grad_(), beta.double().cpu().requires_grad_()
        d = z_ref * keep.cpu() * scale if with_mask else z_ref
        y_ref = torch.relu(torch.nn.functional.layer_norm(d, (feat,), g_ref, b_ref, 1e-5))
        y_ref.backward(grad[:, feat:].double().cpu())

        z_in, g_in, b_in = z.clone().requires_grad_(), gamma.clone().requires_grad_(), beta.clone().requires_grad_()
        cat = sage.dropout_layernorm_relu(z_in, keep, scale, g_in, b_in, 1e-5)
        cat.backward(grad)
        got = cat[:, feat:].detach().double().cpu()
        # a unit sits on the ReLU's edge when |n| is within rounding of 0: compare where fp64 is clear of it
        clear = (y_ref.detach() > 1e-4) | (torch.nn.functional.layer_norm(d, (feat,), g_ref, b_ref, 1e-5).detach() < -1e-4)
        assert float((got - y_ref.detach()).abs().max()) <= 5e-5, what
        gz_err = ((z_in.grad.double().cpu() - z_ref.grad).abs() * clear.all(dim=1, keepdim=True)).max()
        assert float(gz_err) <= 2e-4 * (float(z_ref.grad.abs().max()) + 1e-9), what
        if bool(clear.all()):
            for got_p, want_p in ((g_in.grad, g_ref.grad), (b_in.grad, b_ref.grad)):
                assert float((got_p.double().cpu() - want_p).abs().max()) <= 2e-4 * (float(want_p.abs().max()) + 1.0), what


@pytest.mark.parametrize("form", [gcn.FP32, gcn.BF16X3])
@pytest.mark.parametrize("seed", range(3))
def test_random_fused_layer_kernels_match_fp64(seed, form):
    """The one-kernel dense layer (product, degree division, bias, ReLU, dropout bits) and its one-pass
    gradient (mask, division, bias and weight gradients) over random row counts, widths, row strides and
    option sets, against fp64 torch ops on the units the kernel found active.  The bf16 x 3 form of the
    products (every fp32 operand as three bf16 pieces) is held to the same fp32 tolerances."""
    rng = np.random.default_rng(23000 + seed)
    for case in range(14):
        rows = int(rng.choice([1, 5, 127, 128, 129, 1000, 4097, 20011]))
        k = 16 * int(rng.integers(1, 17))
        n = int(rng.choice([32, 64, 128, 256])) if rng.random() < 0.4 else 4 * int(rng.integers(1, 65))
        pad = 4 * int(rng.integers(0, 3))
        wide = dev(rng.standard_normal((rows, k + 2 * pad)).astype(np.float32))
        x = wide[:, pad:pad + k]
        w = dev((rng.standard_normal((k, n)) / np.sqrt(k)).astype(np.float32))
        bias = dev(rng.standard_normal(n).astype(np.float32))
        with_div, with_mask, relu = (bool(v) for v in rng.integers(0, 2, 3))
        relu = relu or with_mask  # dropout comes behind a ReLU (the gradient reads the mask off the output)
        p = float(rng.choice([0.2, 0.5]))
        div = dev(rng.integers(1, 30, rows).astype(np.float32)) if with_div else None
        keep = dev(rng.random((rows, n)) >= p) if with_mask else None
        scale = 1.0 / (1.0 - p) if with_mask else 1.0
        g = dev(rng.standard_normal((rows, n)).astype(np.float32))
        what = dict(seed=seed, form=form, case=case, rows=rows, k=k, n=n, pad=pad, div=with_div, mask=with_mask, relu=relu)
        assert gcn.fused_layer_supported(x, k, n), what

        x_in, w_in, b_in = x.detach().clone().requires_grad_(), w.clone().requires_grad_(), bias.clone().requires_grad_()
        view = wide.clone()[:, pad:pad + k].requires_grad_() if pad else x_in
        y = gcn._FusedLayer.apply(gcn._kernel_ready(view), w_in, b_in, gcn.pack_keep_mask(keep) if with_mask else None,
                                  scale, div, relu, form)
        y.backward(g)
        z = x.double() @ w.double()
        if with_div:
            z = z / div.double().view(-1, 1)
        z = z + bias.double()
        ref = torch.relu(z) if relu else z
        if with_mask:
            ref = ref * keep * scale
        row_scale = (x.double().abs() @ w.double().abs() + bias.double().abs()).clamp(min=1.0) * scale
        assert bool(((y.double() - ref).abs() <= 1e-5 * row_scale).all()), what
        active = (y.detach() > 0).double() if relu else torch.ones_like(z)
        pre = g.double() * active * scale
        gz = pre / div.double().view(-1, 1) if with_div else pre
        for got, want, name in ((view.grad, gz @ w.double().t(), "x"), (w_in.grad, x.double().t() @ gz, "w"),
                                (b_in.grad, pre.sum(0), "bias")):
            size = float(want.abs().max()) + 1e-12
            assert float((got.double() - want).abs().max()) <= 2e-5 * size, (name, what)
        if relu and n in (32, 64, 128, 256):
            # the same layer writing its output packed: the same values bit for bit, and -- its gradient pass reading
            # the activity from the header's bitmaps -- the same gradients bit for bit
            x2, w2, b2 = x.detach().clone().requires_grad_(), w.clone().requires_grad_(), bias.clone().requires_grad_()
            values, header = gcn._FusedLayerPacked.apply(gcn._kernel_ready(x2), w2, b2,
                                                         gcn.pack_keep_mask(keep) if with_mask else None, scale, div, form)
            assert torch.equal(packed.unpack(values, header), y.detach()), what
            values.backward(g)
            for got, want, name in ((x2.grad, view.grad, "x"), (w2.grad, w_in.grad, "w"), (b2.grad, b_in.grad, "bias")):
                assert torch.equal(got, want), (name, what)
