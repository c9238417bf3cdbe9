"""The compute entry points neither allocate nor synchronise nor enqueue memsets, so a caller can
record them into a HIP graph (here through torch.cuda.CUDAGraph, whose capture stream the library
picks up as the current stream) and replay it.  One graph holds the plan SpMM with a very long row
(block-per-row kernel on the plan's side stream, forked and joined with events), the transposed
product, the strided product, the products with bf16 rows, the product with quantised result rows, the row gather (fp32
and bf16 rows), the codec, the bf16 conversions, both fused epilogues, the weight gradient, and the one-kernel dense layer with its one-pass gradient; it is replayed several times, with eager work and host
synchronisation in between, and every replay must reproduce the eager results bit for bit."""
import numpy as np
import pytest
import torch

from gnn_benchmark_amd import sparse_tensor

from gnn_benchmark_amd import SPMM_backward, SPMM_forward, gcn, sage
from gnn_benchmark_amd import computation_ops as ops
from gnn_benchmark_amd.aggregator import _convert, _gather_rows
from gnn_benchmark_amd.sparse_tensor import SparseTensor
from gpu_util import dev, skewed_csr

pytestmark = pytest.mark.gpu


def test_entry_points_replay_from_a_hip_graph(monkeypatch):
    monkeypatch.setattr(sparse_tensor, "PLAN_OPTIONS", {"block_row_threshold": 2048})
    n, feat, bits = 3000, 64, 2
    rowptr, col, val = skewed_csr(n, n, seed=3, heavy_rows=(5000, 900))
    src = SparseTensor(rowptr=dev(rowptr), col=dev(col), value=dev(val), sparse_sizes=(n, n))
    assert src.get_plan().info()["huge_rows"] == 1
    src.get_plan_for_transpose()                      # setup (allocates, synchronises) stays outside the graph
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = torch.randn(n, feat, device="cuda", generator=gen)
    keep = torch.rand(n, feat, device="cuda", generator=gen) >= 0.5
    gamma = torch.rand(feat, device="cuda", generator=gen) + 0.5
    beta = torch.randn(feat, device="cuda", generator=gen)
    bias = torch.randn(feat, device="cuda", generator=gen)
    index = torch.randint(0, n, (777,), device="cuda", generator=gen)
    weight = torch.randn(feat, feat, device="cuda", generator=gen) / 8
    keep_bits = gcn.pack_keep_mask(keep)
    div = torch.randint(1, 9, (n,), device="cuda", generator=gen).float()
    work_range = torch.tensor([0, 1000, 1000, n], dtype=torch.int32)
    packed_rows = sum(-(-s // (8 // bits)) for s in (1000, 0, n - 1000))
    csr_arrays = src.csr()

    def work():
        out = torch.empty(n, feat, device="cuda")
        SPMM_forward(src, x, out, accumulate=False)
        dx = torch.empty(n, feat, device="cuda")
        SPMM_backward(src, out, dx, accumulate=False)
        wide = torch.empty(n, 2 * feat, device="cuda")
        wide[:, feat:] = dx
        SPMM_forward(src, wide[:, feat:], wide[:, :feat], accumulate=False)          # strided, both halves of one array
        cat = sage._DropoutLayerNormRelu.apply(wide[:, :feat].contiguous(), keep, 2.0, gamma, beta, 1e-5)
        act = gcn._BiasReluDropout.apply(out * 1.0, bias, keep, 2.0, None)
        w = gcn.weight_gradient(x, cat[:, feat:])
        x_in, w_in, b_in = (t.detach().clone().requires_grad_() for t in (x, weight, bias))
        layer = gcn._FusedLayer.apply(x_in, w_in, b_in, keep_bits, 2.0, div, True)
        layer.backward(dx)
        x3, w3, b3 = (t.detach().clone().requires_grad_() for t in (x, weight, bias))
        layer3 = gcn._FusedLayer.apply(x3, w3, b3, keep_bits, 2.0, div, True, gcn.BF16X3)  # the bf16 x 3 product kernels
        layer3.backward(dx)
        rows = torch.empty(index.numel(), feat, device="cuda")
        _gather_rows(act, index, rows)
        packed = torch.empty((packed_rows, feat), dtype=torch.uint8, device="cuda")
        params = torch.empty((n, 2), device="cuda")
        ops.quantize_tensor_for_all_procs(dx, packed, params, work_range, 3, bits)
        back = torch.empty(n, feat, device="cuda")
        ops.dequantize_tensor_for_all_procs(packed, back, params, work_range, 3, bits)
        half = torch.empty(n, feat, dtype=torch.bfloat16, device="cuda")
        _convert(back, half)
        wire = torch.empty(n, feat, device="cuda")
        _convert(half, wire)
        rounded = torch.empty(n, feat, dtype=torch.bfloat16, device="cuda")
        SPMM_forward(src, x, rounded, accumulate=False)               # bf16 result rows (a 16-bit exchange's send side)
        widened = torch.empty(n, feat, device="cuda")
        SPMM_backward(src, rounded, widened, accumulate=False)        # bf16 operand rows (its receive side)
        rows16 = torch.empty(index.numel(), feat, dtype=torch.bfloat16, device="cuda")
        _gather_rows(act, index, rows16)                               # the gather storing bf16 rows
        packed1 = torch.empty((packed_rows, feat), dtype=torch.uint8, device="cuda")
        params1 = torch.empty((n, 2), device="cuda")
        assert ops.spmm_quantize_for_all_procs(csr_arrays[0], csr_arrays[1], csr_arrays[2], x, packed1, params1,
                                               work_range, 3, bits)  # a quantised exchange's send side in one pass
        # (the left half of `cat` is scratch for a following layer and is never written here)
        return [out, dx, wide, cat[:, feat:], act, w, rows, packed, params, back, wire, layer.detach(), x_in.grad,
                w_in.grad, b_in.grad, layer3.detach(), x3.grad, w3.grad, b3.grad, rounded, widened, rows16, packed1,
                params1]

    eager = [t.clone() for t in work()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                     # warm-up on a side stream, as graph capture asks for
        work()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        held = work()
    for replay in range(4):
        noise = torch.randn(512, 512, device="cuda")
        float((noise @ noise).sum())                  # the program's own eager work and a host synchronisation
        for t in held:
            t.zero_()
        graph.replay()
        torch.cuda.synchronize()
        for i, (got, want) in enumerate(zip(held, eager)):
            assert torch.equal(got, want), (replay, i)
