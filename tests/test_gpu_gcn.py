"""The full train step (3-layer GCN around the aggregation path) on the GPU against an
independent CPU autograd run: same weights, same seeded dropout masks, same received halo
rows, aggregation done with torch.sparse.mm on the CPU.  The layer definition after the
aggregation is this build's own (no reference file holds it), so this is a consistency
check of forward, backward and the Adam update -- tolerance 1e-4 relative on the loss and
gradients (fp32 sums in a different order; bf16 variant: 2e-2)."""
import copy

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from gnn_benchmark_amd import gcn, synthetic

pytestmark = pytest.mark.gpu


class ReplayExchange:
    """Delivers the same seeded rows as SeededHaloExchange and keeps a host copy per tag."""

    def __init__(self, seed):
        self.inner = synthetic.SeededHaloExchange(seed)
        self.rows = {}

    def __call__(self, comm_splits, comm_buf, tag, direction):
        self.inner(comm_splits, comm_buf, tag, direction)
        buf = comm_buf.recv_buf if direction == "forward" else comm_buf.send_buf
        self.rows[tag] = buf.detach().cpu().clone()
        return None


def _torch_sparse(m):
    rowptr, col, val = [t.cpu() for t in m.csr()]
    return torch.sparse_csr_tensor(rowptr, col, val, size=m.sparse_sizes())


class CpuAggregate(torch.autograd.Function):
    """out = A_local x + A_from recv ; grad = A_local^T g + A_to^T incoming (CPU, torch.sparse)."""

    @staticmethod
    def forward(ctx, x, a_local, a_from, a_to, recv, incoming):
        ctx.mats = (a_local, a_to, incoming)
        return torch.sparse.mm(a_local, x) + torch.sparse.mm(a_from, recv)

    @staticmethod
    def backward(ctx, g):
        a_local, a_to, incoming = ctx.mats
        gx = torch.sparse.mm(a_local.t().to_sparse_csr(), g) + torch.sparse.mm(a_to.t().to_sparse_csr(), incoming)
        return gx, None, None, None, None, None


def _bf16_mm(a, b):
    return a.to(torch.bfloat16).float() @ b.to(torch.bfloat16).float()


class CpuBf16Linear(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w):
        ctx.save_for_backward(x, w)
        return _bf16_mm(x, w)

    @staticmethod
    def backward(ctx, g):
        x, w = ctx.saved_tensors
        return _bf16_mm(g, w.t()), _bf16_mm(x.t(), g)


# the small shape, and the widths of the full train-step workload (128 -> 256 -> 256 -> 172: the 256-wide
# fused layer instances, the 172-column last layer, aggregation at 128 and 256) on a partition the CPU run
# finishes in seconds: one of 16 ranks, 20 000 local nodes, 8 500 halo nodes, 57 000 remote edges
_SHAPES = {"small": (6000, [32, 64, 64, 12], (4, 2, 6, 1.8, 800, 1500, 9000)),
           "c5_widths": (20_000, [128, 256, 256, 172], (16, 3, 6.8, 1.8, 2000, 8500, 57_000))}


@pytest.mark.parametrize("gemm,tol,fuse", [("fp32", 1e-4, True), ("fp32", 1e-4, False), ("bf16", 2e-2, True),
                                           ("bf16", 2e-2, False), ("bf16x3", 1e-4, True), ("bf16x3", 1e-4, False)])
@pytest.mark.parametrize("linear_first", [False, True])
@pytest.mark.parametrize("shape", ["small", "c5_widths"])
def test_train_step_matches_cpu_autograd(gemm, tol, fuse, linear_first, shape):
    dev = "cuda:0"
    n, dims, part_args = _SHAPES[shape]
    part = synthetic.partition_edges(n, *part_args, seed=3, device=dev)
    ex = ReplayExchange(5)
    graph = synthetic.build_partition_graph(part, max(dims), True, exchange=ex, device=dev)
    torch.manual_seed(0)
    model = gcn.GCN(dims, gemm=gemm, linear_first_when_narrowing=linear_first).to(dev)
    assert [layer.linear_first for layer in model.layers] == [False, False, linear_first]  # only the last layer narrows
    for layer in model.layers:  # layers that aggregate first run through the fused kernels unless told not to
        layer.fuse = fuse
    cpu_model = copy.deepcopy(model).cpu()
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    gen = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    train_idx = torch.randperm(n, device=dev, generator=gen)[: n // 10]
    masks = gcn.make_dropout_masks(n, dims, 0.5, 7, dev)

    # forward + backward on the GPU (no update yet)
    model.train()
    hidden = []
    out = model(graph, x, True, masks, hidden=hidden)
    loss = F.nll_loss(out[train_idx], labels[train_idx])
    loss.backward()

    # independent CPU run with the rows the exchange delivered
    a_local, a_from, a_to = (_torch_sparse(m) for m in (graph.local_adj_t, graph.adj_t_pre_post_aggr_from,
                                                         graph.adj_t_pre_post_aggr_to))
    deg = graph.in_degrees.cpu()
    h = x.cpu()
    for l, layer in enumerate(cpu_model.layers):
        # layer 0's input needs no gradient, so its backward exchange never happens
        def product(t, layer=layer):
            return CpuBf16Linear.apply(t, layer.weight) if gemm == "bf16" else t @ layer.weight

        def aggregate(t, l=l):
            incoming = ex.rows.get(f"backward{l}", torch.zeros(a_to.shape[0], t.size(1)))
            return CpuAggregate.apply(t, a_local, a_from, a_to, ex.rows[f"forward{l}"], incoming)

        z = (aggregate(product(h)) if model.layers[l].linear_first else product(aggregate(h))) / deg + layer.bias
        if l == len(dims) - 2:
            h = z
            continue
        # Same values as the GPU's hidden layer.  A unit whose pre-activation lies within rounding of zero may be
        # active on one side and not on the other (millions of units: some always are); its value is ~0 either way,
        # but its gradient term is not, so the CPU run takes the GPU's set of active units for what follows.
        h_gpu = hidden[l].detach().cpu()
        h_cpu = torch.relu(z) * masks[l].cpu() * 2.0
        assert float((h_cpu.detach() - h_gpu).abs().max()) <= 10 * tol * float(h_gpu.abs().max()), l
        assert float(((h_cpu.detach() > 0) != (h_gpu > 0)).float().mean()) <= 1e-5, l
        h = z * (h_gpu > 0) * 2.0
    cpu_loss = F.nll_loss(F.log_softmax(h, dim=1)[train_idx.cpu()], labels.cpu()[train_idx.cpu()])
    cpu_loss.backward()

    assert abs(float(loss.detach()) - float(cpu_loss.detach())) <= tol * max(1.0, abs(float(cpu_loss.detach())))
    for (name, p_gpu), p_cpu in zip(model.named_parameters(), cpu_model.parameters()):
        scale = float(p_cpu.grad.abs().max()) + 1e-12
        assert float((p_gpu.grad.cpu() - p_cpu.grad).abs().max()) <= 10 * tol * scale, name

    # the full step: loss goes down over a few updates, every Adam update is bounded by lr
    before = [p.detach().clone() for p in model.parameters()]
    losses = [float(gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks)) for _ in range(5)]
    assert all(np.isfinite(losses))
    if not linear_first:  # (received rows are seeded noise; at the output width they reach the logits directly)
        assert losses[-1] < losses[0]
    assert abs(losses[0] - float(cpu_loss.detach())) <= tol * max(1.0, abs(float(cpu_loss.detach())))
    for b, p in zip(before, model.parameters()):
        assert float((p.detach() - b).abs().max()) <= 5 * 0.01 * 1.01


@pytest.mark.parametrize("gemm", ["fp32", "bf16", "bf16x3"])
@pytest.mark.parametrize("packed_activations,linear_first,fused_layers",
                         [(False, False, True), (True, False, True), (False, True, True), (False, False, False),
                          (True, True, False)])
def test_train_step_calls_no_library_product(gemm, packed_activations, linear_first, fused_layers, monkeypatch):
    """At the widths of the full train-step workload every dense product of the step -- layer products, weight
    gradients, input gradients (the last layer's inner width 172 included) -- runs in libgnnagg's kernels, in the
    default form and in the optional ones (the narrowing last layer multiplying first, the product kept apart from
    the elementwise passes): the step goes through with torch's matrix products taken away and the door to the BLAS
    library shut."""
    dev = "cuda:0"
    n, dims, part_args = _SHAPES["c5_widths"]
    part = synthetic.partition_edges(n, *part_args, seed=3, device=dev)
    graph = synthetic.build_partition_graph(part, max(dims), True, exchange=synthetic.SeededHaloExchange(5), device=dev)
    torch.manual_seed(0)
    model = gcn.GCN(dims, gemm=gemm, packed_activations=packed_activations,
                    linear_first_when_narrowing=linear_first, fused_layers=fused_layers).to(dev)
    opt = torch.optim.Adam(model.parameters(), lr=0.01)
    gen = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    train_idx = torch.randperm(n, device=dev, generator=gen)[: n // 10]
    masks = gcn.make_dropout_masks(n, dims, 0.5, 7, dev)
    want = float(gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks))

    def taken_away(*a, **k):
        raise AssertionError("a BLAS-library product inside the train step")

    for name in ("mm", "addmm", "matmul", "bmm", "baddbmm", "einsum"):
        monkeypatch.setattr(torch, name, taken_away)
    monkeypatch.setattr(torch.Tensor, "__matmul__", taken_away)
    monkeypatch.setattr(torch.nn.functional, "linear", taken_away)
    before = gcn.LIBRARY_PRODUCTS["count"]
    with gcn.forbid_library_products():
        for every_node in (False, True):
            loss = float(gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks,
                                        restrict_last_layer=not every_node))
            assert np.isfinite(loss) and abs(loss - want) < 0.5
    assert gcn.LIBRARY_PRODUCTS["count"] == before


def test_a_product_the_kernels_do_not_take_is_counted_or_refused():
    """Widths outside the product kernel (inner width no multiple of 16) go to the BLAS library through the one
    counted door, and raise under ``forbid_library_products()``."""
    a = torch.randn(100, 20, device="cuda")
    b = torch.randn(20, 24, device="cuda")
    before = gcn.LIBRARY_PRODUCTS["count"]
    y = gcn.plain_product(a, b, None, gcn.FP32)
    assert gcn.LIBRARY_PRODUCTS["count"] == before + 1
    assert torch.allclose(y, a @ b, rtol=1e-4, atol=1e-4)
    with gcn.forbid_library_products():
        with pytest.raises(RuntimeError, match="BLAS library"):
            gcn.plain_product(a, b, None, gcn.FP32)
    assert gcn.LIBRARY_PRODUCTS["forbidden"] is False


@pytest.mark.parametrize("num_bits", [2, 16])
@pytest.mark.parametrize("packed_activations", [False, True])
def test_train_step_with_narrow_boundary_rows(num_bits, packed_activations):
    """``GCN(num_bits=2 / 16)``: the boundary rows of every layer travel as int2 / bf16.  The products that write and
    read the exchange format themselves (the default) give, step after step, the losses and parameters of the
    reference's separate codec passes bit for bit; and the loss of the first step stays close to the fp32 exchange's
    (the stand-in delivers other rows, so only roughly)."""
    dev = "cuda:0"
    n, dims, part_args = _SHAPES["c5_widths"]
    part = synthetic.partition_edges(n, *part_args, seed=3, device=dev)
    gen = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    train_idx = torch.randperm(n, device=dev, generator=gen)[: n // 10]
    masks = gcn.make_dropout_masks(n, dims, 0.5, 7, dev)
    runs = []
    for fused in (True, False):
        graph = synthetic.build_partition_graph(part, max(dims), True, exchange=synthetic.SeededHaloExchange(5),
                                                bits=num_bits, exchange_quantized=synthetic.SeededQuantizedHaloExchange(9),
                                                exchange_bf16=synthetic.SeededBf16HaloExchange(9), device=dev)
        graph.fuse_quantize = graph.fuse_dequantize = graph.fuse_bf16_staging = fused
        torch.manual_seed(0)
        model = gcn.GCN(dims, packed_activations=packed_activations, num_bits=num_bits).to(dev)
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        losses = [float(gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks)) for _ in range(3)]
        hook = graph.exchange_quantized if num_bits == 2 else graph.exchange_bf16
        assert len(hook.calls) == 3 * 5 and not graph.exchange.calls  # 3 layers forward, 2 backward (layer 0 needs none)
        runs.append((losses, [p.detach().clone() for p in model.parameters()]))
    assert runs[0][0] == runs[1][0] and all(np.isfinite(runs[0][0]))
    for a, b in zip(runs[0][1], runs[1][1]):
        assert torch.equal(a, b)
    assert 4.0 < runs[0][0][0] < 7.0


@pytest.mark.parametrize("rows,feat", [(1000, 256), (333, 47), (64, 4), (1, 1)])
@pytest.mark.parametrize("with_mask", [True, False])
@pytest.mark.parametrize("with_div", [True, False])
def test_fused_epilogue_equals_separate_ops(rows, feat, with_mask, with_div):
    gen = torch.Generator(device="cuda").manual_seed(rows + feat)
    z = torch.randn(rows, feat, device="cuda", generator=gen)
    bias = torch.randn(feat, device="cuda", generator=gen)
    div = (torch.randint(1, 9, (rows, 1), device="cuda", generator=gen).float()) if with_div else None
    keep = (torch.rand(rows, feat, device="cuda", generator=gen) >= 0.5) if with_mask else None
    scale = 2.0 if with_mask else 1.0
    g = torch.randn(rows, feat, device="cuda", generator=gen)

    z_ref = z.clone().requires_grad_()
    b_ref = bias.clone().requires_grad_()
    y_ref = torch.relu((z_ref / div if with_div else z_ref) + b_ref)
    if with_mask:
        y_ref = y_ref * keep * scale
    y_ref.backward(g)

    z_in = z.clone().requires_grad_()
    b_in = bias.clone().requires_grad_()
    y = gcn._BiasReluDropout.apply(z_in * 1.0, b_in, keep, scale, div)  # * 1.0: a non-leaf the op may overwrite
    y.backward(g)
    assert torch.equal(y.detach(), y_ref.detach())
    assert torch.allclose(z_in.grad, z_ref.grad, rtol=2e-7, atol=0)  # (g*scale)/d vs g*(scale/d): last-bit rounding
    assert torch.allclose(b_in.grad, b_ref.grad, rtol=1e-5, atol=1e-5)  # column sums in another order


@pytest.mark.parametrize("rows,fi,fo", [(100_003, 256, 256), (65_536, 128, 256), (70_001, 256, 172), (999, 40, 47),
                                        (7, 1, 1), (128, 64, 64), (1, 256, 256), (513, 33, 250)])
def test_weight_gradient_kernel_matches_fp64(rows, fi, fo):
    """The hand-written MFMA product x^T @ g against an fp64 product: the error must stay
    within what fp32 accumulation over `rows` terms allows, and equal runs give equal bits."""
    gen = torch.Generator(device="cuda").manual_seed(rows + fi + fo)
    x = torch.randn(rows, fi, device="cuda", generator=gen)
    g = torch.randn(rows, fo, device="cuda", generator=gen)
    got = gcn.weight_gradient(x, g)
    want = x.double().t() @ g.double()
    bound = 4e-7 * (x.double().abs().t() @ g.double().abs())  # |error| <= c * eps * sum |x||g|
    assert got.shape == (fi, fo)
    assert bool(((got.double() - want).abs() <= bound + 1e-6).all()), float((got.double() - want).abs().max())
    assert torch.equal(got, gcn.weight_gradient(x, g))
    blas = x.t() @ g
    assert torch.allclose(got, blas, rtol=1e-4, atol=1e-3 * float(rows) ** 0.5)


def _unpack_bits(bits, feat):
    words = bits.cpu().numpy().view(np.uint32)
    cols = np.arange(feat)
    return ((words[:, cols // 32] >> (cols % 32).astype(np.uint32)) & 1).astype(bool)


@pytest.mark.parametrize("rows,feat", [(1000, 256), (333, 172), (65, 4), (7, 33), (1, 1), (0, 64)])
def test_keep_mask_bits_are_the_mask(rows, feat):
    gen = torch.Generator(device="cuda").manual_seed(rows + feat)
    keep = torch.rand(rows, feat, device="cuda", generator=gen) >= 0.5
    bits = gcn.pack_keep_mask(keep)
    assert bits.shape == (rows, (feat + 31) // 32) and bits.dtype == torch.int32
    if rows:
        assert np.array_equal(_unpack_bits(bits, feat), keep.cpu().numpy())
        # bits past the width are zero
        full = _unpack_bits(bits, 32 * bits.size(1))
        assert not full[:, feat:].any()
    assert torch.equal(bits, gcn.pack_keep_mask(keep.to(torch.uint8)))


@pytest.mark.parametrize("rows,k,n", [(1000, 64, 32), (777, 128, 172), (4099, 256, 256), (130, 16, 4), (1, 16, 8),
                                      (30_001, 128, 256), (513, 48, 100)])
@pytest.mark.parametrize("with_mask,with_div,relu", [(True, True, True), (False, True, False), (False, False, True),
                                                     (True, False, True)])
def test_fused_layer_equals_separate_ops(rows, k, n, with_mask, with_div, relu):
    """One-kernel layer (product, degree division, bias, ReLU, dropout) and its one-kernel gradient
    against the same chain in torch ops with fp64 products: forward within 1e-5 relative to the
    row's scale, the same units zeroed, gradients within 1e-5 of their scale; equal runs give equal bits."""
    gen = torch.Generator(device="cuda").manual_seed(rows + k + n)
    wide = torch.randn(rows, k + 8, device="cuda", generator=gen)
    x = wide[:, 4:4 + k]  # a column block of a wider array: rows 16-byte aligned, not contiguous
    w = (torch.randn(k, n, device="cuda", generator=gen) / k ** 0.5)
    bias = torch.randn(n, device="cuda", generator=gen)
    div = torch.randint(1, 9, (rows,), device="cuda", generator=gen).float() if with_div else None
    keep = (torch.rand(rows, n, device="cuda", generator=gen) >= 0.5) if with_mask else None
    bits = gcn.pack_keep_mask(keep) if with_mask else None
    scale = 2.0 if with_mask else 1.0
    g = torch.randn(rows, n, device="cuda", generator=gen)
    assert gcn.fused_layer_supported(x, k, n)

    z = x.double() @ w.double()
    if with_div:
        z = z / div.double().view(-1, 1)
    z = z + bias.double()
    ref = torch.relu(z) if relu else z
    if with_mask:
        ref = ref * keep * scale

    x_in, w_in, b_in = (t.detach().clone().requires_grad_() for t in (x, w, bias))
    x_view = gcn._kernel_ready(x_in)
    y = gcn._FusedLayer.apply(x_view, w_in, b_in, bits, scale, div, relu)
    y.backward(g)
    row_scale = (x.double().abs() @ w.double().abs() + bias.double().abs()).clamp(min=1.0) * scale
    assert bool(((y.double() - ref).abs() <= 1e-5 * row_scale).all())
    if with_mask:
        assert bool((y[~keep] == 0).all())
    # gradients in fp64 for the units the kernel found active (a pre-activation within rounding of zero
    # may fall either way; the forward check above bounds what that can change)
    active = (y.detach() > 0).double() if (relu or with_mask) else torch.ones_like(z)
    pre = g.double() * active * scale
    gz = pre / div.double().view(-1, 1) if with_div else pre
    for got, want, name in ((x_in.grad, gz @ w.double().t(), "x"), (w_in.grad, x.double().t() @ gz, "w"),
                            (b_in.grad, pre.sum(0), "bias")):
        size = float(want.abs().max()) + 1e-12
        assert float((got.double() - want).abs().max()) <= 1e-5 * size, name
    y2 = gcn._FusedLayer.apply(x_view.detach(), w, bias, bits, scale, div, relu)
    assert torch.equal(y.detach(), y2)


def test_fused_layer_rejects_unsupported_shapes():
    x = torch.randn(64, 20, device="cuda")
    assert not gcn.fused_layer_supported(x, 20, 32)      # contraction width not a multiple of 16
    assert not gcn.fused_layer_supported(x[:, :16], 16, 260)  # more than 256 outputs
    assert not gcn.fused_layer_supported(x[:, :16].cpu(), 16, 32)
    from gnn_benchmark_amd import _lib
    L = _lib.lib()
    y = torch.empty(64, 32, device="cuda")
    w = torch.randn(20, 32, device="cuda")
    rc = L.gnnagg_linear_bias_relu_dropout_f32(_lib.ptr(x), 20, _lib.ptr(w), 32, None, None, None, 1.0, 0, _lib.ptr(y), 32,
                                               64, 20, 32, _lib.current_stream(x.device))
    assert rc == _lib.ERR_UNSUPPORTED
    # packed output and the header-driven gradient pass exist for widths 32, 64, 128, 256 only
    x16, w100 = torch.randn(64, 16, device="cuda"), torch.randn(16, 100, device="cuda")
    vals, hdr = torch.empty(64 * 100 + 4, device="cuda"), torch.zeros(64, 8, dtype=torch.int32, device="cuda")
    rc = L.gnnagg_linear_bias_relu_dropout_pack_f32(_lib.ptr(x16), 16, _lib.ptr(w100), 100, None, None, None, 1.0,
                                                    _lib.ptr(vals), _lib.ptr(hdr), 64, 16, 100, 0,
                                                    _lib.current_stream(x.device))
    assert rc == _lib.ERR_UNSUPPORTED
    g100 = torch.randn(64, 100, device="cuda")
    nbytes = int(L.gnnagg_wgrad_relu_dropout_backward_workspace_bytes(64, 16, 100))
    ws = torch.empty(nbytes // 4, device="cuda")
    gw, gb = torch.empty(16, 100, device="cuda"), torch.empty(100, device="cuda")
    rc = L.gnnagg_wgrad_relu_dropout_backward_from_header_f32(_lib.ptr(x16), 16, _lib.ptr(g100), 100, _lib.ptr(hdr), None,
                                                              1.0, None, _lib.ptr(gw), _lib.ptr(gb), _lib.ptr(ws), nbytes,
                                                              64, 16, 100, 0, _lib.current_stream(x.device))
    assert rc == _lib.ERR_UNSUPPORTED
    # a workspace smaller than the kernels write into is refused before anything is launched
    xs, gs = torch.randn(5000, 64, device="cuda"), torch.randn(5000, 32, device="cuda")
    need = int(L.gnnagg_wgrad_workspace_bytes(5000, 64, 32))
    small = torch.empty(need // 4 - 1, device="cuda")
    out = torch.zeros(64, 32, device="cuda")
    rc = L.gnnagg_wgrad_f32(_lib.ptr(xs), _lib.ptr(gs), _lib.ptr(out), _lib.ptr(small), need - 4, 5000, 64, 32,
                            _lib.current_stream(x.device))
    assert rc == _lib.ERR_INVALID and b"workspace" in L.gnnagg_last_error()
    assert not out.any()
    with pytest.raises(RuntimeError, match="behind a ReLU"):
        gcn._FusedLayer.apply(x16, torch.randn(16, 32, device="cuda"), torch.zeros(32, device="cuda"),
                              torch.zeros(64, 1, dtype=torch.int32, device="cuda"), 2.0, None, False)


@pytest.mark.parametrize("rows,fi,fo", [(70_001, 256, 172), (999, 40, 48), (128, 64, 64), (1, 4, 4), (5000, 128, 256)])
def test_weight_and_bias_gradient_in_one_pass(rows, fi, fo):
    """x^T @ g and the column sums of g from one pass over g; x may be a column block of a wider array."""
    gen = torch.Generator(device="cuda").manual_seed(rows + fi + fo)
    wide = torch.randn(rows, 2 * fi, device="cuda", generator=gen)
    g = torch.randn(rows, fo, device="cuda", generator=gen)
    for x in (wide[:, :fi], wide[:, fi:]):
        gw, gb = gcn.weight_and_bias_gradient(x, g)
        assert torch.equal(gw, gcn.weight_gradient(x, g))  # the same MFMA chain
        want = g.double().sum(0)
        bound = 4e-7 * g.double().abs().sum(0) + 1e-6
        assert bool(((gb.double() - want).abs() <= bound).all())
        assert torch.equal(gb, gcn.weight_and_bias_gradient(x, g)[1])
    # a shape the kernel does not take falls back to torch ops
    x = torch.randn(64, 6, device="cuda", generator=gen)
    g6 = torch.randn(64, 6, device="cuda", generator=gen)
    gw, gb = gcn.weight_and_bias_gradient(x, g6)
    assert torch.allclose(gw, x.t() @ g6, rtol=1e-5, atol=1e-5) and torch.allclose(gb, g6.sum(0), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("rows,k,n", [(1000, 64, 32), (777, 128, 172), (4099, 256, 256), (130, 16, 4), (20_001, 128, 256)])
def test_fused_layer_with_bf16_inputs(rows, k, n):
    """The bf16-input form: operands rounded to bf16 (round to nearest even, as torch's .bfloat16()), exact
    products, fp32 accumulation -- within 1e-5 of the fp64 product of the rounded operands; the input
    gradient is the same kind of product of the masked gradient with w^T."""
    gen = torch.Generator(device="cuda").manual_seed(rows + k + n)
    x = torch.randn(rows, k, device="cuda", generator=gen)
    w = torch.randn(k, n, device="cuda", generator=gen) / k ** 0.5
    bias = torch.randn(n, device="cuda", generator=gen)
    div = torch.randint(1, 9, (rows,), device="cuda", generator=gen).float()
    keep = torch.rand(rows, n, device="cuda", generator=gen) >= 0.5
    g = torch.randn(rows, n, device="cuda", generator=gen)
    x_in, w_in, b_in = (t.detach().clone().requires_grad_() for t in (x, w, bias))
    y = gcn._FusedLayer.apply(x_in, w_in, b_in, gcn.pack_keep_mask(keep), 2.0, div, True, True)
    y.backward(g)
    xb, wb = x.bfloat16().double(), w.bfloat16().double()
    ref = torch.relu((xb @ wb) / div.double().view(-1, 1) + bias.double()) * keep * 2.0
    row_scale = (xb.abs() @ wb.abs() + bias.double().abs()).clamp(min=1.0) * 2.0
    assert bool(((y.double() - ref).abs() <= 1e-5 * row_scale).all())
    gz = g.double() * (y.detach() > 0) * 2.0 / div.double().view(-1, 1)
    want_x = gz.float().bfloat16().double() @ wb.t()          # the kernel rounds the fp32 masked gradient
    assert float((x_in.grad.double() - want_x).abs().max()) <= 1e-4 * (float(want_x.abs().max()) + 1e-12)
    want_w = xb.t() @ gz.float().bfloat16().double()          # ... and so does the weight gradient
    assert float((w_in.grad.double() - want_w).abs().max()) <= 1e-4 * (float(want_w.abs().max()) + 1e-12)
    want_b = (g.double() * (y.detach() > 0) * 2.0).sum(0)      # the bias gradient is summed in fp32
    assert float((b_in.grad.double() - want_b).abs().max()) <= 1e-5 * (float(want_b.abs().max()) + 1e-12)


@pytest.mark.parametrize("rows,k,n", [(1000, 64, 32), (777, 128, 172), (4099, 256, 256), (130, 16, 4), (2000, 1024, 128),
                                      (20_001, 128, 256)])
def test_product_in_three_bf16_pieces_is_as_exact_as_the_fp32_product(rows, k, n):
    """The bf16 x 3 form cuts every fp32 operand into hi + mid + lo bf16 pieces (the cuts are exact) and sums six
    bf16 MFMAs per product; what it leaves out is below 2^-24 |x||w| per term.  Rows spread over e^+-9 in size:
    per element the error stays within 1e-6 of sum |x||w| -- the bound the fp32 MFMA product meets, and three
    orders of magnitude under the bf16-input form's."""
    gen = torch.Generator(device="cuda").manual_seed(rows + k + n)
    x = torch.randn(rows, k, device="cuda", generator=gen) * torch.exp(3 * torch.randn(rows, 1, device="cuda", generator=gen))
    w = torch.randn(k, n, device="cuda", generator=gen) / k ** 0.5
    ref = x.double() @ w.double()
    size = x.double().abs() @ w.double().abs()
    errors = {}
    for name, form in (("fp32", gcn.FP32), ("bf16", gcn.BF16), ("bf16x3", gcn.BF16X3)):
        y = gcn._fused_product(x, w, None, None, None, 1.0, False, form)
        errors[name] = float(((y.double() - ref).abs() / size).max())
    assert errors["bf16x3"] <= 1e-6 and errors["fp32"] <= 1e-6, errors
    assert errors["bf16"] > 1e-4, errors  # (what rounding the operands to one bf16 piece costs)
    # an operand that one bf16 piece holds exactly goes through unchanged: integers below 256 times a power of two
    xi = torch.randint(-255, 256, (rows, k), device="cuda", generator=gen).float()
    wi = torch.randint(-255, 256, (k, n), device="cuda", generator=gen).float() / 64
    exact = xi.double() @ wi.double()  # every partial sum is an integer / 64 below 2^24: exact in fp32 too
    if k <= 128:
        assert torch.equal(gcn._fused_product(xi, wi, None, None, None, 1.0, False, gcn.BF16X3).double(), exact)


@pytest.mark.parametrize("fused", [True, False])
def test_degrees_folded_into_the_matrices_change_rounding_only(fused):
    """With the in-degree division carried by the matrix values (sage.fold_in_degrees) the layers skip their own
    division: the same model up to rounding (sum(a/d * x) against sum(a * x) / d)."""
    from gnn_benchmark_amd import sage

    dev = "cuda:0"
    n, dims = 5000, [32, 64, 64, 12]
    part = synthetic.partition_edges(n, 4, 2, 6, 1.8, 800, 1500, 9000, seed=4, device=dev)
    graph = synthetic.build_partition_graph(part, max(dims), True, exchange=synthetic.SeededHaloExchange(5), device=dev)
    folded = sage.fold_in_degrees(graph)
    torch.manual_seed(0)
    model = gcn.GCN(dims, fused_layers=fused).to(dev)
    gen = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    masks = gcn.make_dropout_masks(n, dims, 0.5, 7, dev)
    model.train()
    grads = []
    for g in (graph, folded):
        model.zero_grad(set_to_none=True)
        out = model(g, x, True, masks)
        F.nll_loss(out, labels).backward()
        grads.append([out.detach().clone()] + [p.grad.detach().clone() for p in model.parameters()])
    for a, b in zip(*grads):
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-6 + 1e-4 * float(a.abs().max()))


@pytest.mark.parametrize("bf16", [gcn.FP32, gcn.BF16, gcn.BF16X3])
def test_fused_layer_with_no_rows(bf16):
    """An empty partition: empty outputs, zero weight and bias gradients, nothing launched out of bounds."""
    x = torch.empty(0, 32, device="cuda", requires_grad=True)
    w = torch.randn(32, 64, device="cuda", requires_grad=True)
    b = torch.randn(64, device="cuda", requires_grad=True)
    y = gcn._FusedLayer.apply(x, w, b, None, 1.0, None, True, bf16)
    assert y.shape == (0, 64)
    y.backward(torch.empty(0, 64, device="cuda"))
    assert x.grad.shape == (0, 32) and not w.grad.any() and not b.grad.any()
    values, header = gcn._FusedLayerPacked.apply(x, w, b, None, 1.0, None, bf16)
    assert values.shape == (0, 64) and header.shape == (0, 4)


def _full_step(forward, opt, labels, train_idx):
    """The train step the long way round: every node through the last layer, the loss on the training rows."""
    opt.zero_grad(set_to_none=True)
    out = forward()
    loss = F.nll_loss(out[train_idx], labels[train_idx])
    loss.backward()
    opt.step()
    return loss.detach()


@pytest.mark.parametrize("model_kind", ["gcn", "gcn_separate_kernels", "gcn_linear_first", "gcn_packed", "gcn_bf16", "sage",
                                        "sage_linear_first"])
def test_scoring_only_the_training_rows_changes_nothing(model_kind):
    """A loss over the training rows needs only those rows of the last layer.  The train steps evaluate the last layer
    for the training rows only (``restrict_output_rows``: every row kept is the same FMA chain); where the last layer
    has no such form (a SAGE layer that multiplies first) they declare the zero rows of its gradient for the backward
    pass instead (``scored_rows``: every term skipped is a product with zero).  The gradients are those of the step
    that evaluates every node -- to the rounding of the last layer's dense products, which now sum the training rows
    only; bit for bit in the ``scored_rows`` case, where the same kernels run on the same rows."""
    from gnn_benchmark_amd import sage

    dev = "cuda:0"
    n, dims = 6000, [32, 64, 64, 12]
    part = synthetic.partition_edges(n, 4, 2, 6, 1.8, 800, 1500, 9000, seed=3, device=dev)
    gen = torch.Generator(device=dev).manual_seed(1)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    train_idx = torch.randperm(n, device=dev, generator=gen)[: n // 10]
    results = []
    for short_cut in (True, False):
        graph = synthetic.build_partition_graph(part, max(dims), True, exchange=synthetic.SeededHaloExchange(5), device=dev)
        torch.manual_seed(0)
        if model_kind.startswith("sage"):
            model = sage.DistSAGE(dims[0], dims[1], dims[-1], num_layers=3, dropout=0.5, is_pre_delay=True,
                                  linear_first_when_narrowing=(model_kind == "sage_linear_first")).to(dev)
            masks = sage.make_dropout_masks(n, dims[1], 3, 0.5, 8, dev)
            feats = sage.stage_input(x)
            quick = lambda: sage.train_step(model, opt, graph, feats, labels, train_idx, masks)
            full = lambda: _full_step(lambda: model(graph, feats, masks), opt, labels, train_idx)
        else:
            model = gcn.GCN(dims, gemm="bf16" if model_kind == "gcn_bf16" else "fp32",
                            linear_first_when_narrowing=(model_kind == "gcn_linear_first"),
                            packed_activations=(model_kind == "gcn_packed"),
                            fused_layers=(model_kind != "gcn_separate_kernels")).to(dev)
            masks = gcn.make_dropout_masks(n, dims, 0.5, 7, dev)
            quick = lambda: gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks)
            full = lambda: _full_step(lambda: model(graph, x, True, masks), opt, labels, train_idx)
        model.train()
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        losses = [float((quick if short_cut else full)())]
        results.append((losses, [p.grad.detach().clone() for p in model.parameters()]))
        assert getattr(graph, "backward_row_support", None) is None  # declared for the backward pass only
    assert np.allclose(results[0][0], results[1][0], rtol=1e-6)
    for a, b in zip(results[0][1], results[1][1]):
        if model_kind == "sage_linear_first":
            assert torch.equal(a, b)
        else:
            assert float((a - b).abs().max()) <= 1e-5 * float(b.abs().max()) + 1e-12


@pytest.mark.parametrize("model_kind", ["gcn", "sage"])
def test_train_step_can_send_every_node_through_the_last_layer(model_kind):
    """``restrict_last_layer=False`` is the reference's epoch (train.py:87-90): every node through every layer, the
    loss on the labelled rows.  The gradients of the weights are those of the step spelled out with torch's own
    ``nll_loss`` (the log-softmax of a row does not depend on which other rows are evaluated beside it)."""
    from gnn_benchmark_amd import sage

    dev = "cuda:0"
    n, dims = 5000, [32, 64, 64, 12]
    part = synthetic.partition_edges(n, 4, 2, 6, 1.8, 700, 1200, 8000, seed=4, device=dev)
    gen = torch.Generator(device=dev).manual_seed(2)
    x = torch.randn(n, dims[0], device=dev, generator=gen)
    labels = torch.randint(0, dims[-1], (n,), device=dev, generator=gen)
    train_idx = torch.randperm(n, device=dev, generator=gen)[: n // 8]
    results = []
    for own_step in (True, False):
        graph = synthetic.build_partition_graph(part, max(dims), True, exchange=synthetic.SeededHaloExchange(6), device=dev)
        torch.manual_seed(0)
        if model_kind == "sage":
            model = sage.DistSAGE(dims[0], dims[1], dims[-1], num_layers=3, dropout=0.5, is_pre_delay=True).to(dev)
            masks = sage.make_dropout_masks(n, dims[1], 3, 0.5, 8, dev)
            feats = sage.stage_input(x)
            step = lambda: sage.train_step(model, opt, graph, feats, labels, train_idx, masks, restrict_last_layer=False)
            full = lambda: _full_step(lambda: model(graph, feats, masks), opt, labels, train_idx)
        else:
            model = gcn.GCN(dims).to(dev)
            masks = gcn.make_dropout_masks(n, dims, 0.5, 7, dev)
            step = lambda: gcn.train_step(model, opt, graph, x, labels, train_idx, True, masks, restrict_last_layer=False)
            full = lambda: _full_step(lambda: model(graph, x, True, masks), opt, labels, train_idx)
        model.train()
        opt = torch.optim.Adam(model.parameters(), lr=0.01)
        loss = float((step if own_step else full)())
        results.append((loss, [p.grad.detach().clone() for p in model.parameters()]))
    assert np.isclose(results[0][0], results[1][0], rtol=1e-6)
    for a, b in zip(results[0][1], results[1][1]):
        assert float((a - b).abs().max()) <= 1e-5 * float(b.abs().max()) + 1e-12


@pytest.mark.parametrize("form", [gcn.FP32, gcn.BF16, gcn.BF16X3])
@pytest.mark.parametrize("rows,k,n", [(70_001, 48, 64), (66_000, 256, 256), (1, 16, 32), (129, 32, 128)])
def test_layer_kernels_walk_several_tiles_per_block(form, rows, k, n):
    """Rows beyond one tile per resident block (256 compute units x 128-row tiles = 32 768 rows, twice that for the
    kernels with two blocks per unit): every block walks several tiles, the chunk stream crosses tile boundaries, and
    K = 48 leaves a chunk count that is no multiple of the loading waves' unroll.  The dense result is checked against
    fp64 on the operands as the form sees them; the packed result must be the dense one bit for bit."""
    gen = torch.Generator(device="cuda").manual_seed(rows + k + n)
    x = torch.randn(rows, k, device="cuda", generator=gen)
    w = torch.randn(k, n, device="cuda", generator=gen) / k ** 0.5
    bias = torch.randn(n, device="cuda", generator=gen)
    div = torch.randint(1, 9, (rows,), device="cuda", generator=gen).float()
    keep = torch.rand(rows, n, device="cuda", generator=gen) >= 0.5
    bits = gcn.pack_keep_mask(keep)
    y = gcn._FusedLayer.apply(x, w, bias, bits, 2.0, div, True, form)
    xs, ws = (x.bfloat16().double(), w.bfloat16().double()) if form == gcn.BF16 else (x.double(), w.double())
    ref = torch.relu((xs @ ws) / div.double().view(-1, 1) + bias.double()) * keep * 2.0
    scale = (xs.abs() @ ws.abs() + bias.double().abs()).clamp(min=1.0) * 2.0
    assert bool(((y.double() - ref).abs() <= 1e-5 * scale).all())
    # the last rows and the first rows of the second round of tiles, where a wrong tile walk would show
    for r in {0, rows - 1, min(rows - 1, 32768), min(rows - 1, 65536)}:
        assert bool(((y[r].double() - ref[r]).abs() <= 1e-5 * scale[r]).all()), r
    values, header = gcn._FusedLayerPacked.apply(x, w, bias, bits, 2.0, div, form)
    from gnn_benchmark_amd import packed
    assert torch.equal(packed.unpack(values, header), y)
    # no bias, no mask, no divisor, no ReLU: the bare product (what the input-gradient product runs)
    bare = gcn._fused_product(x, w, None, None, None, 1.0, False, form)
    assert bool(((bare.double() - xs @ ws).abs() <= 1e-5 * (xs.abs() @ ws.abs()).clamp(min=1.0)).all())


@pytest.mark.parametrize("feat", [32, 64, 256, 172, 47, 1])
def test_keep_bits_are_the_mask_bytes_little_end_first(feat):
    """``gcn.pack_keep_mask``: bit q of word w of a row is mask byte 32 w + q (any non-zero byte counts); widths of
    whole words on a 16-byte boundary take the 16-byte-load kernel, others and unaligned views the byte one."""
    rng = np.random.default_rng(feat)
    rows = 1003
    keep = rng.integers(0, 2, (rows, feat)).astype(np.uint8) * rng.integers(1, 255, (rows, feat)).astype(np.uint8)
    words = (feat + 31) // 32
    padded = np.zeros((rows, words * 32), dtype=np.uint8)
    padded[:, :feat] = keep != 0
    want = np.packbits(padded.reshape(rows, words, 32), axis=2, bitorder="little").view(np.uint32).reshape(rows, words)
    got = gcn.pack_keep_mask(torch.from_numpy(keep).cuda())
    assert np.array_equal(got.cpu().numpy().view(np.uint32).reshape(rows, words), want)
    if feat % 32 == 0:  # the same rows one byte off the 16-byte boundary
        shifted = torch.empty(rows * feat + 1, dtype=torch.uint8, device="cuda")[1:].view(rows, feat)
        shifted.copy_(torch.from_numpy(keep))
        got = gcn.pack_keep_mask(shifted)
        assert np.array_equal(got.cpu().numpy().view(np.uint32).reshape(rows, words), want)
