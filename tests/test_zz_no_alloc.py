"""The weight-gradient entry point that allocates nothing (``gnnagg_wgrad_noalloc_f32``): its per-slice partial
results live in a device array built into the library instead of a caller's workspace.  Same kernels as
``gnnagg_wgrad_f32``, so the results must be equal bit for bit -- on two calls in a row, the second on a smaller
input (the array still holds the first call's partial results), and on a third that goes back up."""
import ctypes

import pytest
import torch

from gnn_benchmark_amd import _lib

pytestmark = pytest.mark.gpu


def _with_workspace(L, x, g):
    rows, fi = x.shape
    fo = g.shape[1]
    nbytes = L.gnnagg_wgrad_workspace_bytes(rows, fi, fo)
    assert nbytes > 0
    ws = torch.empty(nbytes // 4, dtype=torch.float32, device=x.device)
    out = torch.empty(fi, fo, dtype=torch.float32, device=x.device)
    _lib.check(L.gnnagg_wgrad_f32(_lib.ptr(x), _lib.ptr(g), _lib.ptr(out), _lib.ptr(ws), nbytes, rows, fi, fo,
                                  _lib.current_stream(x.device)))
    return out


def _no_alloc(L, x, g):
    rows, fi = x.shape
    fo = g.shape[1]
    out = torch.full((fi, fo), float("nan"), dtype=torch.float32, device=x.device)
    _lib.check(L.gnnagg_wgrad_noalloc_f32(_lib.ptr(x), _lib.ptr(g), _lib.ptr(out), rows, fi, fo,
                                          _lib.current_stream(x.device)))
    return out


def test_two_calls_in_a_row_equal_the_workspace_entry_point():
    L = _lib.lib()
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev).manual_seed(11)
    for rows, fi, fo in ((150_001, 256, 256), (4_097, 128, 172), (70_000, 256, 172), (37, 4, 8)):
        print(f"wgrad without allocation: rows={rows} fi={fi} fo={fo}", flush=True)
        x = torch.randn(rows, fi, device=dev, generator=gen)
        g = torch.randn(rows, fo, device=dev, generator=gen)
        want = _with_workspace(L, x, g)
        got = _no_alloc(L, x, g)
        torch.cuda.synchronize()
        assert torch.equal(got, want), (rows, fi, fo, (got - want).abs().max().item())
        ref = x.double().t() @ g.double()
        bound = 4e-7 * (x.double().abs().t() @ g.double().abs())
        assert bool(((got.double() - ref).abs() <= bound + 1e-30).all())


def test_empty_input_and_sizes_beyond_the_array():
    L = _lib.lib()
    dev = torch.device("cuda:0")
    x = torch.empty(0, 8, device=dev)
    g = torch.empty(0, 12, device=dev)
    got = _no_alloc(L, x, g)
    torch.cuda.synchronize()
    assert torch.equal(got, torch.zeros(8, 12, device=dev))
    x = torch.zeros(64, 512, device=dev)
    g = torch.zeros(64, 8, device=dev)
    out = torch.zeros(512, 8, device=dev)
    rc = L.gnnagg_wgrad_noalloc_f32(_lib.ptr(x), _lib.ptr(g), _lib.ptr(out), 64, 512, 8, ctypes.c_void_p(0))
    assert rc == _lib.ERR_UNSUPPORTED
    assert b"built-in scratch array" in L.gnnagg_last_error()
