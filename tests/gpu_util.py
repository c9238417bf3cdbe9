"""Helpers shared by the GPU parity tests (not collected by pytest)."""
import numpy as np
import scipy.sparse as sp
import torch

# fp32 tolerance of the parity gate: |got - want| <= ABS + REL * |want|
REL, ABS = 1e-5, 1e-6


def assert_close(got: torch.Tensor, want: np.ndarray, what: str = ""):
    got = got.detach().cpu().numpy().astype(np.float64)
    want = np.asarray(want, dtype=np.float64)
    err = np.abs(got - want) - (ABS + REL * np.abs(want))
    assert got.shape == want.shape, (what, got.shape, want.shape)
    assert err.max(initial=-1.0) <= 0.0, f"{what}: worst excess {err.max():.3e} at {np.unravel_index(err.argmax(), err.shape)}"


def assert_math_close(got: torch.Tensor, want_fp64: np.ndarray, what: str = ""):
    """Against an exact (fp64, differently associated) product: only fp32 rounding of sums
    with cancellation separates the two, so this is a looser, independent sanity bound --
    the parity gate proper is assert_close against the oracle."""
    got = got.detach().cpu().numpy().astype(np.float64)
    assert got.shape == want_fp64.shape, (what, got.shape, want_fp64.shape)
    assert np.allclose(got, want_fp64, rtol=1e-4, atol=1e-4), f"{what}: max abs diff {np.abs(got - want_fp64).max():.3e}"


def random_csr(rows, cols, density, seed, dtype=np.float32):
    a = sp.rand(rows, cols, density=density, format="csr", dtype=dtype, random_state=seed)
    a.sort_indices()
    return a


def skewed_csr(rows, cols, seed, heavy_rows=(2000, 900, 700), mean_deg=6, empty_every=7):
    """Ragged test matrix: a few very long rows, many short ones, some empty ones,
    repeated column indices allowed (as the reference's CSR build keeps them)."""
    rng = np.random.default_rng(seed)
    deg = rng.poisson(mean_deg, rows)
    deg[::empty_every] = 0
    for i, h in enumerate(heavy_rows):
        deg[(i * 37 + 3) % rows] = h
    rowptr = np.concatenate(([0], np.cumsum(deg))).astype(np.int64)
    col = rng.integers(0, cols, rowptr[-1]).astype(np.int64)
    for r in range(rows):
        col[rowptr[r]:rowptr[r + 1]].sort()
    val = rng.standard_normal(rowptr[-1]).astype(np.float32)
    return rowptr, col, val


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()
