"""Sort / unique / run-numbering steps of the index-map builders.  On GPU (HIP) tensors they run in libgnnagg's own
kernels (``csrc/sort.hip``: a stable radix sort and the run structure of a sorted list); on CPU tensors -- the host
tier that checks the builders against the reference's vectors -- as the torch host ops of the same meaning.  What the
reference does with ``torch.argsort`` / ``torch.unique`` followed by per-edge Python loops
(self_benchmark/a64fx/data_manager/DataProcessor.py:21, :39-53, :127, :238-246, :259, :306, :434-444)."""
import ctypes
from typing import Optional, Tuple

import torch

from .. import _lib


def _on_gpu(x: torch.Tensor) -> bool:
    return x.is_cuda and x.dtype == torch.int64 and x.dim() == 1


def _workspace(nbytes: int, device) -> torch.Tensor:
    """The kernels' temporaries, from torch's caching allocator (a call with no workspace allocates from the driver)."""
    return torch.empty(max(int(nbytes), 16), dtype=torch.uint8, device=device)


def stable_argsort(x: torch.Tensor) -> torch.Tensor:
    """Positions that put ``x`` in ascending order, equal values in their input order."""
    if not _on_gpu(x) or x.numel() == 0:
        return torch.sort(x, stable=True).indices
    x = x.contiguous()
    perm = torch.empty_like(x)
    L = _lib.lib()
    nbytes = int(L.gnnagg_argsort_workspace_bytes(x.numel()))
    workspace = _workspace(nbytes, x.device)
    with torch.cuda.device(x.device):
        _lib.check(L.gnnagg_argsort_i64(_lib.ptr(x), x.numel(), _lib.ptr(perm), None, _lib.ptr(workspace), nbytes,
                                        _lib.current_stream(x.device)))
    return perm


def runs(x: torch.Tensor, forced_starts: Optional[torch.Tensor] = None, want_values: bool = True,
         want_inverse: bool = True, want_counts: bool = True) -> Tuple[Optional[torch.Tensor], ...]:
    """(values, inverse, counts) of the runs of equal neighbours of ``x`` (``torch.unique_consecutive``); a run also
    starts at every position in ``forced_starts``.  Entries not asked for come back as None."""
    n = x.numel()
    if not _on_gpu(x) or n == 0:
        new = torch.ones(n, dtype=torch.bool, device=x.device)
        if n > 1:
            new[1:] = x[1:] != x[:-1]
        if forced_starts is not None and n:
            s = forced_starts.to(x.device)
            new[s[(s >= 0) & (s < n)]] = True
        inverse = torch.cumsum(new.to(torch.int64), 0) - 1
        starts = torch.nonzero(new).reshape(-1)
        ends = torch.cat([starts[1:], torch.tensor([n], dtype=torch.int64, device=x.device)]) if n else starts
        return (x[starts] if want_values else None, inverse if want_inverse else None,
                (ends - starts) if want_counts else None)
    x = x.contiguous()
    values = torch.empty_like(x) if want_values else None
    inverse = torch.empty_like(x) if want_inverse else None
    counts = torch.empty_like(x) if want_counts else None
    forced = None if forced_starts is None else forced_starts.to(device=x.device, dtype=torch.int64).contiguous()
    found = ctypes.c_int64(0)
    L = _lib.lib()
    nbytes = int(L.gnnagg_runs_workspace_bytes(n))
    workspace = _workspace(nbytes, x.device)
    with torch.cuda.device(x.device):
        _lib.check(L.gnnagg_runs_i64(_lib.ptr(x), n, _lib.ptr(forced), 0 if forced is None else forced.numel(),
                                     _lib.ptr(values), _lib.ptr(inverse), _lib.ptr(counts), ctypes.byref(found),
                                     _lib.ptr(workspace), nbytes, _lib.current_stream(x.device)))
    k = int(found.value)
    return (None if values is None else values[:k], inverse, None if counts is None else counts[:k])


def unique_sorted(x: torch.Tensor) -> torch.Tensor:
    """``torch.unique(x, sorted=True)``."""
    if not _on_gpu(x):
        return torch.unique(x, sorted=True)
    perm = stable_argsort(x)
    return runs(x[perm], want_inverse=False, want_counts=False)[0]


def occurrences_per_entry(x: torch.Tensor) -> torch.Tensor:
    """For every entry of ``x`` how often its value occurs in ``x``."""
    if not _on_gpu(x):
        _, inverse, counts = torch.unique(x, return_inverse=True, return_counts=True)
        return counts[inverse]
    perm = stable_argsort(x)
    _, inverse, counts = runs(x[perm], want_values=False)
    out = torch.empty_like(x)
    out[perm] = counts[inverse]
    return out
