"""The compiled drop-in for the reference's native module: ``load()`` returns the pybind11 module
``computation_ops`` built from ``computation_ops.cpp`` by ``build.sh`` (same module name, ``spmm`` with the
reference's eight positional arguments, self_benchmark/a64fx/model/ops/src/spmm.h:3-6, ops.cpp:23).

The package's own Python mirror (``gnn_benchmark_amd.computation_ops``) is what the rest of the package calls; this
module is the binding a maintainer of the reference would ship in place of the CPU operator module."""
import glob
import importlib.util
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_module = None
_DOC_PREFIX = "MI355X drop-in"   # how computation_ops.cpp documents the module


def build(verbose: bool = False) -> str:
    """Compile the module with g++ against the installed PyTorch-ROCm (libgnnagg.so must exist already)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call([os.path.join(_HERE, "build.sh")], stdout=out, stderr=out)
    return _path()


def _path():
    hits = glob.glob(os.path.join(_HERE, "computation_ops*.so"))
    return hits[0] if hits else None


def load():
    """The compiled ``computation_ops`` module; raises when it has not been built."""
    global _module
    if _module is None:
        path = _path()
        if path is None:
            raise RuntimeError(f"{_HERE}/computation_ops*.so is missing: build it first "
                               "(python -c 'import __graft_entry__ as g; g.build()' or gnn_benchmark_amd/ext/build.sh)")
        import torch  # noqa: F401  (the module links against libtorch)

        spec = importlib.util.spec_from_file_location("computation_ops", path)
        module = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(module)
        # pybind11 keeps one module object per module NAME in a process: had another pybind11 module called
        # `computation_ops` (the reference's CPU build, say) been imported first, its object would come back here
        if not (module.__doc__ or "").startswith(_DOC_PREFIX):
            raise RuntimeError("another compiled module named computation_ops is already loaded in this process; "
                               f"{path} cannot be loaded beside it")
        _module = module
    return _module
