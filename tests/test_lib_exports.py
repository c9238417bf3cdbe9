"""CPU-only: the C-ABI library loads and exports every entry point include/gnn_agg.h
declares; argument checks that need no GPU work are exercised (no compute calls)."""
import ctypes
import os
import re

import pytest

from gnn_benchmark_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    with open(os.path.join(ROOT, "include", "gnn_agg.h")) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(gnnagg_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared() == sorted(_lib.EXPORTS)


def _prototype_digest():
    """sha256 over every exported prototype of the header, comments and white space taken out."""
    import hashlib

    with open(os.path.join(ROOT, "include", "gnn_agg.h")) as f:
        text = f.read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    protos = re.findall(r"[A-Za-z_][A-Za-z0-9_ \*]*\bgnnagg_[a-z0-9_]+\s*\([^;{]*\)\s*;", text)
    assert len(protos) == len(_declared())
    canon = sorted(re.sub(r"\s+", " ", p).replace(" *", "*").replace("* ", "*").strip() for p in protos)
    return hashlib.sha256("\n".join(canon).encode()).hexdigest()[:16]


# GNNAGG_ABI_VERSION -> digest of the prototypes it stands for.  A changed, added or removed prototype changes the
# digest: raise GNNAGG_ABI_VERSION (header) and ABI_VERSION (_lib.py) together and record the new pair here, so that a
# library or extension module built from the old header is refused instead of being called with shifted arguments.
ABI_DIGESTS = {6: "d32bfa6402ead32b"}


def test_a_changed_prototype_needs_a_new_abi_version():
    with open(os.path.join(ROOT, "include", "gnn_agg.h")) as f:
        version = int(re.search(r"#define GNNAGG_ABI_VERSION (\d+)", f.read()).group(1))
    assert version == _lib.ABI_VERSION
    assert version in ABI_DIGESTS, "record the digest of the new ABI version in ABI_DIGESTS"
    assert _prototype_digest() == ABI_DIGESTS[version], (
        "an exported prototype changed: raise GNNAGG_ABI_VERSION / _lib.ABI_VERSION and record "
        f"{{{version + 1}: '{_prototype_digest()}'}}")


def test_library_exports_every_declared_symbol():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libgnnagg.so not built yet (python -c 'import __graft_entry__ as g; g.build()')")
    cdll = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(cdll, name), name
    assert _lib.lib().gnnagg_abi_version() == _lib.ABI_VERSION


def test_argument_errors_without_gpu_work():
    if not os.path.exists(_lib.LIB_PATH):
        pytest.skip("libgnnagg.so not built yet")
    L = _lib.lib()
    assert L.gnnagg_spmm_csr_f32(None, None, None, None, None, -1, 4, None) == _lib.ERR_INVALID
    assert b"negative" in L.gnnagg_last_error()
    assert L.gnnagg_spmm_csr_f32(None, None, None, None, None, 0, 4, None) == _lib.OK  # empty problem
    assert L.gnnagg_spmm_csr_f32(None, None, None, None, None, 3, 4, None) == _lib.ERR_INVALID
    assert L.gnnagg_plan_create(None, None, 1, 1, 0, None, None) == _lib.ERR_INVALID
    assert L.gnnagg_plan_destroy(None) == _lib.OK
    assert L.gnnagg_gather_rows_f32(None, 0, None, None, 0, 8, None) == _lib.OK
    with pytest.raises(_lib.GnnAggError):
        _lib.check(L.gnnagg_gather_rows_f32(None, 3, None, None, 5, 8, None))
    assert L.gnnagg_gather_rows_f32_bf16(None, 0, None, None, 0, 8, None) == _lib.OK
    assert L.gnnagg_gather_rows_f32_bf16(None, 3, None, None, 5, 8, None) == _lib.ERR_INVALID
    assert L.gnnagg_check_index(None, 8, 0, 0, 10, None) == _lib.OK
    assert L.gnnagg_check_index(None, 3, 5, 0, 10, None) == _lib.ERR_INVALID
    assert L.gnnagg_wgrad_f32(None, None, None, None, 0, 5, 8, 8, None) == _lib.ERR_INVALID   # null operands
    assert L.gnnagg_plan_create_ex(None, None, 1, 1, 0, None, None, None) == _lib.ERR_INVALID
    handle = ctypes.c_void_p()
    reserved = _lib.PlanOptions()
    reserved.reserved[1] = 7
    assert L.gnnagg_plan_create_ex(256, None, 1, 1, 0, ctypes.byref(reserved), None, ctypes.byref(handle)) == _lib.ERR_INVALID
    assert b"reserved" in L.gnnagg_last_error()
    # a null partial-sums workspace is refused on the host, not dereferenced on the device (fake non-null operands)
    assert L.gnnagg_dropout_layernorm_relu_backward_f32(256, 128, 256, None, 1.0, 256, 256, 1e-5, 256, None, 4, 128, None) == _lib.ERR_INVALID
    assert b"partial" in L.gnnagg_last_error()
    # the producers that write the exchange format themselves: argument checks before any launch (fake operands)
    fake = 256
    assert L.gnnagg_spmm_csr_quantize_segments_f32(fake, fake, fake, fake, 128, fake, fake, fake, fake, 1, 8, 2, 128, 3,
                                                   None) == _lib.ERR_INVALID
    assert b"bits" in L.gnnagg_last_error()
    assert L.gnnagg_spmm_csr_quantize_segments_f32(None, fake, fake, fake, 128, fake, fake, fake, fake, 1, 8, 2, 128, 2,
                                                   None) == _lib.ERR_INVALID   # null rowptr
    assert L.gnnagg_spmm_csr_quantize_segments_f32(fake, fake, fake, fake, 64, fake, fake, fake, fake, 1, 8, 2, 128, 2,
                                                   None) == _lib.ERR_INVALID   # row stride below the width
    assert L.gnnagg_spmm_csr_quantize_segments_f32(fake, fake, fake, fake, 516, fake, fake, fake, fake, 1, 8, 2, 516, 2,
                                                   None) == _lib.ERR_UNSUPPORTED   # wider than the kernel's rows
    assert L.gnnagg_spmm_csr_quantize_segments_f32(None, None, None, None, 0, None, None, None, None, 1, 0, 0, 128, 2,
                                                   None) == _lib.OK   # no rows
    assert L.gnnagg_gather_quantize_segments_f32(fake, 5, None, fake, fake, fake, fake, 1, 8, 2, 128, 2,
                                                 None) == _lib.ERR_INVALID   # null index
    assert L.gnnagg_gather_quantize_segments_f32(fake, 0, fake, fake, fake, fake, fake, 1, 8, 2, 128, 2,
                                                 None) == _lib.ERR_INVALID   # rows asked of an empty source


def test_product_refuses_cpu_tensors():
    import torch

    from gnn_benchmark_amd import SPMM_forward, SparseTensor, computation_ops

    rowptr = torch.tensor([0, 1, 2])
    col = torch.tensor([0, 1])
    val = torch.ones(2)
    x = torch.ones(2, 4)
    out = torch.zeros(2, 4)
    with pytest.raises(RuntimeError, match="GPU"):
        computation_ops.spmm(rowptr, col, val, x, out, 2, torch.empty(0, dtype=torch.int32), torch.tensor([0, 4], dtype=torch.int32))
    src = SparseTensor(rowptr=rowptr, col=col, value=val, sparse_sizes=(2, 2), is_sorted=True)
    with pytest.raises(RuntimeError, match="GPU"):
        SPMM_forward(src, x, out)
    assert torch.equal(out, torch.zeros(2, 4))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    """No fallback: with the shared library absent the binding raises, naming the file."""
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libgnnagg.so"))
    with pytest.raises(RuntimeError, match="libgnnagg.so is missing"):
        _lib.lib()


def test_compiled_extension_module_keeps_the_reference_signature():
    """``computation_ops.spmm`` as a compiled pybind11 module (self_benchmark/a64fx/model/ops/src/ops.cpp:23): eight
    positional arguments, value optional in the signature, ``(out, None)`` back; CPU tensors are refused before any
    GPU work."""
    import torch

    from gnn_benchmark_amd import ext

    try:
        mod = ext.load()
    except RuntimeError:
        pytest.skip("the extension module is not built yet (gnn_benchmark_amd/ext/build.sh)")
    assert mod.__name__ == "computation_ops"
    doc = mod.spmm.__doc__
    assert doc.count("torch.Tensor") >= 8 and "tuple[torch.Tensor, torch.Tensor | None]" in doc.replace("Optional[torch.Tensor]", "torch.Tensor | None")
    empty = torch.empty(0, dtype=torch.int32)
    args = (torch.tensor([0, 1]), torch.tensor([0]), torch.ones(1), torch.ones(1, 4), torch.zeros(1, 4), 1, empty, empty)
    with pytest.raises(RuntimeError, match="GPU"):
        mod.spmm(*args)
    with pytest.raises(TypeError):
        mod.spmm(*args[:7])
    # the codec functions the trainer's quantizer calls, with the positional arguments of
    # self_benchmark/a64fx/model/ops/src/quantization_arm.h (bound at model/ops/src/ops.cpp:12-18)
    for name, tensors in (("quantize_tensor", 3), ("dequantize_tensor", 3), ("quantize_tensor_v1", 4),
                          ("dequantize_tensor_v1", 4), ("quantize_tensor_for_all_procs", 4),
                          ("dequantize_tensor_for_all_procs", 4)):
        doc = getattr(mod, name).__doc__
        assert doc.count("torch.Tensor") == tensors and "-> None" in doc, doc
    with pytest.raises(RuntimeError, match="GPU"):
        mod.quantize_tensor(torch.ones(2, 4), torch.zeros(4, dtype=torch.uint8), torch.zeros(2, 2), 2)


def test_reference_build_and_drop_in_module_stay_apart_in_one_process(reference_op):
    """pybind11 keeps one module object per module name in a process, so the checker's build of the reference's
    module carries its own name: loaded in either order, it and the product's ``computation_ops`` are two modules
    (the reference's build binds the x86 flavour of the quantisation kernels, the drop-in the flavour the trainer's
    quantizer calls, and refuses CPU tensors; the tests of the oracle call the reference's ``spmm`` on CPU tensors in
    this same process)."""
    import torch

    from gnn_benchmark_amd import ext

    try:
        mod = ext.load()
    except RuntimeError:
        pytest.skip("the extension module is not built yet (gnn_benchmark_amd/ext/build.sh)")
    assert mod is not reference_op
    assert mod.__name__ == "computation_ops" and reference_op.__name__ == "reference_computation_ops"
    assert hasattr(reference_op, "quantize_tensor_v2_torch") and not hasattr(mod, "quantize_tensor_v2_torch")
    empty = torch.empty(0, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="GPU"):   # the drop-in has no CPU path (the reference's module computes)
        mod.spmm(torch.tensor([0, 1]), torch.tensor([0]), torch.ones(1), torch.ones(1, 4), torch.zeros(1, 4), 1, empty,
                 empty)
