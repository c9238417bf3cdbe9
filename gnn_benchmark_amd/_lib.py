"""ctypes binding of ``csrc/libgnnagg.so`` (the C ABI declared in ``include/gnn_agg.h``).

There is no fallback: if the library has not been built, or a tensor is not on a HIP
device, the callers in this package raise.
"""
import ctypes
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_CSRC = os.path.join(_HERE, "csrc")
LIB_PATH = os.path.join(_CSRC, "libgnnagg.so")

OK, ERR_INVALID, ERR_HIP, ERR_UNSUPPORTED = 0, 1, 2, 3
ABI_VERSION = 6   # GNNAGG_ABI_VERSION of include/gnn_agg.h this binding was written against

EXPORTS = (
    "gnnagg_abi_version",
    "gnnagg_last_error",
    "gnnagg_spmm_csr_f32",
    "gnnagg_plan_create",
    "gnnagg_plan_create_ex",
    "gnnagg_plan_destroy",
    "gnnagg_plans_release",
    "gnnagg_plan_spmm_f32",
    "gnnagg_plan_spmm_strided_f32",
    "gnnagg_plan_spmm_two_sources_f32",
    "gnnagg_plan_spmm_dense_then_bf16_f32",
    "gnnagg_plan_spmm_dense_then_quantized_f32",
    "gnnagg_plan_info",
    "gnnagg_plan_profile",
    "gnnagg_plan_profile_read",
    "gnnagg_csr_transpose",
    "gnnagg_coo_to_csr",
    "gnnagg_argsort_workspace_bytes",
    "gnnagg_argsort_i64",
    "gnnagg_runs_workspace_bytes",
    "gnnagg_runs_i64",
    "gnnagg_gather_rows_f32",
    "gnnagg_gather_rows_f32_bf16",
    "gnnagg_check_index",
    "gnnagg_bias_relu_dropout_f32",
    "gnnagg_relu_dropout_backward_blocks",
    "gnnagg_relu_dropout_backward_f32",
    "gnnagg_wgrad_workspace_bytes",
    "gnnagg_wgrad_f32",
    "gnnagg_wgrad_strided_f32",
    "gnnagg_wgrad_noalloc_f32",
    "gnnagg_linear_shape_supported",
    "gnnagg_pack_keep_bits",
    "gnnagg_linear_bias_relu_dropout_f32",
    "gnnagg_linear_bias_relu_dropout_bf16_f32",
    "gnnagg_linear_bias_relu_dropout_bf16x3_f32",
    "gnnagg_linear_bias_relu_dropout_pack_f32",
    "gnnagg_wgrad_relu_dropout_backward_workspace_bytes",
    "gnnagg_wgrad_relu_dropout_backward_f32",
    "gnnagg_wgrad_relu_dropout_backward_bf16_f32",
    "gnnagg_wgrad_relu_dropout_backward_bf16x3_f32",
    "gnnagg_wgrad_relu_dropout_backward_from_header_f32",
    "gnnagg_dropout_layernorm_relu_blocks",
    "gnnagg_dropout_layernorm_relu_f32",
    "gnnagg_dropout_layernorm_relu_backward_f32",
    "gnnagg_packed_header_words",
    "gnnagg_bias_relu_dropout_pack_f32",
    "gnnagg_relu_dropout_backward_packed_f32",
    "gnnagg_plan_spmm_packed_f32",
    "gnnagg_quantize_segments_f32",
    "gnnagg_spmm_csr_quantize_segments_f32",
    "gnnagg_gather_quantize_segments_f32",
    "gnnagg_dequantize_segments_f32",
    "gnnagg_plan_spmm_quantized_f32",
    "gnnagg_plan_spmm_quantized_elements_f32",
    "gnnagg_plan_spmm_bf16_f32",
    "gnnagg_quantize_mixed_f32",
    "gnnagg_dequantize_mixed_f32",
    "gnnagg_f32_to_bf16",
    "gnnagg_bf16_to_f32",
)

_lib = None


class PlanOptions(ctypes.Structure):
    """``gnnagg_plan_options`` of include/gnn_agg.h (a field left 0: the library's default)."""
    _fields_ = [("long_row_threshold", ctypes.c_int32), ("block_row_threshold", ctypes.c_int32),
                ("rows_per_group", ctypes.c_int32), ("short_rows_per_group", ctypes.c_int32),
                ("lanes_per_row", ctypes.c_int32), ("loads_per_lane", ctypes.c_int32),
                ("reserved", ctypes.c_int32 * 2)]


class GnnAggError(RuntimeError):
    """A libgnnagg entry point returned an error code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libgnnagg error {code}: {message}")
        self.code = code


def build(verbose: bool = False) -> str:
    """Compile libgnnagg.so for gfx950 with hipcc (cross-compiles without a GPU)."""
    out = None if verbose else subprocess.DEVNULL
    subprocess.check_call(["make", "-C", _CSRC, "-B", "-j4", "libgnnagg.so"], stdout=out, stderr=out)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it first (python -c 'import __graft_entry__ as g; g.build()' "
            "or make -C gnn_benchmark_amd/csrc). There is no CPU fallback.")
    L = ctypes.CDLL(LIB_PATH)
    vp, i64, i32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int
    L.gnnagg_abi_version.restype = i32
    L.gnnagg_abi_version.argtypes = []
    built = L.gnnagg_abi_version()
    if built != ABI_VERSION:   # before any prototype is trusted: a stale library would be called with shifted arguments
        raise RuntimeError(f"{LIB_PATH} has ABI version {built}, this binding was written against {ABI_VERSION} "
                           "(include/gnn_agg.h changed since it was built): rebuild it (make -C gnn_benchmark_amd/csrc)")
    L.gnnagg_last_error.restype = ctypes.c_char_p
    L.gnnagg_last_error.argtypes = []
    L.gnnagg_spmm_csr_f32.restype = i32
    L.gnnagg_spmm_csr_f32.argtypes = [vp, vp, vp, vp, vp, i64, i64, vp]
    L.gnnagg_plan_create.restype = i32
    L.gnnagg_plan_create.argtypes = [vp, vp, i64, i64, i64, vp, ctypes.POINTER(vp)]
    L.gnnagg_plan_create_ex.restype = i32
    L.gnnagg_plan_create_ex.argtypes = [vp, vp, i64, i64, i64, ctypes.POINTER(PlanOptions), vp, ctypes.POINTER(vp)]
    L.gnnagg_plan_destroy.restype = i32
    L.gnnagg_plan_destroy.argtypes = [vp]
    L.gnnagg_plans_release.restype = i32
    L.gnnagg_plans_release.argtypes = []
    L.gnnagg_plan_spmm_f32.restype = i32
    L.gnnagg_plan_spmm_f32.argtypes = [vp, vp, vp, vp, i64, i32, vp]
    L.gnnagg_plan_spmm_strided_f32.restype = i32
    L.gnnagg_plan_spmm_strided_f32.argtypes = [vp, vp, vp, i64, vp, i64, i64, i32, vp]
    L.gnnagg_plan_spmm_two_sources_f32.restype = i32
    L.gnnagg_plan_spmm_two_sources_f32.argtypes = [vp, vp, vp, i64, i64, vp, i64, vp, i64, i64, i32, vp]
    L.gnnagg_plan_spmm_dense_then_bf16_f32.restype = i32
    L.gnnagg_plan_spmm_dense_then_bf16_f32.argtypes = [vp, vp, vp, vp, i64, i64, vp, i64, vp, i64, i64, i32, vp]
    L.gnnagg_plan_spmm_dense_then_quantized_f32.restype = i32
    L.gnnagg_plan_spmm_dense_then_quantized_f32.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp, vp, i32, vp, i64, i64, i32, vp]
    L.gnnagg_plan_info.restype = i32
    L.gnnagg_plan_info.argtypes = [vp, ctypes.POINTER(i64)]
    L.gnnagg_plan_profile.restype = i32
    L.gnnagg_plan_profile.argtypes = [vp, i32]
    L.gnnagg_plan_profile_read.restype = i32
    L.gnnagg_plan_profile_read.argtypes = [vp, ctypes.POINTER(ctypes.c_double)]
    L.gnnagg_csr_transpose.restype = i32
    L.gnnagg_csr_transpose.argtypes = [vp, vp, vp, i64, i64, i64, vp, vp, vp, vp]
    L.gnnagg_coo_to_csr.restype = i32
    L.gnnagg_coo_to_csr.argtypes = [vp, vp, vp, i64, i64, i64, vp, vp, vp, vp]
    L.gnnagg_argsort_i64.restype = i32
    L.gnnagg_argsort_i64.argtypes = [vp, i64, vp, vp, vp, i64, vp]
    L.gnnagg_runs_i64.restype = i32
    L.gnnagg_runs_i64.argtypes = [vp, i64, vp, i64, vp, vp, vp, ctypes.POINTER(i64), vp, i64, vp]
    for name in ("gnnagg_argsort_workspace_bytes", "gnnagg_runs_workspace_bytes"):
        getattr(L, name).restype = i64
        getattr(L, name).argtypes = [i64]
    L.gnnagg_gather_rows_f32.restype = i32
    L.gnnagg_gather_rows_f32.argtypes = [vp, i64, vp, vp, i64, i64, vp]
    L.gnnagg_gather_rows_f32_bf16.restype = i32
    L.gnnagg_gather_rows_f32_bf16.argtypes = [vp, i64, vp, vp, i64, i64, vp]
    L.gnnagg_check_index.restype = i32
    L.gnnagg_check_index.argtypes = [vp, i32, i64, i32, i64, vp]
    L.gnnagg_bias_relu_dropout_f32.restype = i32
    L.gnnagg_bias_relu_dropout_f32.argtypes = [vp, vp, vp, vp, ctypes.c_float, vp, i64, i64, vp]
    L.gnnagg_relu_dropout_backward_f32.restype = i32
    L.gnnagg_relu_dropout_backward_f32.argtypes = [vp, vp, vp, ctypes.c_float, vp, vp, i64, i64, vp]
    L.gnnagg_relu_dropout_backward_blocks.restype = i32
    L.gnnagg_relu_dropout_backward_blocks.argtypes = [i64, i64]
    L.gnnagg_wgrad_workspace_bytes.restype = i64
    L.gnnagg_wgrad_workspace_bytes.argtypes = [i64, i64, i64]
    L.gnnagg_wgrad_f32.restype = i32
    L.gnnagg_wgrad_f32.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, vp]
    L.gnnagg_f32_to_bf16.restype = i32
    L.gnnagg_f32_to_bf16.argtypes = [vp, vp, i64, vp]
    L.gnnagg_bf16_to_f32.restype = i32
    L.gnnagg_bf16_to_f32.argtypes = [vp, vp, i64, vp]
    L.gnnagg_wgrad_strided_f32.restype = i32
    L.gnnagg_wgrad_strided_f32.argtypes = [vp, i64, vp, i64, vp, vp, i64, i64, i64, i64, vp]
    L.gnnagg_wgrad_noalloc_f32.restype = i32
    L.gnnagg_wgrad_noalloc_f32.argtypes = [vp, vp, vp, i64, i64, i64, vp]
    L.gnnagg_linear_shape_supported.restype = i32
    L.gnnagg_linear_shape_supported.argtypes = [i64, i64]
    L.gnnagg_pack_keep_bits.restype = i32
    L.gnnagg_pack_keep_bits.argtypes = [vp, vp, i64, i64, vp]
    L.gnnagg_linear_bias_relu_dropout_f32.restype = i32
    L.gnnagg_linear_bias_relu_dropout_f32.argtypes = [vp, i64, vp, i64, vp, vp, vp, ctypes.c_float, i32, vp, i64, i64,
                                                      i64, i64, vp]
    L.gnnagg_linear_bias_relu_dropout_bf16_f32.restype = i32
    L.gnnagg_linear_bias_relu_dropout_bf16_f32.argtypes = L.gnnagg_linear_bias_relu_dropout_f32.argtypes
    L.gnnagg_linear_bias_relu_dropout_bf16x3_f32.restype = i32
    L.gnnagg_linear_bias_relu_dropout_bf16x3_f32.argtypes = L.gnnagg_linear_bias_relu_dropout_f32.argtypes
    L.gnnagg_linear_bias_relu_dropout_pack_f32.restype = i32
    L.gnnagg_linear_bias_relu_dropout_pack_f32.argtypes = [vp, i64, vp, i64, vp, vp, vp, ctypes.c_float, vp, vp, i64, i64,
                                                           i64, i32, vp]
    L.gnnagg_wgrad_relu_dropout_backward_workspace_bytes.restype = i64
    L.gnnagg_wgrad_relu_dropout_backward_workspace_bytes.argtypes = [i64, i64, i64]
    L.gnnagg_wgrad_relu_dropout_backward_f32.restype = i32
    L.gnnagg_wgrad_relu_dropout_backward_f32.argtypes = [vp, i64, vp, i64, vp, i64, vp, ctypes.c_float, vp, vp, vp, vp,
                                                         i64, i64, i64, i64, vp]
    L.gnnagg_wgrad_relu_dropout_backward_bf16_f32.restype = i32
    L.gnnagg_wgrad_relu_dropout_backward_bf16_f32.argtypes = L.gnnagg_wgrad_relu_dropout_backward_f32.argtypes
    L.gnnagg_wgrad_relu_dropout_backward_bf16x3_f32.restype = i32
    L.gnnagg_wgrad_relu_dropout_backward_bf16x3_f32.argtypes = L.gnnagg_wgrad_relu_dropout_backward_f32.argtypes
    L.gnnagg_wgrad_relu_dropout_backward_from_header_f32.restype = i32
    L.gnnagg_wgrad_relu_dropout_backward_from_header_f32.argtypes = [vp, i64, vp, i64, vp, vp, ctypes.c_float, vp, vp, vp,
                                                                     vp, i64, i64, i64, i64, i32, vp]
    L.gnnagg_dropout_layernorm_relu_blocks.restype = i32
    L.gnnagg_dropout_layernorm_relu_blocks.argtypes = [i64, i64]
    L.gnnagg_dropout_layernorm_relu_f32.restype = i32
    L.gnnagg_dropout_layernorm_relu_f32.argtypes = [vp, vp, ctypes.c_float, vp, vp, ctypes.c_float, vp, i64, i64, i64, vp]
    L.gnnagg_dropout_layernorm_relu_backward_f32.restype = i32
    L.gnnagg_dropout_layernorm_relu_backward_f32.argtypes = [vp, i64, vp, vp, ctypes.c_float, vp, vp, ctypes.c_float, vp, vp, i64, i64, vp]
    L.gnnagg_packed_header_words.restype = i32
    L.gnnagg_packed_header_words.argtypes = [i64]
    L.gnnagg_bias_relu_dropout_pack_f32.restype = i32
    L.gnnagg_bias_relu_dropout_pack_f32.argtypes = [vp, vp, vp, vp, ctypes.c_float, vp, vp, i64, i64, vp]
    L.gnnagg_relu_dropout_backward_packed_f32.restype = i32
    L.gnnagg_relu_dropout_backward_packed_f32.argtypes = [vp, vp, vp, ctypes.c_float, vp, vp, i64, i64, vp]
    L.gnnagg_plan_spmm_packed_f32.restype = i32
    L.gnnagg_plan_spmm_packed_f32.argtypes = [vp, vp, vp, vp, vp, i64, i32, vp]
    L.gnnagg_quantize_segments_f32.restype = i32
    L.gnnagg_quantize_segments_f32.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, vp]
    L.gnnagg_gather_quantize_segments_f32.restype = i32
    L.gnnagg_gather_quantize_segments_f32.argtypes = [vp, i64, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, vp]
    L.gnnagg_spmm_csr_quantize_segments_f32.restype = i32
    L.gnnagg_spmm_csr_quantize_segments_f32.argtypes = [vp, vp, vp, vp, i64, vp, vp, vp, vp, i64, i64, i64, i64, i32, vp]
    L.gnnagg_dequantize_segments_f32.restype = i32
    L.gnnagg_dequantize_segments_f32.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, vp]
    L.gnnagg_plan_spmm_quantized_f32.restype = i32
    L.gnnagg_plan_spmm_quantized_f32.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i32, i32, vp]
    L.gnnagg_plan_spmm_quantized_elements_f32.restype = i32
    L.gnnagg_plan_spmm_quantized_elements_f32.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i32, i32, vp]
    L.gnnagg_plan_spmm_bf16_f32.restype = i32
    L.gnnagg_plan_spmm_bf16_f32.argtypes = [vp, vp, vp, i32, i64, vp, i32, i64, i64, i32, vp]
    L.gnnagg_quantize_mixed_f32.restype = i32
    L.gnnagg_quantize_mixed_f32.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp]
    L.gnnagg_dequantize_mixed_f32.restype = i32
    L.gnnagg_dequantize_mixed_f32.argtypes = [vp, vp, vp, vp, i64, i64, vp, vp]
    _lib = L
    return L


def check(rc: int) -> None:
    if rc != OK:
        raise GnnAggError(rc, lib().gnnagg_last_error().decode("utf-8", "replace"))


def ptr(t):
    """Device address of a tensor (None -> NULL)."""
    return None if t is None else ctypes.c_void_p(t.data_ptr())


_CHECKED_INDEX = {}


def check_index(index, bound: int, shift: int = 0, what: str = "index") -> None:
    """Raise unless every ``index[i] >> shift`` lies in [0, bound).  The values are looked at on the device once per
    (tensor, bound, shift) -- one stream synchronisation -- and the verdict is remembered for as long as the same
    tensor, unchanged, comes back (an in-place change bumps ``_version``; a new tensor at a freed one's address fails
    the identity check).  The counterpart of the bounds checks torch's indexing ops make in the reference
    (``torch.index_select`` raises on a bad index, self_benchmark/a64fx/model/layers/aggregator.py:51)."""
    import weakref

    n = int(index.numel())
    if n == 0:
        return
    key = (index.data_ptr(), index._version, n, index.dtype, str(index.device), int(bound), int(shift))
    hit = _CHECKED_INDEX.get(key)
    if hit is not None and hit() is index:
        return
    if not index.is_contiguous():
        raise RuntimeError(f"Input mismatch: {what} must be contiguous")
    import torch

    with torch.cuda.device(index.device):
        rc = lib().gnnagg_check_index(ptr(index), index.element_size(), n, int(shift), int(bound),
                                      current_stream(index.device))
    if rc != OK:
        raise RuntimeError(f"Input mismatch: {what}: " + lib().gnnagg_last_error().decode("utf-8", "replace"))
    if len(_CHECKED_INDEX) >= 64:
        _CHECKED_INDEX.clear()
    _CHECKED_INDEX[key] = weakref.ref(index)


def current_stream(device):
    import torch

    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)
