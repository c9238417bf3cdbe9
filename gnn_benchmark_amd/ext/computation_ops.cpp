// The pybind11 module a maintainer of the reference trainer would build in place of its CPU operator module: same
// module name (`computation_ops`), same function name and the same eight positional arguments as
// `spmm_cpu_optimized_no_tile_v1` (self_benchmark/a64fx/model/ops/src/spmm.h:3-6, bound at
// model/ops/src/ops.cpp:23), same `(out, None)` return with `out` accumulated into in place -- but the tensors
// live on an MI355X and the work is one call into the C ABI of libgnnagg.so on the current HIP stream.
//
// This file is glue only: argument checks in the spirit of the reference's CHECK_INPUT (model/ops/src/utils.h:12-13,
// spmm.cpp:335-348), then `gnnagg_spmm_csr_f32`.  The two CPU thread-split tensors are accepted and ignored.
#include <torch/extension.h>

#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <stdexcept>
#include <string>
#include <tuple>

#include "gnn_agg.h"

namespace {

#define CHECK_HIP(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU (HIP) tensor; there is no CPU path")
#define CHECK_INPUT(x) TORCH_CHECK(x, "Input mismatch: " #x)

std::tuple<torch::Tensor, torch::optional<torch::Tensor>> spmm_mi355x(
    torch::Tensor rowptr, torch::Tensor col, torch::optional<torch::Tensor> optional_value, torch::Tensor mat,
    torch::Tensor out, int64_t sparse_rows, torch::Tensor /*parallel_row_split*/,
    torch::Tensor /*parallel_col_split*/) {
    CHECK_HIP(rowptr);
    CHECK_HIP(col);
    CHECK_HIP(mat);
    CHECK_HIP(out);
    // the reference dereferences the optional unconditionally (spmm.cpp:377); here a missing value is an error
    TORCH_CHECK(optional_value.has_value(), "Input mismatch: value is required");
    torch::Tensor value = optional_value.value();
    CHECK_HIP(value);
    const auto device = rowptr.device();
    TORCH_CHECK(col.device() == device && value.device() == device && mat.device() == device && out.device() == device,
                "Input mismatch: all operands must be on one device");
    CHECK_INPUT(rowptr.dim() == 1);
    CHECK_INPUT(col.dim() == 1);
    CHECK_INPUT(value.dim() == 1);
    CHECK_INPUT(value.size(0) == col.size(0));
    CHECK_INPUT(mat.dim() == 2);
    CHECK_INPUT(out.dim() == 2 && out.is_contiguous());
    CHECK_INPUT(rowptr.scalar_type() == torch::kInt64 && col.scalar_type() == torch::kInt64);
    // the reference prints a message and returns for other types (spmm.cpp:498-503); raising is the safer form
    CHECK_INPUT(mat.scalar_type() == torch::kFloat32 && value.scalar_type() == torch::kFloat32 &&
                out.scalar_type() == torch::kFloat32);
    CHECK_INPUT(sparse_rows >= 0 && rowptr.size(0) >= sparse_rows + 1);
    CHECK_INPUT(out.size(0) >= sparse_rows && out.size(1) == mat.size(1));
    mat = mat.contiguous();  // spmm.cpp:350
    rowptr = rowptr.contiguous();
    col = col.contiguous();
    value = value.contiguous();
    const auto stream = c10::hip::getCurrentHIPStream(device.index());
    c10::hip::HIPGuard guard(device.index());
    const int rc = gnnagg_spmm_csr_f32(rowptr.data_ptr<int64_t>(), col.data_ptr<int64_t>(), value.data_ptr<float>(),
                                       mat.data_ptr<float>(), out.data_ptr<float>(), sparse_rows, mat.size(1),
                                       stream.stream());
    TORCH_CHECK(rc == GNNAGG_OK, "libgnnagg error ", rc, ": ", gnnagg_last_error());
    return std::make_tuple(out, torch::optional<torch::Tensor>());  // spmm.cpp:505-506
}

}  // namespace

PYBIND11_MODULE(computation_ops, m) {
    // the library found at run time must be the one this module was compiled against: with another version of the
    // header its entry points may take other arguments
    if (gnnagg_abi_version() != GNNAGG_ABI_VERSION)
        throw std::runtime_error("computation_ops was compiled against libgnnagg ABI version " +
                                 std::to_string(GNNAGG_ABI_VERSION) + " but the library it loaded reports " +
                                 std::to_string(gnnagg_abi_version()) + ": rebuild both (gnn_benchmark_amd/ext/build.sh)");
    m.doc() = "MI355X drop-in for the reference's computation_ops.spmm (libgnnagg.so underneath)";
    m.def("spmm", &spmm_mi355x);
}
