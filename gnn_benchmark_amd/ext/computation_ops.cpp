// The pybind11 module a maintainer of the reference trainer would build in place of its CPU operator module: same
// module name (`computation_ops`), same function names and positional arguments as the module bound at
// self_benchmark/a64fx/model/ops/src/ops.cpp:11-24 -- `spmm` with the eight arguments of
// `spmm_cpu_optimized_no_tile_v1` (model/ops/src/spmm.h:3-6) and its `(out, None)` return with `out` accumulated into
// in place, and the six boundary-buffer codec functions the trainer's quantizer calls (quantizer.py:18,43,55,62,85,90;
// signatures of model/ops/src/quantization_arm.h) -- but the tensors live on an MI355X and the work is one call into
// the C ABI of libgnnagg.so on the current HIP stream.
//
// This file is glue only: argument checks in the spirit of the reference's CHECK_INPUT (model/ops/src/utils.h:12-13,
// spmm.cpp:335-348), then the C entry point.  The two CPU thread-split tensors of `spmm` are accepted and ignored.
#include <torch/extension.h>

#include <c10/hip/HIPGuard.h>
#include <c10/hip/HIPStream.h>

#include <map>
#include <mutex>
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


// ---------------------------------------------------------------------------------------------------------------
// Boundary-buffer codec.  A buffer's rows belong to `num_procs` peers, `work_range_per_proc` [num_procs + 1] is their
// prefix; every peer's segment is packed on its own, 8 / bits rows to a packed row (divide_work_v1,
// quantization_arm.cpp:21-31).  The kernels read the row prefix and the packed-row prefix from the device: both are
// derived once per range tensor and kept (the entry holds the range tensor, so its address cannot pass to another
// tensor meanwhile; a change in place shows in its version counter).
struct SegmentRanges {
    torch::Tensor range_kept, rows_prefix, packed_prefix;  // the last two int32 on the device
    int64_t rows = 0, packed_rows = 0;
};

const SegmentRanges &segment_ranges(const torch::Tensor &range, int64_t num_procs, int bits, const c10::Device &device) {
    using Key = std::tuple<const void *, int64_t, int64_t, int, int>;
    static std::map<Key, SegmentRanges> cache;
    static std::mutex guard;
    TORCH_CHECK(range.dim() == 1 && range.numel() == num_procs + 1 && num_procs >= 1,
                "Input mismatch: work range must hold num_procs + 1 entries");
    const Key key{range.data_ptr(), (int64_t)range._version(), range.numel(), bits, (int)device.index()};
    std::lock_guard<std::mutex> lock(guard);
    auto hit = cache.find(key);
    if (hit != cache.end()) return hit->second;
    const torch::Tensor host = range.detach().to(torch::kCPU, torch::kInt64).contiguous();
    const int64_t *h = host.data_ptr<int64_t>();
    TORCH_CHECK(h[0] == 0, "Input mismatch: work range must be a prefix sum from 0");
    const int64_t per_byte = 8 / bits;
    torch::Tensor rows32 = torch::empty({num_procs + 1}, torch::kInt32), packed32 = torch::empty({num_procs + 1}, torch::kInt32);
    int32_t *r = rows32.data_ptr<int32_t>(), *p = packed32.data_ptr<int32_t>();
    r[0] = p[0] = 0;
    int64_t packed = 0;
    for (int64_t i = 0; i < num_procs; ++i) {
        TORCH_CHECK(h[i + 1] >= h[i], "Input mismatch: work range must be a prefix sum from 0");
        TORCH_CHECK(h[i + 1] < (int64_t(1) << 31), "Input mismatch: more than 2^31-1 rows");
        packed += (h[i + 1] - h[i] + per_byte - 1) / per_byte;
        r[i + 1] = (int32_t)h[i + 1];
        p[i + 1] = (int32_t)packed;
    }
    if (cache.size() > 64) cache.clear();
    SegmentRanges made;
    made.range_kept = range;
    made.rows_prefix = rows32.to(device);
    made.packed_prefix = packed32.to(device);
    made.rows = h[num_procs];
    made.packed_rows = packed;
    return cache.emplace(key, std::move(made)).first->second;
}

c10::Device check_codec_operands(const torch::Tensor &fp32, const torch::Tensor &packed, const torch::Tensor &params, int bits,
                                 int64_t params_cols) {
    TORCH_CHECK(bits == 2 || bits == 4 || bits == 8, "Input mismatch: bits must be 2, 4 or 8");
    CHECK_HIP(fp32);
    CHECK_HIP(packed);
    CHECK_HIP(params);
    const auto device = fp32.device();
    TORCH_CHECK(packed.device() == device && params.device() == device, "Input mismatch: all operands must be on one device");
    TORCH_CHECK(fp32.scalar_type() == torch::kFloat32 && fp32.dim() == 2 && fp32.is_contiguous(),
                "Input mismatch: fp32 buffer must be contiguous float32 2-D");
    TORCH_CHECK(packed.scalar_type() == torch::kUInt8 && packed.is_contiguous(),
                "Input mismatch: packed buffer must be contiguous uint8");
    TORCH_CHECK(params.scalar_type() == torch::kFloat32 && params.is_contiguous() && params.dim() == 2 &&
                    params.size(0) >= fp32.size(0) && params.size(1) == params_cols,
                "Input mismatch: parameters must be contiguous float32 [rows, ", params_cols, "]");
    return device;
}

// quantization_arm.cpp:364-435: every peer's segment packed on its own; quantized_params [rows, 2] receives
// (zero_point, scale) per row.  The reference packs 2 bits whatever `bits` says (:380-381); here bits is honoured.
void quantize_tensor_for_all_procs(torch::Tensor input, torch::Tensor output, torch::Tensor quantized_params,
                                   torch::Tensor work_range_per_proc, int num_procs, int bits) {
    const auto device = check_codec_operands(input, output, quantized_params, bits, 2);
    const SegmentRanges &sr = segment_ranges(work_range_per_proc, num_procs, bits, device);
    TORCH_CHECK(sr.rows == input.size(0), "Input mismatch: work range does not cover the buffer's rows");
    TORCH_CHECK(output.numel() >= sr.packed_rows * input.size(1), "Input mismatch: packed buffer too small");
    const auto stream = c10::hip::getCurrentHIPStream(device.index());
    c10::hip::HIPGuard guard(device.index());
    const int rc = gnnagg_quantize_segments_f32(input.data_ptr<float>(), output.data_ptr<uint8_t>(),
                                                quantized_params.data_ptr<float>(), sr.rows_prefix.data_ptr<int32_t>(),
                                                sr.packed_prefix.data_ptr<int32_t>(), num_procs, sr.rows, sr.packed_rows,
                                                input.size(1), bits, stream.stream());
    TORCH_CHECK(rc == GNNAGG_OK, "libgnnagg error ", rc, ": ", gnnagg_last_error());
}

// quantization_arm.cpp:437-479: output = q * scale + zero_point with one rounding
void dequantize_tensor_for_all_procs(torch::Tensor input, torch::Tensor output, torch::Tensor dequantized_params,
                                     torch::Tensor work_range_per_proc, int num_procs, int bits) {
    const auto device = check_codec_operands(output, input, dequantized_params, bits, 2);
    const SegmentRanges &sr = segment_ranges(work_range_per_proc, num_procs, bits, device);
    TORCH_CHECK(sr.rows == output.size(0), "Input mismatch: work range does not cover the buffer's rows");
    TORCH_CHECK(input.numel() >= sr.packed_rows * output.size(1), "Input mismatch: packed buffer too small");
    const auto stream = c10::hip::getCurrentHIPStream(device.index());
    c10::hip::HIPGuard guard(device.index());
    const int rc = gnnagg_dequantize_segments_f32(input.data_ptr<uint8_t>(), dequantized_params.data_ptr<float>(),
                                                  output.data_ptr<float>(), sr.rows_prefix.data_ptr<int32_t>(),
                                                  sr.packed_prefix.data_ptr<int32_t>(), num_procs, sr.rows, sr.packed_rows,
                                                  output.size(1), bits, stream.stream());
    TORCH_CHECK(rc == GNNAGG_OK, "libgnnagg error ", rc, ": ", gnnagg_last_error());
}

// the [0, rows] range of a buffer that is one segment: one tensor per height, so that its device copies are found again
torch::Tensor one_segment(int64_t rows) {
    static std::map<int64_t, torch::Tensor> kept;
    static std::mutex guard;
    std::lock_guard<std::mutex> lock(guard);
    auto hit = kept.find(rows);
    if (hit != kept.end()) return hit->second;
    if (kept.size() >= 16) kept.clear();
    torch::Tensor range = torch::empty({2}, torch::kInt64);
    range.data_ptr<int64_t>()[0] = 0;
    range.data_ptr<int64_t>()[1] = rows;
    return kept.emplace(rows, range).first->second;
}

// quantization_arm.cpp:302-331 / :333-362: the whole buffer as one segment
void quantize_tensor(torch::Tensor input, torch::Tensor output, torch::Tensor quantized_params, int bits) {
    TORCH_CHECK(input.dim() == 2, "Input mismatch: fp32 buffer must be contiguous float32 2-D");
    quantize_tensor_for_all_procs(input, output, quantized_params, one_segment(input.size(0)), 1, bits);
}

void dequantize_tensor(torch::Tensor input, torch::Tensor output, torch::Tensor dequantized_params, int bits) {
    TORCH_CHECK(output.dim() == 2, "Input mismatch: fp32 buffer must be contiguous float32 2-D");
    dequantize_tensor_for_all_procs(input, output, dequantized_params, one_segment(output.size(0)), 1, bits);
}

// Feature-packed rows with a width per row (quantization_x86.cpp:164-243 / :245-305): quantized_params [rows, 3] holds
// the width in column 0 and (zero_point, scale) in columns 1-2; row i owns bytes range[i] .. range[i + 1] of the packed
// buffer.  The width check is read back: these two wait for the stream.
void mixed_codec(bool quantize, torch::Tensor fp32, torch::Tensor packed, torch::Tensor feat_range, torch::Tensor params) {
    CHECK_HIP(fp32);
    CHECK_HIP(packed);
    CHECK_HIP(feat_range);
    CHECK_HIP(params);
    const auto device = fp32.device();
    TORCH_CHECK(packed.device() == device && feat_range.device() == device && params.device() == device,
                "Input mismatch: all operands must be on one device");
    TORCH_CHECK(fp32.scalar_type() == torch::kFloat32 && fp32.dim() == 2 && fp32.is_contiguous(),
                "Input mismatch: fp32 buffer must be contiguous float32 2-D");
    TORCH_CHECK(packed.scalar_type() == torch::kUInt8 && packed.is_contiguous(),
                "Input mismatch: packed buffer must be contiguous uint8");
    TORCH_CHECK(feat_range.scalar_type() == torch::kInt64 && feat_range.is_contiguous() &&
                    feat_range.numel() == fp32.size(0) + 1,
                "Input mismatch: feature range must be int64 [rows + 1]");
    TORCH_CHECK(params.scalar_type() == torch::kFloat32 && params.is_contiguous() && params.dim() == 2 &&
                    params.size(0) == fp32.size(0) && params.size(1) == 3,
                "Input mismatch: parameters must be contiguous float32 [rows, 3]");
    torch::Tensor bad_width = torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt32).device(device));
    const auto stream = c10::hip::getCurrentHIPStream(device.index());
    c10::hip::HIPGuard guard(device.index());
    const int rc = quantize
        ? gnnagg_quantize_mixed_f32(fp32.data_ptr<float>(), packed.data_ptr<uint8_t>(), feat_range.data_ptr<int64_t>(),
                                    params.data_ptr<float>(), fp32.size(0), fp32.size(1), bad_width.data_ptr<int32_t>(),
                                    stream.stream())
        : gnnagg_dequantize_mixed_f32(packed.data_ptr<uint8_t>(), feat_range.data_ptr<int64_t>(), params.data_ptr<float>(),
                                      fp32.data_ptr<float>(), fp32.size(0), fp32.size(1), bad_width.data_ptr<int32_t>(),
                                      stream.stream());
    TORCH_CHECK(rc == GNNAGG_OK, "libgnnagg error ", rc, ": ", gnnagg_last_error());
    // the reference prints "Error: unsupported num_bits" and goes on
    TORCH_CHECK(bad_width.item<int32_t>() == 0, "Input mismatch: a row's bit width is not 2, 4 or 8");
}

void quantize_tensor_v1(torch::Tensor input, torch::Tensor output, torch::Tensor quantized_nodes_feat_range,
                        torch::Tensor quantized_params) {
    mixed_codec(true, input, output, quantized_nodes_feat_range, quantized_params);
}

void dequantize_tensor_v1(torch::Tensor input, torch::Tensor output, torch::Tensor quantized_nodes_feat_range,
                          torch::Tensor quantized_params) {
    mixed_codec(false, output, input, quantized_nodes_feat_range, quantized_params);
}

}  // namespace

PYBIND11_MODULE(computation_ops, m) {
    // the library found at run time must be the one this module was compiled against: with another version of the
    // header its entry points may take other arguments
    if (gnnagg_abi_version() != GNNAGG_ABI_VERSION)
        throw std::runtime_error("computation_ops was compiled against libgnnagg ABI version " +
                                 std::to_string(GNNAGG_ABI_VERSION) + " but the library it loaded reports " +
                                 std::to_string(gnnagg_abi_version()) + ": rebuild both (gnn_benchmark_amd/ext/build.sh)");
    m.doc() = "MI355X drop-in for the reference's computation_ops module (libgnnagg.so underneath)";
    m.def("quantize_tensor", &quantize_tensor);
    m.def("dequantize_tensor", &dequantize_tensor);
    m.def("quantize_tensor_v1", &quantize_tensor_v1);
    m.def("dequantize_tensor_v1", &dequantize_tensor_v1);
    m.def("quantize_tensor_for_all_procs", &quantize_tensor_for_all_procs);
    m.def("dequantize_tensor_for_all_procs", &dequantize_tensor_for_all_procs);
    m.def("spmm", &spmm_mi355x);
}
