// Python extension module `int4matmul`: the reference's eleven entry points
// (int4matmul.cpp:65-82) with the same names, positional argument order and
// in-place semantics, implemented as thin calls into the C ABI of
// libint4mm_hip.so (include/int4mm.h).  This file is compiled by the host
// compiler only; torch appears here for tensor metadata, the current HIP
// stream, the device guard and the scratch allocation -- nothing else.
//
// Differences from the reference, all of them stricter:
//  * every shape / dtype / device rule the reference only assert()s
//    (matmul_kernel.cu:379-416, matvec_kernel.cu:307-337, utils_kernel.cu:74-82)
//    raises an exception here;
//  * launches go to the current stream of the tensors' device, under a device
//    guard (the reference uses the legacy default stream of the current device);
//  * weight_matrix_packing raises if a 32-row block does not keep exactly 16
//    rows (the reference's device-side assert, utils_kernel.cu:41).
#include <torch/extension.h>
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <c10/hip/HIPStream.h>

#include <map>
#include <mutex>
#include <stdexcept>
#include <string>

#include "int4mm.h"

namespace {

#define TENSOR_MULT_ARGS                                                         \
    torch::Tensor outs, torch::Tensor matrix, torch::Tensor multiplier,          \
        torch::Tensor scales, torch::Tensor zeros, int group_size,               \
        c10::optional<torch::Tensor> sparse_mask
#define TENSOR_MULT_PASS outs, matrix, multiplier, scales, zeros, group_size, sparse_mask

void check_rc(int rc, const char* what) {
    if (rc == INT4MM_OK) return;
    std::string msg = std::string("int4matmul.") + what + ": " + int4mm_error_string(rc);
    if (rc == INT4MM_ERR_LAUNCH) msg += " (hipError " + std::to_string(int4mm_last_hip_error()) + ")";
    if (rc == INT4MM_ERR_BITS) throw std::invalid_argument(msg);     // -> ValueError, as the reference
    throw std::runtime_error(msg);
}

void check_tensor(const torch::Tensor& t, const char* name, c10::ScalarType dtype,
                  const c10::Device& dev) {
    TORCH_CHECK(t.defined(), name, " is undefined");
    TORCH_CHECK(t.device() == dev, name, " must be on ", dev, " but is on ", t.device());
    TORCH_CHECK(t.scalar_type() == dtype, name, " must have dtype ", dtype, " but has ", t.scalar_type());
    TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
}

// One scratch buffer per (device, stream): calls on one stream are ordered, so
// they may share it; the kernels leave it zeroed where it must be zero.
struct Scratch { torch::Tensor buf; };
std::mutex g_mu;
std::map<std::pair<int, int64_t>, Scratch> g_scratch;

torch::Tensor workspace_for(const c10::Device& dev, c10::hip::HIPStream stream, const int4mm_shape& shape, bool sparse) {
    // (covers the matvec's need; more when a matmul of this shape wants to split K)
    const size_t need = int4mm_matmul_workspace_bytes(&shape, sparse ? 1 : 0);
    std::lock_guard<std::mutex> lock(g_mu);
    auto key = std::make_pair((int)dev.index(), (int64_t)stream.id());
    auto it = g_scratch.find(key);
    if (it == g_scratch.end() || (size_t)it->second.buf.numel() < need) {
        // allocated (and zero-filled) on the current stream, which is `stream`
        auto buf = torch::zeros({(int64_t)need}, torch::TensorOptions().dtype(torch::kUInt8).device(dev));
        g_scratch[key] = Scratch{buf};
        return buf;
    }
    return it->second.buf;
}

struct Prepared {
    int4mm_shape shape;
    const void* mask;
    void* ws;
    size_t ws_bytes;
    hipStream_t stream;
};

Prepared prepare(TENSOR_MULT_ARGS, torch::Tensor& ws_keepalive) {
    TORCH_CHECK(outs.defined() && outs.is_cuda(), "outs must be a GPU tensor");
    const c10::Device dev = outs.device();
    check_tensor(outs, "outs", torch::kHalf, dev);
    check_tensor(matrix, "matrix", torch::kInt, dev);
    check_tensor(multiplier, "multiplier", torch::kHalf, dev);
    check_tensor(scales, "scales", torch::kHalf, dev);
    check_tensor(zeros, "zeros", torch::kHalf, dev);
    const bool is_sparse = sparse_mask.has_value() && sparse_mask.value().defined();
    if (is_sparse) check_tensor(sparse_mask.value(), "sparse_mask", torch::kInt, dev);

    TORCH_CHECK(multiplier.dim() == 3, "multiplier must be [batch, seq_len, in_size]");
    TORCH_CHECK(outs.dim() == 3, "outs must be [batch, seq_len, out_size]");
    TORCH_CHECK(matrix.dim() == 2, "matrix must be [packed_rows, out_size]");
    const int64_t B = multiplier.size(0), M = multiplier.size(1), K = multiplier.size(2);
    const int64_t R = matrix.size(0), S = matrix.size(1);
    TORCH_CHECK(outs.size(0) == B && outs.size(1) == M && outs.size(2) == S,
                "outs must be [", B, ", ", M, ", ", S, "] but is ", outs.sizes());

    // scales / zeros: [n_groups, out_size]; a 1-D [out_size] tensor is accepted for
    // the single-group mode, as the reference's kernels index it (kernel_test.py:177-179)
    auto group_rows = [&](const torch::Tensor& t, const char* name) -> int64_t {
        if (t.dim() == 1) {
            TORCH_CHECK(group_size < 0, name, " may be 1-D only when group_size < 0");
            TORCH_CHECK(t.size(0) == S, name, " must have out_size = ", S, " entries");
            return 1;
        }
        TORCH_CHECK(t.dim() == 2 && t.size(1) == S, name, " must be [n_groups, ", S, "]");
        return t.size(0);
    };
    const int64_t G = group_rows(scales, "scales");
    TORCH_CHECK(group_rows(zeros, "zeros") == G, "scales and zeros must have the same number of groups");
    if (is_sparse) {
        const auto& m = sparse_mask.value();
        TORCH_CHECK(m.dim() == 2 && m.size(0) * 2 == R && m.size(1) == S,
                    "sparse_mask must be [", R / 2, ", ", S, "] but is ", m.sizes());
    }

    Prepared p;
    p.shape = int4mm_shape{B, M, K, S, R, G, (int64_t)group_size};
    p.mask = is_sparse ? sparse_mask.value().data_ptr() : nullptr;
    auto stream = c10::hip::getCurrentHIPStream(dev.index());
    p.stream = stream.stream();
    ws_keepalive = workspace_for(dev, stream, p.shape, is_sparse);
    p.ws = ws_keepalive.data_ptr();
    p.ws_bytes = (size_t)ws_keepalive.numel();
    return p;
}

void matvec_bits(uint32_t bits, TENSOR_MULT_ARGS) {
    TORCH_CHECK(outs.defined(), "outs is undefined");
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(outs.device());
    torch::Tensor ws;
    Prepared p = prepare(TENSOR_MULT_PASS, ws);
    check_rc(int4mm_matvec((int)bits, outs.data_ptr(), matrix.data_ptr(), multiplier.data_ptr(),
                           scales.data_ptr(), zeros.data_ptr(), p.mask, &p.shape, p.ws, p.ws_bytes,
                           (void*)p.stream),
             "matvec");
}

void matmul_bits(uint32_t bits, TENSOR_MULT_ARGS) {
    TORCH_CHECK(outs.defined(), "outs is undefined");
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(outs.device());
    torch::Tensor ws;
    Prepared p = prepare(TENSOR_MULT_PASS, ws);
    check_rc(int4mm_matmul((int)bits, outs.data_ptr(), matrix.data_ptr(), multiplier.data_ptr(),
                           scales.data_ptr(), zeros.data_ptr(), p.mask, &p.shape, p.ws, p.ws_bytes,
                           (void*)p.stream),
             "matmul");
}

// int4matmul.cpp:9-22 -- one trio per bit width
#define REGISTER_WIDTH(N)                                                        \
    void matmul_int##N(TENSOR_MULT_ARGS) { matmul_bits(N, TENSOR_MULT_PASS); }   \
    void matvec_int##N(TENSOR_MULT_ARGS) { matvec_bits(N, TENSOR_MULT_PASS); }   \
    void spec_mm_int##N(TENSOR_MULT_ARGS) {                                      \
        TORCH_CHECK(multiplier.dim() == 3, "multiplier must be 3-D");            \
        if (multiplier.size(1) == 1) matvec_int##N(TENSOR_MULT_PASS);            \
        else matmul_int##N(TENSOR_MULT_PASS);                                    \
    }
REGISTER_WIDTH(4)
REGISTER_WIDTH(3)
REGISTER_WIDTH(2)
#undef REGISTER_WIDTH

// int4matmul.cpp:26-48
void quant_matmul(uint32_t bits, TENSOR_MULT_ARGS) {
    TORCH_CHECK(multiplier.defined() && multiplier.dim() == 3, "multiplier must be 3-D");
    const bool vec = multiplier.size(1) == 1;
    if (bits != 4 && bits != 3 && bits != 2)
        throw std::invalid_argument(vec ? "Unsupported bit width for matvec"
                                        : "Unsupported bit width for matmul");
    if (vec) matvec_bits(bits, TENSOR_MULT_PASS);
    else matmul_bits(bits, TENSOR_MULT_PASS);
}

// int4matmul.cpp:50-63, utils_kernel.cu:67-119
void weight_matrix_packing(torch::Tensor wt_outs, torch::Tensor msk_outs, torch::Tensor wt_in,
                           torch::Tensor msk_in) {
    TORCH_CHECK(wt_outs.defined() && wt_outs.is_cuda(), "wt_outs must be a GPU tensor");
    const c10::Device dev = wt_outs.device();
    c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard(dev);
    check_tensor(wt_outs, "wt_outs", torch::kInt, dev);
    check_tensor(msk_outs, "msk_outs", torch::kInt, dev);
    check_tensor(wt_in, "wt_in", torch::kByte, dev);
    check_tensor(msk_in, "msk_in", torch::kByte, dev);
    TORCH_CHECK(wt_in.dim() == 2 && msk_in.dim() == 2 && wt_outs.dim() == 2 && msk_outs.dim() == 2,
                "all four tensors must be 2-D");
    const int64_t S = wt_in.size(0), K = wt_in.size(1);
    TORCH_CHECK(msk_in.size(0) == S && msk_in.size(1) == K, "msk_in must match wt_in");
    TORCH_CHECK(K % 32 == 0, "the unpacked row count must be a multiple of 32");
    TORCH_CHECK(wt_outs.size(0) * 16 == K && wt_outs.size(1) == S, "wt_outs must be [", K / 16, ", ", S, "]");
    TORCH_CHECK(msk_outs.size(0) * 32 == K && msk_outs.size(1) == S, "msk_outs must be [", K / 32, ", ", S, "]");
    auto stream = c10::hip::getCurrentHIPStream(dev.index());
    auto bad = torch::zeros({1}, torch::TensorOptions().dtype(torch::kInt).device(dev));
    check_rc(int4mm_sparse_pack(wt_outs.data_ptr(), msk_outs.data_ptr(), wt_in.data_ptr(),
                                msk_in.data_ptr(), S, K, bad.data_ptr(), (void*)stream.stream()),
             "weight_matrix_packing");
    const int n_bad = bad.item<int>();      // packing is an offline step: synchronising is fine
    TORCH_CHECK(n_bad == 0, "weight_matrix_packing: ", n_bad,
                " 32-row blocks do not keep exactly 16 rows");
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("weight_matrix_packing", &weight_matrix_packing, "int4_sparse_pack");

    m.def("quant_matmul", &quant_matmul, "intn_fp16_mult");

    m.def("quant_int4_linear_mult", &spec_mm_int4, "int4_fp16_mult");
    m.def("quant_int4_linear_mult_mtx", &matmul_int4, "int4_fp16_mult_mtx");
    m.def("quant_int4_linear_mult_vec", &matvec_int4, "int4_fp16_mult_vec");

    m.def("quant_int3_linear_mult", &spec_mm_int3, "int3_fp16_mult");
    m.def("quant_int3_linear_mult_mtx", &matmul_int3, "int3_fp16_mult_mtx");
    m.def("quant_int3_linear_mult_vec", &matvec_int3, "int3_fp16_mult_vec");

    m.def("quant_int2_linear_mult", &spec_mm_int2, "int2_fp16_mult");
    m.def("quant_int2_linear_mult_mtx", &matmul_int2, "int2_fp16_mult_mtx");
    m.def("quant_int2_linear_mult_vec", &matvec_int2, "int2_fp16_mult_vec");
}
