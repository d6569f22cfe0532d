// PyTorch (ROCm) extension module over the C-ABI of include/brokefish_hip.h: the counterpart of the
// reference's pybind module (reference csrc/encoder.cu:1770-1876 model_forward, :1905-1930 the
// exported functions; loaded by brokefish/nn/_build.py:149-190).  Tensors in, one asynchronous
// launch on the current HIP stream of the tensors' device, caller-allocated outputs, argument
// errors as TORCH_CHECK failures (Python RuntimeError).  No device code here: the kernels live in
// libbrokefish_hip.so, which this module links.
#include <torch/extension.h>

// PyTorch on ROCm presents its devices under the type name "cuda": these are the guard and stream
// classes of that arrangement
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <string>
#include <vector>

#include "brokefish_hip.h"

namespace {

typedef c10::optional<torch::Tensor> OptTensor;

// None (or an empty tensor, as in the reference binding, csrc/encoder.cu:1607-1612) means "absent".
torch::Tensor get(const OptTensor& t) { return t.has_value() ? *t : torch::Tensor(); }
bool absent(const torch::Tensor& t) { return !t.defined() || t.numel() == 0; }
const void* ptr_or_null(const torch::Tensor& t) { return absent(t) ? nullptr : t.data_ptr(); }

struct Checked {
    bf_eval_args a;
    c10::Device device;
};

Checked check(const torch::Tensor& boards, const torch::Tensor& control, const torch::Tensor& rep,
              const torch::Tensor& weights, const torch::Tensor& params, const torch::Tensor& policy,
              const torch::Tensor& promo, const torch::Tensor& value, int64_t d_model, int64_t n_layers,
              int64_t n_heads, int64_t d_ff, double eps, int64_t quant, int64_t kernel, int64_t n_value,
              int64_t vmode, const OptTensor& mask_, const OptTensor& best_move_, const OptTensor& active_,
              const OptTensor& workspace_, const OptTensor& leaf_index_ = c10::nullopt,
              const OptTensor& leaf_count_ = c10::nullopt) {
    const torch::Tensor mask = get(mask_), best_move = get(best_move_), active = get(active_), workspace = get(workspace_);
    const torch::Tensor leaf_index = get(leaf_index_), leaf_count = get(leaf_count_);
    TORCH_CHECK(boards.is_cuda() && boards.scalar_type() == torch::kShort && boards.is_contiguous() &&
                    boards.dim() == 2 && boards.size(1) == BF_TOKENS,
                "boards must be [n, 32] int16 contiguous on the GPU");
    const int64_t n = boards.size(0);
    TORCH_CHECK(n >= 1, "boards must hold at least one position");
    const auto dev = boards.device();
    auto on_dev = [&](const torch::Tensor& t) { return t.is_cuda() && t.device() == dev && t.is_contiguous(); };
    TORCH_CHECK(on_dev(control) && control.scalar_type() == torch::kShort && control.numel() == n,
                "control must be [n] int16 contiguous on the boards' device");
    TORCH_CHECK(on_dev(rep) && rep.scalar_type() == torch::kByte && rep.numel() == n,
                "rep must be [n] uint8 contiguous on the boards' device");
    TORCH_CHECK(on_dev(weights) && weights.scalar_type() == torch::kByte, "weights must be a uint8 blob on the boards' device");
    TORCH_CHECK(on_dev(params) && params.scalar_type() == torch::kFloat, "params must be a float32 blob on the boards' device");
    TORCH_CHECK(on_dev(policy) && on_dev(promo) && policy.scalar_type() == promo.scalar_type() &&
                    (policy.scalar_type() == torch::kHalf || policy.scalar_type() == torch::kFloat) &&
                    policy.numel() == n * BF_TOKENS * BF_POLICY && promo.numel() == n * BF_TOKENS * BF_PROMO,
                "policy must be [n, 32, 64] and promo [n, 32, 4], both fp16 or both fp32, contiguous");
    TORCH_CHECK(on_dev(value) && value.scalar_type() == torch::kFloat && value.numel() == n, "value must be [n] float32");
    if (!absent(mask))
        TORCH_CHECK(on_dev(mask) && mask.scalar_type() == torch::kLong && mask.numel() == n * BF_TOKENS,
                    "mask must be [n, 32] int64 (legal-move words)");
    if (!absent(best_move))
        TORCH_CHECK(!absent(mask) && on_dev(best_move) && best_move.scalar_type() == torch::kInt && best_move.numel() == n,
                    "best_move must be [n] int32 and needs a mask");
    if (!absent(active))
        TORCH_CHECK(on_dev(active) && (active.scalar_type() == torch::kByte || active.scalar_type() == torch::kBool) &&
                        active.numel() == n,
                    "active must be [n] uint8 or bool");
    if (!absent(workspace)) TORCH_CHECK(on_dev(workspace) && workspace.scalar_type() == torch::kByte, "workspace must be uint8");
    TORCH_CHECK(absent(leaf_index) == absent(leaf_count), "leaf_index and leaf_count come together");
    if (!absent(leaf_index))
        TORCH_CHECK(on_dev(leaf_index) && on_dev(leaf_count) && leaf_index.scalar_type() == torch::kInt &&
                        leaf_count.scalar_type() == torch::kInt && leaf_index.numel() >= n && leaf_count.numel() == 1,
                    "leaf_index must be [n] int32 and leaf_count [1] int32 (see bf_compact_leaves)");

    Checked c{bf_eval_args{}, dev};
    bf_eval_args& a = c.a;
    a.boards = static_cast<const uint16_t*>(boards.data_ptr());
    a.control = static_cast<const int16_t*>(control.data_ptr());
    a.rep = static_cast<const uint8_t*>(rep.data_ptr());
    a.mask = static_cast<const uint64_t*>(ptr_or_null(mask));
    a.n = n;
    a.shape = bf_shape{(int32_t)d_model, (int32_t)n_layers, (int32_t)n_heads, (int32_t)d_ff, (int32_t)n_value, (float)eps};
    // one pair of blobs, in the layout of the kernel that is to run
    if (kernel == BF_KERNEL_QUAD) {
        a.wstream = static_cast<const uint8_t*>(weights.data_ptr());
        a.fparams = static_cast<const float*>(params.data_ptr());
        TORCH_CHECK((size_t)weights.numel() == bf_wstream_bytes(&a.shape) && (size_t)params.numel() == bf_fparams_floats(&a.shape),
                    "weights / params are not the blobs of this shape for the four-positions-per-workgroup kernel");
        TORCH_CHECK(!absent(workspace) && (size_t)workspace.numel() >= bf_workspace_bytes(&a.shape, n),
                    "the four-positions-per-workgroup kernel needs a workspace of bf_workspace_bytes(shape, n) bytes");
        a.workspace = workspace.data_ptr();
        a.workspace_bytes = (size_t)workspace.numel();
    } else {
        a.board_wstream = static_cast<const uint8_t*>(weights.data_ptr());
        a.board_fparams = static_cast<const float*>(params.data_ptr());
        TORCH_CHECK((size_t)weights.numel() == bf_board_wstream_bytes(&a.shape) &&
                        (size_t)params.numel() == bf_board_fparams_floats(&a.shape),
                    "weights / params are not the blobs of this shape for the one-position-per-workgroup kernels");
    }
    a.policy = policy.data_ptr();
    a.promo = promo.data_ptr();
    a.value = static_cast<float*>(value.data_ptr());
    a.best_move = absent(best_move) ? nullptr : static_cast<int32_t*>(best_move.data_ptr());
    a.out_fp32 = policy.scalar_type() == torch::kFloat;
    a.quant = (int32_t)quant;
    a.active = static_cast<const uint8_t*>(ptr_or_null(active));
    a.kernel = (int32_t)kernel;
    a.value_mode = (int32_t)vmode;
    a.leaf_index = static_cast<const int32_t*>(ptr_or_null(leaf_index));
    a.leaf_count = static_cast<const int32_t*>(ptr_or_null(leaf_count));
    return c;
}

void model_forward(torch::Tensor boards, torch::Tensor control, torch::Tensor rep, torch::Tensor weights,
                   torch::Tensor params, torch::Tensor policy, torch::Tensor promo, torch::Tensor value,
                   int64_t d_model, int64_t n_layers, int64_t n_heads, int64_t d_ff, double eps, int64_t quant,
                   int64_t kernel, int64_t n_value, int64_t vmode, OptTensor mask, OptTensor best_move,
                   OptTensor active, OptTensor workspace, OptTensor leaf_index, OptTensor leaf_count) {
    const Checked c = check(boards, control, rep, weights, params, policy, promo, value, d_model, n_layers, n_heads,
                            d_ff, eps, quant, kernel, n_value, vmode, mask, best_move, active, workspace, leaf_index, leaf_count);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(c.device);     // the launch goes to the tensors' device
    const int rc = bf_model_forward(&c.a, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(c.device.index()).stream());
    TORCH_CHECK(rc == BF_OK, "bf_model_forward failed (", rc, "): ", bf_last_error());
}

// The encoder stack alone, in place on y (reference csrc/encoder.cu:1752-1764 encoder_forward(y,
// weights, alive, n_layers, eps, debug_stage)): y [n, 32, d_model] float32 is the residual stream
// entering the first layer and, on return, the stream leaving the last; alive [n, 32] int8 or bool
// masks dead tokens out of attention as keys.  No heads run and nothing is allocated.
void encoder_forward(torch::Tensor y, torch::Tensor weights, torch::Tensor params, torch::Tensor alive,
                     int64_t d_model, int64_t n_layers, int64_t n_heads, int64_t d_ff, double eps, int64_t quant,
                     int64_t kernel, int64_t n_value, OptTensor workspace_) {
    const torch::Tensor workspace = get(workspace_);
    TORCH_CHECK(y.is_cuda() && y.scalar_type() == torch::kFloat && y.is_contiguous() && y.dim() == 3 &&
                    y.size(1) == BF_TOKENS && y.size(2) == d_model && y.size(0) >= 1,
                "y must be [n, 32, d_model] float32 contiguous on the GPU");
    const auto dev = y.device();
    auto on_dev = [&](const torch::Tensor& t) { return t.is_cuda() && t.device() == dev && t.is_contiguous(); };
    TORCH_CHECK(on_dev(alive) && (alive.scalar_type() == torch::kChar || alive.scalar_type() == torch::kBool) &&
                    alive.numel() == y.size(0) * BF_TOKENS,
                "alive must be [n, 32] int8 or bool on y's device");
    TORCH_CHECK(on_dev(weights) && weights.scalar_type() == torch::kByte, "weights must be a uint8 blob on y's device");
    TORCH_CHECK(on_dev(params) && params.scalar_type() == torch::kFloat, "params must be a float32 blob on y's device");
    bf_eval_args a{};
    bf_taps taps{};
    a.n = y.size(0);
    a.shape = bf_shape{(int32_t)d_model, (int32_t)n_layers, (int32_t)n_heads, (int32_t)d_ff, (int32_t)n_value, (float)eps};
    if (kernel == BF_KERNEL_QUAD) {
        a.wstream = static_cast<const uint8_t*>(weights.data_ptr());
        a.fparams = static_cast<const float*>(params.data_ptr());
        TORCH_CHECK((size_t)weights.numel() == bf_wstream_bytes(&a.shape) && (size_t)params.numel() == bf_fparams_floats(&a.shape),
                    "weights / params are not the blobs of this shape for the four-positions-per-workgroup kernel");
        TORCH_CHECK(!absent(workspace) && on_dev(workspace) && (size_t)workspace.numel() >= bf_workspace_bytes(&a.shape, a.n),
                    "the four-positions-per-workgroup kernel needs a workspace of bf_workspace_bytes(shape, n) bytes");
        a.workspace = workspace.data_ptr();
        a.workspace_bytes = (size_t)workspace.numel();
    } else {
        a.board_wstream = static_cast<const uint8_t*>(weights.data_ptr());
        a.board_fparams = static_cast<const float*>(params.data_ptr());
        TORCH_CHECK((size_t)weights.numel() == bf_board_wstream_bytes(&a.shape) &&
                        (size_t)params.numel() == bf_board_fparams_floats(&a.shape),
                    "weights / params are not the blobs of this shape for the one-position-per-workgroup kernels");
    }
    a.quant = (int32_t)quant;
    a.kernel = (int32_t)kernel;
    taps.x_in = static_cast<const float*>(y.data_ptr());
    taps.resid_last = static_cast<float*>(y.data_ptr());
    taps.alive = static_cast<const int8_t*>(alive.data_ptr());
    a.taps = &taps;   // copied by the library before the call returns
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(dev);
    const int rc = bf_model_forward(&a, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(dev.index()).stream());
    TORCH_CHECK(rc == BF_OK, "bf_model_forward failed (", rc, "): ", bf_last_error());
}

// Cycles per phase summed over the wavefronts of one launch of the profiling build (see
// bf_profile_phases); returns an int64 tensor on the device, already written when it is read.
torch::Tensor profile_phases(torch::Tensor boards, torch::Tensor control, torch::Tensor rep, torch::Tensor weights,
                             torch::Tensor params, torch::Tensor policy, torch::Tensor promo, torch::Tensor value,
                             int64_t d_model, int64_t n_layers, int64_t n_heads, int64_t d_ff, double eps, int64_t kernel,
                             int64_t n_value, int64_t vmode, OptTensor mask, OptTensor best_move, OptTensor workspace) {
    const Checked c = check(boards, control, rep, weights, params, policy, promo, value, d_model, n_layers, n_heads,
                            d_ff, eps, BF_QUANT_INT8, kernel, n_value, vmode, mask, best_move, c10::nullopt, workspace);
    const c10::hip::HIPGuardMasqueradingAsCUDA guard(c.device);
    auto cycles = torch::zeros({(int64_t)bf_profile_phase_count()}, torch::dtype(torch::kLong).device(c.device));
    const int rc = bf_profile_phases(&c.a, c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(c.device.index()).stream(),
                                     reinterpret_cast<uint64_t*>(cycles.data_ptr<int64_t>()));
    TORCH_CHECK(rc == BF_OK, "bf_profile_phases failed (", rc, "): ", bf_last_error());
    return cycles;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.doc() = "MI355X evaluator: torch tensors in, one launch on the current HIP stream";
    m.def("model_forward", &model_forward, "boards in, policy / promo / value out", py::arg("boards"), py::arg("control"),
          py::arg("rep"), py::arg("weights"), py::arg("params"), py::arg("policy"), py::arg("promo"), py::arg("value"),
          py::arg("d_model"), py::arg("n_layers"), py::arg("n_heads"), py::arg("d_ff"), py::arg("eps"),
          py::arg("quant") = 0, py::arg("kernel") = 0, py::arg("n_value") = 1, py::arg("vmode") = 0,
          py::arg("mask") = py::none(), py::arg("best_move") = py::none(), py::arg("active") = py::none(),
          py::arg("workspace") = py::none(), py::arg("leaf_index") = py::none(), py::arg("leaf_count") = py::none());
    m.def("encoder_forward", &encoder_forward, "the encoder stack alone, in place on y", py::arg("y"), py::arg("weights"),
          py::arg("params"), py::arg("alive"), py::arg("d_model"), py::arg("n_layers"), py::arg("n_heads"), py::arg("d_ff"),
          py::arg("eps"), py::arg("quant") = 0, py::arg("kernel") = 0, py::arg("n_value") = 1, py::arg("workspace") = py::none());
    m.def("profile_phases", &profile_phases, "cycles per phase of one profiled launch", py::arg("boards"),
          py::arg("control"), py::arg("rep"), py::arg("weights"), py::arg("params"), py::arg("policy"), py::arg("promo"),
          py::arg("value"), py::arg("d_model"), py::arg("n_layers"), py::arg("n_heads"), py::arg("d_ff"), py::arg("eps"),
          py::arg("kernel") = 0, py::arg("n_value") = 1, py::arg("vmode") = 0, py::arg("mask") = py::none(),
          py::arg("best_move") = py::none(), py::arg("workspace") = py::none());
    m.def("profile_phase_names", []() {
        std::vector<std::string> names;
        for (int i = 0; i < bf_profile_phase_count(); i++) names.emplace_back(bf_profile_phase_name(i));
        return names;
    }, "phase names, in slot order");
    m.def("int8_q_max", []() {
        double s8 = 0.0, u8 = 0.0;
        bf_int8_q_max(&s8, &u8);
        return std::pair<double, double>{s8, u8};
    }, "the s8 and u8 quantisation maxima compiled into the library");
    m.def("fp8_q_max", []() { return bf_fp8_q_max(); }, "what a row's largest magnitude maps to in e4m3");
    m.def("abi_tag", []() { return (uint64_t)BF_ABI_TAG; }, "interface tag of the header this module was compiled against");
    m.def("library_abi_tag", []() { return bf_abi_tag(); }, "interface tag of the library this module is linked to");
    m.def("kernel_choice", [](int64_t d_model, int64_t n_layers, int64_t n_heads, int64_t d_ff, int64_t n_value, int64_t n,
                              int64_t quant, int64_t kernel, bool board_blobs) {
        bf_eval_args a{};
        a.shape = bf_shape{(int32_t)d_model, (int32_t)n_layers, (int32_t)n_heads, (int32_t)d_ff, (int32_t)n_value, 1e-5f};
        a.n = n;
        a.quant = (int32_t)quant;
        a.kernel = (int32_t)kernel;
        const auto nonnull = reinterpret_cast<const uint8_t*>(uintptr_t(16));     // only tested for NULL
        if (board_blobs) { a.board_wstream = nonnull; a.board_fparams = reinterpret_cast<const float*>(nonnull); }
        else { a.wstream = nonnull; a.fparams = reinterpret_cast<const float*>(nonnull); }
        const int rc = bf_kernel_choice(&a);
        TORCH_CHECK(rc >= 0, "bf_kernel_choice failed (", rc, "): ", bf_last_error());
        return rc;
    }, "which kernel (enum bf_kernel) a call with these arguments runs");
}
