// Thin PyTorch-ROCm binding `warp_ctct._C` over the C ABI of
// libwarpctct_hip.so.  torch is used for device memory (caching allocator),
// the current HIP stream and argument checking only; all arithmetic happens
// in the HIP kernels behind include/warp_ctct_hip.h.
//
// The operator names, argument names and error behaviour follow the
// reference's module (csrc/binding.cpp:326-345): wrong dtype / device /
// layout raises RuntimeError through TORCH_CHECK.  Unlike the reference there
// is no device-to-host synchronisation (its binding.cpp:68 reads
// (lx-ly).max() on the host) and a failed launch raises instead of exiting.
#include <torch/extension.h>

// PyTorch-ROCm presents HIP devices under the "cuda" device type; these are
// its guard and stream accessors for that arrangement.
#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <tuple>

#include "warp_ctct_hip.h"

namespace {

#define CHECK_CONTIGUOUS(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_DEVICE(x) TORCH_CHECK((x).device().is_cuda(), #x " must be located on the GPU")
#define CHECK_FLOAT(x) \
    TORCH_CHECK((x).scalar_type() == at::ScalarType::Float, #x " must be a Float tensor")
#define CHECK_INT(x) \
    TORCH_CHECK((x).scalar_type() == at::ScalarType::Int, #x " must be a Int tensor")

void check_rc(int rc, const char *what) {
    TORCH_CHECK(rc == WARPCTCT_OK, what, ": ", warpctct_error_string(rc));
}

using DeviceGuard = c10::hip::OptionalHIPGuardMasqueradingAsCUDA;

void *current_stream() {
    return static_cast<void *>(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA().stream());
}

void check_lengths(const torch::Tensor &ys, const torch::Tensor &lx, const torch::Tensor &ly,
                   int64_t N, int64_t U) {
    CHECK_CONTIGUOUS(ys);
    CHECK_CONTIGUOUS(lx);
    CHECK_CONTIGUOUS(ly);
    CHECK_INT(ys);
    CHECK_INT(lx);
    CHECK_INT(ly);
    CHECK_DEVICE(ys);
    CHECK_DEVICE(lx);
    CHECK_DEVICE(ly);
    TORCH_CHECK(ys.dim() == 2, "targets must have 2 dims.");
    TORCH_CHECK(lx.dim() == 1, "lx must have only 1 dim.");
    TORCH_CHECK(ly.dim() == 1, "ly must have only 1 dim.");
    TORCH_CHECK(ys.size(0) == N && lx.size(0) == N && ly.size(0) == N,
                "input args should match at dim 0 (batch N)");
    TORCH_CHECK(ys.size(1) == U, "targets must have U columns where the joint has U+1 contexts");
}

torch::Tensor make_workspace(const torch::Tensor &like, int N, int T, int U) {
    const size_t bytes = warpctct_workspace_bytes(N, T, U);
    return torch::empty({static_cast<int64_t>(bytes)},
                        like.options().dtype(at::ScalarType::Byte));
}

// Reference surface: _C.ctct_loss_fwd (csrc/binding.cpp:31-100).
// log_probs is already gathered to (N,T,U+1,3).
std::tuple<torch::Tensor, torch::Tensor> ctct_loss_fwd(const torch::Tensor &log_probs,
                                                       const torch::Tensor &ys,
                                                       const torch::Tensor &lx,
                                                       const torch::Tensor &ly,
                                                       const bool requires_grad) {
    CHECK_CONTIGUOUS(log_probs);
    CHECK_FLOAT(log_probs);
    CHECK_DEVICE(log_probs);
    TORCH_CHECK(log_probs.dim() == 4, "log probs must have 4 dims.");
    TORCH_CHECK(log_probs.size(3) == 3,
                "log probs should be first gathered to length 3 at last dim.");
    const int N = log_probs.size(0), T = log_probs.size(1), U = log_probs.size(2) - 1;
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(log_probs));

    auto ws = make_workspace(log_probs, N, T, U);
    auto costs = torch::empty({N}, log_probs.options());
    torch::Tensor grads;
    if (requires_grad) grads = torch::empty_like(log_probs);
    check_rc(warpctct_loss_forward_units_f32(
                 log_probs.data_ptr<float>(), ys.data_ptr<int>(), lx.data_ptr<int>(),
                 ly.data_ptr<int>(), N, T, U, ws.data_ptr(), ws.numel(), costs.data_ptr<float>(),
                 requires_grad ? grads.data_ptr<float>() : nullptr, current_stream()),
             "ctct_loss_fwd");
    if (requires_grad) return std::make_tuple(costs, grads);
    return std::make_tuple(costs, costs);   // as the reference, binding.cpp:98
}

// Fused entry for ctct_loss: takes the un-gathered joint (N,T,U+1,V), so the
// index build + torch.gather of warp_ctct/__init__.py:124-131 happens inside.
std::tuple<torch::Tensor, torch::Tensor> ctct_loss_joint_fwd(const torch::Tensor &joint,
                                                             const torch::Tensor &ys,
                                                             const torch::Tensor &lx,
                                                             const torch::Tensor &ly,
                                                             const bool requires_grad) {
    CHECK_CONTIGUOUS(joint);
    CHECK_FLOAT(joint);
    CHECK_DEVICE(joint);
    TORCH_CHECK(joint.dim() == 4, "log probs must have 4 dims.");
    const int N = joint.size(0), T = joint.size(1), U = joint.size(2) - 1, V = joint.size(3);
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(joint));

    auto ws = make_workspace(joint, N, T, U);
    auto costs = torch::empty({N}, joint.options());
    torch::Tensor grads;
    if (requires_grad) grads = torch::empty({N, T, U + 1, 3}, joint.options());
    check_rc(warpctct_loss_forward_f32(joint.data_ptr<float>(), ys.data_ptr<int>(),
                                       lx.data_ptr<int>(), ly.data_ptr<int>(), N, T, U, V,
                                       ws.data_ptr(), ws.numel(), costs.data_ptr<float>(),
                                       requires_grad ? grads.data_ptr<float>() : nullptr,
                                       current_stream()),
             "ctct_loss_joint_fwd");
    if (requires_grad) return std::make_tuple(costs, grads);
    return std::make_tuple(costs, costs);
}

// Backward of the fused entry: CTCTLoss.backward (warp_ctct/__init__.py:30-33)
// and the gather backward in one pass.  grad_out (N) scales sample n.
torch::Tensor ctct_loss_joint_bwd(const torch::Tensor &unit_grads, const torch::Tensor &ys,
                                  const torch::Tensor &lx, const torch::Tensor &ly,
                                  const torch::Tensor &grad_out, const int64_t V) {
    CHECK_CONTIGUOUS(unit_grads);
    CHECK_FLOAT(unit_grads);
    CHECK_DEVICE(unit_grads);
    CHECK_CONTIGUOUS(grad_out);
    CHECK_FLOAT(grad_out);
    CHECK_DEVICE(grad_out);
    TORCH_CHECK(unit_grads.dim() == 4 && unit_grads.size(3) == 3,
                "unit_grads must be (N,T,U+1,3)");
    const int N = unit_grads.size(0), T = unit_grads.size(1), U = unit_grads.size(2) - 1;
    TORCH_CHECK(grad_out.dim() == 1 && grad_out.size(0) == N, "grad_out must be (N,)");
    TORCH_CHECK(V >= 1, "V must be positive");
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(unit_grads));
    auto dense = torch::empty({N, T, U + 1, V}, unit_grads.options());
    check_rc(warpctct_dense_grad_f32(unit_grads.data_ptr<float>(), ys.data_ptr<int>(),
                                     lx.data_ptr<int>(), ly.data_ptr<int>(),
                                     grad_out.data_ptr<float>(), dense.data_ptr<float>(), N, T, U,
                                     static_cast<int>(V), current_stream()),
             "ctct_loss_joint_bwd");
    return dense;
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("ctct_loss_fwd", &ctct_loss_fwd, "CTC-Transducer loss on gathered units (forward).",
          pybind11::arg("log_probs"), pybind11::arg("ys"), pybind11::arg("lx"),
          pybind11::arg("ly"), pybind11::arg("requires_grad"));
    m.def("ctct_loss_joint_fwd", &ctct_loss_joint_fwd,
          "CTC-Transducer loss on the un-gathered joint (forward).", pybind11::arg("log_probs"),
          pybind11::arg("ys"), pybind11::arg("lx"), pybind11::arg("ly"),
          pybind11::arg("requires_grad"));
    m.def("ctct_loss_joint_bwd", &ctct_loss_joint_bwd,
          "Dense gradient wrt the joint from unit gradients.", pybind11::arg("unit_grads"),
          pybind11::arg("ys"), pybind11::arg("lx"), pybind11::arg("ly"),
          pybind11::arg("grad_out"), pybind11::arg("V"));
    m.def("library_version", []() { return std::string(warpctct_version()); });
}
