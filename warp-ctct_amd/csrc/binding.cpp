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

torch::Tensor make_bytes(const torch::Tensor &like, size_t bytes) {
    return torch::empty({static_cast<int64_t>(bytes)}, like.options().dtype(at::ScalarType::Byte));
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

// Element type of a joint tensor for the C ABI; anything but float, half and
// bfloat16 is refused (the Python wrapper converts other types to float).
int io_type_of(const torch::Tensor &t) {
    switch (t.scalar_type()) {
        case at::ScalarType::Float: return WARPCTCT_F32;
        case at::ScalarType::Half: return WARPCTCT_F16;
        case at::ScalarType::BFloat16: return WARPCTCT_BF16;
        default: TORCH_CHECK(false, "joint must be float32, float16 or bfloat16");
    }
    return -1;
}

// Fused entry for ctct_loss: takes the un-gathered joint (N,T,U+1,V) of type
// float, half or bfloat16, so the index build + torch.gather + .float() of
// warp_ctct/__init__.py:124-136 happen inside, and the reduction of :138-147
// too: reduction 0 = none, 1 = sum, 2 = mean.  Returns (loss, workspace): loss
// is the (N,) costs (divided by lx if average_frames) or the reduced scalar,
// always float32; the workspace (units, alpha, beta) is what
// dense_patch_lattice needs in backward; without requires_grad only beta runs
// and loss is returned twice (as the reference does, binding.cpp:98).
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor> ctct_loss_joint_fwd(
    const torch::Tensor &joint, const torch::Tensor &ys, const torch::Tensor &lx,
    const torch::Tensor &ly, const bool requires_grad, const int64_t reduction,
    const bool average_frames, const bool clear_gradient) {
    // the joint may be any strided view (the reference's torch.gather takes
    // views as they are, warp_ctct/__init__.py:131): no copy is made
    CHECK_DEVICE(joint);
    const int dtype = io_type_of(joint);
    TORCH_CHECK(joint.dim() == 4, "log probs must have 4 dims.");
    TORCH_CHECK(reduction >= 0 && reduction <= 2, "reduction must be 0 (none), 1 (sum), 2 (mean)");
    const int N = joint.size(0), T = joint.size(1), U = joint.size(2) - 1, V = joint.size(3);
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(joint));

    auto ws = make_workspace(joint, N, T, U);
    const auto f32 = joint.options().dtype(at::ScalarType::Float);
    // the per-sample costs and the reduced scalar share one allocation
    auto costs_and_sum = N > 0 ? torch::empty({N + 1}, f32) : torch::zeros({1}, f32);
    auto costs = costs_and_sum.narrow(0, 0, N);
    torch::Tensor reduced;
    if (reduction != 0) reduced = costs_and_sum.select(0, N);
    const long strides[4] = {static_cast<long>(joint.stride(0)), static_cast<long>(joint.stride(1)),
                             static_cast<long>(joint.stride(2)), static_cast<long>(joint.stride(3))};
    // With clear_gradient the buffer of the dense gradient is allocated now and
    // cleared beside the gather and the lattices; the backward then only
    // patches it (dense_patch_lattice).  Otherwise `dense` comes back empty.
    torch::Tensor dense;
    if (requires_grad && clear_gradient)
        dense = torch::empty({N, T, U + 1, V}, joint.options());
    else
        dense = torch::empty({0}, joint.options());
    check_rc(warpctct_loss_lattice_clearing(
                 joint.data_ptr(), dtype, strides, ys.data_ptr<int>(), lx.data_ptr<int>(),
                 ly.data_ptr<int>(), N, T, U, V, ws.data_ptr(), ws.numel(),
                 costs.data_ptr<float>(), requires_grad ? 1 : 0, static_cast<int>(reduction),
                 average_frames ? 1 : 0, reduction != 0 ? reduced.data_ptr<float>() : nullptr,
                 dense.numel() > 0 ? dense.data_ptr() : nullptr,
                 static_cast<size_t>(dense.numel()) * dense.element_size(), current_stream()),
             "ctct_loss_joint_fwd");
    const torch::Tensor &loss = reduction != 0 ? reduced : costs;
    if (requires_grad) return std::make_tuple(loss, ws, dense);
    return std::make_tuple(loss, loss, dense);
}

// The two halves of the dense gradient as separate operators, so that a caller
// can bracket the zero-fill kernel alone with HIP events.  `like` gives the
// device and the element type (float, half or bfloat16).
torch::Tensor dense_zero_fill(const torch::Tensor &like, const int64_t N, const int64_t T,
                              const int64_t U1, const int64_t V) {
    CHECK_DEVICE(like);
    io_type_of(like);
    TORCH_CHECK(N >= 0 && T >= 0 && U1 >= 1 && V >= 1, "invalid sizes");
    const DeviceGuard device_guard(device_of(like));
    auto dense = torch::empty({N, T, U1, V}, like.options());
    check_rc(warpctct_zero_fill(dense.data_ptr(),
                                static_cast<size_t>(dense.numel()) * dense.element_size(),
                                current_stream()),
             "dense_zero_fill");
    return dense;
}

// grad_out: (N,) per-sample upstream gradients, or a 0-dim / 1-element tensor
// that is broadcast; every sample is further scaled by `scale` and, with
// average_frames, divided by lx[n].
void dense_patch_lattice(const torch::Tensor &workspace, const torch::Tensor &ys,
                         const torch::Tensor &lx, const torch::Tensor &ly,
                         const torch::Tensor &grad_out, const double scale,
                         const bool average_frames, torch::Tensor &dense) {
    CHECK_CONTIGUOUS(workspace);
    CHECK_DEVICE(workspace);
    TORCH_CHECK(workspace.scalar_type() == at::ScalarType::Byte, "workspace must be a byte tensor");
    CHECK_CONTIGUOUS(grad_out);
    CHECK_FLOAT(grad_out);
    CHECK_DEVICE(grad_out);
    CHECK_CONTIGUOUS(dense);
    CHECK_DEVICE(dense);
    const int dtype = io_type_of(dense);
    TORCH_CHECK(dense.dim() == 4, "dense must be (N,T,U+1,V)");
    const int N = dense.size(0), T = dense.size(1), U = dense.size(2) - 1, V = dense.size(3);
    TORCH_CHECK(grad_out.numel() == N || grad_out.numel() == 1, "grad_out must have N or 1 elements");
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(dense));
    const int stride = (grad_out.numel() == 1 && N > 1) ? 0 : 1;
    check_rc(warpctct_dense_patch_lattice(
                 workspace.data_ptr(), workspace.numel(), ys.data_ptr<int>(), lx.data_ptr<int>(),
                 ly.data_ptr<int>(), grad_out.data_ptr<float>(), stride, static_cast<float>(scale),
                 average_frames ? 1 : 0, dense.data_ptr(), dtype, N, T, U, V, current_stream()),
             "dense_patch_lattice");
}

// Compact hand-off for callers that own the joiner: costs (N,) and the unit
// gradients (N,T,U+1,3) = d costs[n] / d joint[n,t,u,{0, y[u-1], y[u]}] (what
// _C.ctct_loss_fwd of the reference returns, csrc/binding.cpp:31-100), from the
// un-gathered joint; no dense gradient is formed.
std::tuple<torch::Tensor, torch::Tensor> ctct_loss_compact_fwd(const torch::Tensor &joint,
                                                               const torch::Tensor &ys,
                                                               const torch::Tensor &lx,
                                                               const torch::Tensor &ly) {
    CHECK_CONTIGUOUS(joint);
    CHECK_DEVICE(joint);
    const int dtype = io_type_of(joint);
    TORCH_CHECK(joint.dim() == 4, "log probs must have 4 dims.");
    const int N = joint.size(0), T = joint.size(1), U = joint.size(2) - 1, V = joint.size(3);
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(joint));
    auto ws = make_workspace(joint, N, T, U);
    const auto f32 = joint.options().dtype(at::ScalarType::Float);
    auto costs = torch::empty({N}, f32);
    auto grads = torch::empty({N, T, U + 1, 3}, f32);
    check_rc(warpctct_loss_forward(joint.data_ptr(), dtype, ys.data_ptr<int>(), lx.data_ptr<int>(),
                                   ly.data_ptr<int>(), N, T, U, V, ws.data_ptr(), ws.numel(),
                                   costs.data_ptr<float>(), grads.data_ptr<float>(),
                                   current_stream()),
             "ctct_loss_compact_fwd");
    return std::make_tuple(costs, grads);
}

// ctct_loss on logits: log_softmax over the vocabulary happens inside (the
// caller of the reference applies it before warp_ctct.ctct_loss).  Same
// contract as ctct_loss_joint_fwd; the workspace also holds the row-wise
// logsumexp that logits_grad needs.
std::tuple<torch::Tensor, torch::Tensor> ctct_loss_logits_fwd(const torch::Tensor &logits,
                                                              const torch::Tensor &ys,
                                                              const torch::Tensor &lx,
                                                              const torch::Tensor &ly,
                                                              const bool requires_grad,
                                                              const int64_t reduction,
                                                              const bool average_frames) {
    CHECK_CONTIGUOUS(logits);
    CHECK_DEVICE(logits);
    const int dtype = io_type_of(logits);
    TORCH_CHECK(logits.dim() == 4, "logits must have 4 dims.");
    TORCH_CHECK(reduction >= 0 && reduction <= 2, "reduction must be 0 (none), 1 (sum), 2 (mean)");
    const int N = logits.size(0), T = logits.size(1), U = logits.size(2) - 1, V = logits.size(3);
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(logits));
    auto ws = make_bytes(logits, warpctct_logits_workspace_bytes(N, T, U));
    const auto f32 = logits.options().dtype(at::ScalarType::Float);
    auto costs_and_sum = N > 0 ? torch::empty({N + 1}, f32) : torch::zeros({1}, f32);
    auto costs = costs_and_sum.narrow(0, 0, N);
    torch::Tensor reduced;
    if (reduction != 0) reduced = costs_and_sum.select(0, N);
    check_rc(warpctct_logits_loss_lattice(logits.data_ptr(), dtype, ys.data_ptr<int>(),
                                          lx.data_ptr<int>(), ly.data_ptr<int>(), N, T, U, V,
                                          ws.data_ptr(), ws.numel(), costs.data_ptr<float>(),
                                          requires_grad ? 1 : 0, static_cast<int>(reduction),
                                          average_frames ? 1 : 0,
                                          reduction != 0 ? reduced.data_ptr<float>() : nullptr,
                                          current_stream()),
             "ctct_loss_logits_fwd");
    const torch::Tensor &loss = reduction != 0 ? reduced : costs;
    if (requires_grad) return std::make_tuple(loss, ws);
    return std::make_tuple(loss, loss);
}

// d(loss)/d(logits), every element written; grad_out, scale, average_frames as
// in dense_patch_lattice.
torch::Tensor ctct_loss_logits_bwd(const torch::Tensor &workspace, const torch::Tensor &logits,
                                   const torch::Tensor &ys, const torch::Tensor &lx,
                                   const torch::Tensor &ly, const torch::Tensor &grad_out,
                                   const double scale, const bool average_frames) {
    CHECK_CONTIGUOUS(workspace);
    CHECK_DEVICE(workspace);
    TORCH_CHECK(workspace.scalar_type() == at::ScalarType::Byte, "workspace must be a byte tensor");
    CHECK_CONTIGUOUS(grad_out);
    CHECK_FLOAT(grad_out);
    CHECK_DEVICE(grad_out);
    CHECK_CONTIGUOUS(logits);
    CHECK_DEVICE(logits);
    const int dtype = io_type_of(logits);
    TORCH_CHECK(logits.dim() == 4, "logits must be (N,T,U+1,V)");
    const int N = logits.size(0), T = logits.size(1), U = logits.size(2) - 1, V = logits.size(3);
    TORCH_CHECK(grad_out.numel() == N || grad_out.numel() == 1, "grad_out must have N or 1 elements");
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(logits));
    auto grad = torch::empty_like(logits);
    const int stride = (grad_out.numel() == 1 && N > 1) ? 0 : 1;
    check_rc(warpctct_logits_grad_lattice(
                 workspace.data_ptr(), workspace.numel(), logits.data_ptr(), dtype,
                 ys.data_ptr<int>(), lx.data_ptr<int>(), ly.data_ptr<int>(),
                 grad_out.data_ptr<float>(), stride, static_cast<float>(scale),
                 average_frames ? 1 : 0, grad.data_ptr(), N, T, U, V, current_stream()),
             "ctct_loss_logits_bwd");
    return grad;
}

// Backward of the fused entry: CTCTLoss.backward (warp_ctct/__init__.py:30-33)
// and the gather backward.  grad_out (N) scales sample n.
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

// Reference surface: _C.ctct_loss_simple_fwd (csrc/binding.cpp:103-222).
// f (N,T,U+1) and g (N,U+1,3) are already gathered; den is (N,T,U+1), or any
// tensor that is not 3-d to select the unnormalised variant (binding.cpp:144).
// Returns (costs, grad_f, grad_g, grad_den); the gradients are undefined
// (None in Python) when requires_grad is false, grad_den also when
// unnormalised.
std::tuple<torch::Tensor, torch::Tensor, torch::Tensor, torch::Tensor> ctct_loss_simple_fwd(
    const torch::Tensor &f, const torch::Tensor &g, const torch::Tensor &ys,
    const torch::Tensor &den, const torch::Tensor &lx, const torch::Tensor &ly,
    const bool requires_grad) {
    CHECK_CONTIGUOUS(f);
    CHECK_CONTIGUOUS(g);
    CHECK_FLOAT(f);
    CHECK_FLOAT(g);
    CHECK_DEVICE(f);
    CHECK_DEVICE(g);
    TORCH_CHECK(f.dim() == 3, "f must have 3 dims.");
    TORCH_CHECK(g.dim() == 3, "g must have 3 dims.");
    TORCH_CHECK(f.size(2) == g.size(1),
                "f should be gathered at last dim to length U matching the g at dim 1.");
    TORCH_CHECK(g.size(2) == 3, "g should be first gathered to length 3 at last dim.");
    const int N = f.size(0), T = f.size(1), U = g.size(1) - 1;
    TORCH_CHECK(g.size(0) == N, "input args should match at dim 0 (batch N)");
    check_lengths(ys, lx, ly, N, U);
    const bool normalized = (den.dim() == 3);
    if (normalized) {
        CHECK_CONTIGUOUS(den);
        CHECK_DEVICE(den);
        CHECK_FLOAT(den);
        TORCH_CHECK(den.size(0) == N && den.size(1) == T && den.size(2) == U + 1,
                    "den must be (N,T,U+1)");
    }
    const DeviceGuard device_guard(device_of(f));
    auto ws = make_bytes(f, warpctct_simple_workspace_bytes(N, T, U));
    auto costs = torch::empty({N}, f.options());
    torch::Tensor grad_f, grad_g, grad_den;
    if (requires_grad) {
        grad_f = torch::empty_like(f);
        grad_g = torch::empty_like(g);
        if (normalized) grad_den = torch::empty_like(den);
    }
    check_rc(warpctct_simple_forward_units_f32(
                 f.data_ptr<float>(), g.data_ptr<float>(),
                 normalized ? den.data_ptr<float>() : nullptr, ys.data_ptr<int>(),
                 lx.data_ptr<int>(), ly.data_ptr<int>(), N, T, U, ws.data_ptr(), ws.numel(),
                 costs.data_ptr<float>(), requires_grad ? grad_f.data_ptr<float>() : nullptr,
                 requires_grad ? grad_g.data_ptr<float>() : nullptr,
                 (requires_grad && normalized) ? grad_den.data_ptr<float>() : nullptr,
                 current_stream()),
             "ctct_loss_simple_fwd");
    return std::make_tuple(costs, grad_f, grad_g, grad_den);
}

// Fused entry for ctct_simple_loss: un-gathered f (N,T,V), g (N,U+1,V).
// Returns (loss, den, shifted, grad_f_g, grad_g_g, grad_den); loss is the (N,)
// costs (divided by lx with average_frames) for reduction 0, their sum (1) or
// mean (2) as a 0-dim tensor otherwise.  When normalized,
// den is defined and shifted = [fmax (N,T), gmax (N,U+1), fexp (N,T,Vp),
// gexp (N,U+1,Vp)], the row maxima of f and g and the operands shifted by them
// and exponentiated, which the backward reuses; otherwise shifted is empty.
// The three compact gradients are defined when requires_grad.
std::tuple<torch::Tensor, torch::Tensor, std::vector<torch::Tensor>, torch::Tensor, torch::Tensor,
           torch::Tensor>
ctct_simple_fwd(const torch::Tensor &f, const torch::Tensor &g, const torch::Tensor &ys,
                const torch::Tensor &lx, const torch::Tensor &ly, const bool normalized,
                const bool requires_grad, const int64_t reduction, const bool average_frames) {
    CHECK_CONTIGUOUS(f);
    CHECK_CONTIGUOUS(g);
    CHECK_FLOAT(f);
    CHECK_FLOAT(g);
    CHECK_DEVICE(f);
    CHECK_DEVICE(g);
    TORCH_CHECK(reduction >= 0 && reduction <= 2, "reduction must be 0 (none), 1 (sum), 2 (mean)");
    TORCH_CHECK(f.dim() == 3, "f must have 3 dims.");
    TORCH_CHECK(g.dim() == 3, "g must have 3 dims.");
    TORCH_CHECK(f.size(2) == g.size(2), "f and g must share the vocabulary dim");
    const int N = f.size(0), T = f.size(1), U = g.size(1) - 1, V = f.size(2);
    TORCH_CHECK(g.size(0) == N, "input args should match at dim 0 (batch N)");
    check_lengths(ys, lx, ly, N, U);
    const DeviceGuard device_guard(device_of(f));
    auto ws = make_bytes(f, warpctct_simple_workspace_bytes(N, T, U));
    // the per-sample costs and the reduced scalar share one allocation
    auto costs_and_sum = N > 0 ? torch::empty({N + 1}, f.options()) : torch::zeros({1}, f.options());
    auto costs = costs_and_sum.narrow(0, 0, N);
    torch::Tensor reduced;
    if (reduction != 0) reduced = costs_and_sum.select(0, N);
    torch::Tensor den, fmax, gmax, fexp, gexp, grad_f, grad_g, grad_den;
    std::vector<torch::Tensor> shifted;
    if (normalized) {
        const int Vp = warpctct_logmm_padded_reduction(V);
        den = torch::empty({N, T, U + 1}, f.options());
        fmax = torch::empty({N, T}, f.options());
        gmax = torch::empty({N, U + 1}, f.options());
        // (not needed where the kernels read f itself)
        const bool keeps = warpctct_simple_needs_fexp(f.data_ptr<float>(), T, U, V) != 0;
        fexp = keeps ? torch::empty({N, T, Vp}, f.options()) : torch::empty({0}, f.options());
        gexp = torch::empty({N, U + 1, Vp}, f.options());
        shifted = {fmax, gmax, fexp, gexp};
    }
    if (requires_grad) {
        grad_f = torch::empty({N, T, U + 1}, f.options());
        grad_g = torch::empty({N, U + 1, 3}, f.options());
        if (normalized) grad_den = torch::empty({N, T, U + 1}, f.options());
    }
    check_rc(warpctct_simple_forward_reduced_f32(
                 f.data_ptr<float>(), g.data_ptr<float>(), ys.data_ptr<int>(), lx.data_ptr<int>(),
                 ly.data_ptr<int>(), N, T, U, V, normalized ? 1 : 0, ws.data_ptr(), ws.numel(),
                 normalized ? den.data_ptr<float>() : nullptr,
                 normalized ? fmax.data_ptr<float>() : nullptr,
                 normalized ? gmax.data_ptr<float>() : nullptr,
                 (normalized && fexp.numel() > 0) ? fexp.data_ptr<float>() : nullptr,
                 normalized ? gexp.data_ptr<float>() : nullptr, costs.data_ptr<float>(),
                 requires_grad ? grad_f.data_ptr<float>() : nullptr,
                 requires_grad ? grad_g.data_ptr<float>() : nullptr,
                 (requires_grad && normalized) ? grad_den.data_ptr<float>() : nullptr,
                 static_cast<int>(reduction), average_frames ? 1 : 0,
                 reduction != 0 ? reduced.data_ptr<float>() : nullptr, current_stream()),
             "ctct_simple_fwd");
    return std::make_tuple(reduction != 0 ? reduced : costs, den, shifted, grad_f, grad_g, grad_den);
}

// Dense gradients (N,T,V) and (N,U+1,V) of the fused entry; sample n is
// weighted by grad_out ((N,), or one element that is broadcast) times `scale`,
// divided by lx[n] with average_frames.  den / grad_den undefined selects the
// unnormalised variant.
std::tuple<torch::Tensor, torch::Tensor> ctct_simple_bwd(
    const torch::Tensor &f, const torch::Tensor &g, const c10::optional<torch::Tensor> &den,
    const std::vector<torch::Tensor> &shifted,
    const torch::Tensor &grad_f_g, const torch::Tensor &grad_g_g,
    const c10::optional<torch::Tensor> &grad_den, const torch::Tensor &ys, const torch::Tensor &lx,
    const torch::Tensor &ly, const torch::Tensor &grad_out, const bool want_f, const bool want_g,
    const double scale, const bool average_frames) {
    CHECK_CONTIGUOUS(f);
    CHECK_CONTIGUOUS(g);
    CHECK_FLOAT(f);
    CHECK_FLOAT(g);
    CHECK_DEVICE(f);
    CHECK_DEVICE(g);
    CHECK_CONTIGUOUS(grad_f_g);
    CHECK_CONTIGUOUS(grad_g_g);
    CHECK_FLOAT(grad_f_g);
    CHECK_FLOAT(grad_g_g);
    CHECK_CONTIGUOUS(grad_out);
    CHECK_FLOAT(grad_out);
    CHECK_DEVICE(grad_out);
    TORCH_CHECK(f.dim() == 3 && g.dim() == 3 && f.size(2) == g.size(2), "f (N,T,V), g (N,U+1,V)");
    const int N = f.size(0), T = f.size(1), U = g.size(1) - 1, V = f.size(2);
    check_lengths(ys, lx, ly, N, U);
    TORCH_CHECK(grad_out.dim() == 1 && (grad_out.size(0) == N || grad_out.size(0) == 1),
                "grad_out must be (N,) or one element");
    const int grad_out_stride = grad_out.size(0) == N ? 1 : 0;
    TORCH_CHECK(grad_f_g.dim() == 3 && grad_f_g.size(0) == N && grad_f_g.size(1) == T &&
                    grad_f_g.size(2) == U + 1, "grad_f must be (N,T,U+1)");
    TORCH_CHECK(grad_g_g.dim() == 3 && grad_g_g.size(0) == N && grad_g_g.size(1) == U + 1 &&
                    grad_g_g.size(2) == 3, "grad_g must be (N,U+1,3)");
    const bool normalized = den.has_value() && den->defined();
    if (normalized) {
        TORCH_CHECK(grad_den.has_value() && grad_den->defined(), "grad_den is required with den");
        CHECK_CONTIGUOUS(*den);
        CHECK_FLOAT(*den);
        CHECK_DEVICE(*den);
        CHECK_CONTIGUOUS(*grad_den);
        CHECK_FLOAT(*grad_den);
        TORCH_CHECK(den->numel() == (int64_t)N * T * (U + 1) && grad_den->numel() == den->numel(),
                    "den and grad_den must be (N,T,U+1)");
        const int Vp = warpctct_logmm_padded_reduction(V);
        TORCH_CHECK(shifted.size() == 4, "shifted = [fmax, gmax, fexp, gexp] is required with den");
        for (const auto &t : shifted) {
            CHECK_CONTIGUOUS(t);
            CHECK_FLOAT(t);
            CHECK_DEVICE(t);
        }
        TORCH_CHECK(shifted[0].numel() == (int64_t)N * T &&
                        shifted[1].numel() == (int64_t)N * (U + 1),
                    "fmax must be (N,T), gmax (N,U+1)");
        const bool keeps = warpctct_simple_needs_fexp(f.data_ptr<float>(), T, U, V) != 0;
        TORCH_CHECK((shifted[2].numel() == (int64_t)N * T * Vp || !keeps) &&
                        shifted[3].numel() == (int64_t)N * (U + 1) * Vp,
                    "fexp must be (N,T,Vp), gexp (N,U+1,Vp)");
    }
    const DeviceGuard device_guard(device_of(f));
    torch::Tensor dense_f, dense_g;
    if (want_f) dense_f = torch::empty_like(f);
    if (want_g) dense_g = torch::empty_like(g);
    auto ws = make_bytes(f, normalized ? warpctct_simple_backward_workspace_bytes(N, T, U) : 0);
    // scratch for the per-sample weights, where grad_out is not yet that array
    torch::Tensor weights;
    if (grad_out_stride != 1 || scale != 1.0 || average_frames) weights = torch::empty({N}, f.options());
    check_rc(warpctct_simple_backward_weighted_f32(
                 f.data_ptr<float>(), g.data_ptr<float>(),
                 normalized ? den->data_ptr<float>() : nullptr,
                 normalized ? shifted[0].data_ptr<float>() : nullptr,
                 normalized ? shifted[1].data_ptr<float>() : nullptr,
                 (normalized && shifted[2].numel() > 0) ? shifted[2].data_ptr<float>() : nullptr,
                 normalized ? shifted[3].data_ptr<float>() : nullptr, grad_f_g.data_ptr<float>(),
                 grad_g_g.data_ptr<float>(), normalized ? grad_den->data_ptr<float>() : nullptr,
                 ys.data_ptr<int>(), lx.data_ptr<int>(), ly.data_ptr<int>(),
                 grad_out.data_ptr<float>(), grad_out_stride, static_cast<float>(scale),
                 average_frames ? 1 : 0, weights.defined() ? weights.data_ptr<float>() : nullptr, N,
                 T, U, V, ws.data_ptr(), ws.numel(),
                 want_f ? dense_f.data_ptr<float>() : nullptr,
                 want_g ? dense_g.data_ptr<float>() : nullptr, current_stream()),
             "ctct_simple_bwd");
    return std::make_tuple(dense_f, dense_g);
}

long batch_stride(const torch::Tensor &t, int64_t B) {
    return (t.size(0) == 1 && B > 1) ? 0L : static_cast<long>(t.stride(0));
}

// Reference surface: _C.log_matmul (csrc/binding.cpp:224-245).  Strided
// operands are accepted as they are (the reference passes a transposed view).
torch::Tensor log_matmul(const torch::Tensor &self, const torch::Tensor &other) {
    CHECK_FLOAT(self);
    CHECK_FLOAT(other);
    TORCH_CHECK(self.is_cuda(), "need cuda tensors");
    TORCH_CHECK(self.device() == other.device(), "need tensors on same GPU");
    TORCH_CHECK(self.dim() == 3 && other.dim() == 3, "invalid sizes");
    TORCH_CHECK(self.size(2) == other.size(1), "invalid sizes");
    TORCH_CHECK(other.size(0) == self.size(0) || other.size(0) == 1, "invalid sizes");
    const DeviceGuard device_guard(device_of(self));
    const int B = self.size(0), M = self.size(1), K = self.size(2), Nn = other.size(2);
    auto out = torch::empty({B, M, Nn}, self.options());
    auto ws = make_bytes(self, warpctct_logmm_workspace_bytes(B, M, K, Nn));
    check_rc(warpctct_logmm_fwd_f32(self.data_ptr<float>(), self.stride(0), self.stride(1),
                                    self.stride(2), other.data_ptr<float>(),
                                    batch_stride(other, B), other.stride(1), other.stride(2), B, M,
                                    K, Nn, ws.data_ptr(), ws.numel(), out.data_ptr<float>(),
                                    current_stream()),
             "log_matmul");
    return out;
}

// Reference surface: _C.log_matmul_backward (csrc/binding.cpp:247-324).
std::tuple<torch::Tensor, torch::Tensor> log_matmul_backward(
    const torch::Tensor &grad_out, const torch::Tensor &lhs, const torch::Tensor &rhs,
    const torch::Tensor &result, const std::array<bool, 2> grad_input_mask) {
    torch::Tensor grad_lhs, grad_rhs;
    if (!grad_out.defined()) return std::make_tuple(grad_lhs, grad_rhs);
    CHECK_FLOAT(grad_out);
    CHECK_FLOAT(lhs);
    CHECK_FLOAT(rhs);
    CHECK_FLOAT(result);
    TORCH_CHECK(lhs.is_cuda() && rhs.is_cuda() && result.is_cuda() && grad_out.is_cuda(),
                "need cuda tensors");
    TORCH_CHECK(lhs.dim() == 3 && rhs.dim() == 3 && result.dim() == 3 && grad_out.dim() == 3,
                "invalid sizes");
    int B = lhs.size(0), M = lhs.size(1);
    const int K = lhs.size(2), Nn = rhs.size(2);
    TORCH_CHECK((rhs.size(0) == B || rhs.size(0) == 1) && rhs.size(1) == K, "invalid sizes");
    TORCH_CHECK(result.size(0) == B && result.size(1) == M && result.size(2) == Nn &&
                    grad_out.sizes() == result.sizes(), "invalid sizes");
    const DeviceGuard device_guard(device_of(lhs));
    auto go = grad_out.contiguous();
    auto res = result.contiguous();
    // A size-1 batch of rhs is shared by every batch entry of lhs (the
    // reference expands it in the forward and undoes the broadcast with a
    // reduction over the batch, csrc/binding.cpp:283-296).  With one rhs the
    // batch of lhs is just more rows: the (B,M,K) problem is the (1,B*M,K)
    // problem, whose rhs gradient already sums over all B*M rows.
    torch::Tensor lhs_rows = lhs;
    const int64_t out_B = B, out_M = M;
    const bool shared_rhs = rhs.size(0) == 1 && B > 1;
    if (shared_rhs) {
        if (lhs.stride(0) != (int64_t)M * lhs.stride(1)) lhs_rows = lhs.contiguous();
        M = B * M;
        B = 1;
    }
    if (grad_input_mask[0]) grad_lhs = torch::empty({out_B, out_M, K}, lhs.options());
    if (grad_input_mask[1]) grad_rhs = torch::empty({rhs.size(0), K, Nn}, rhs.options());
    auto ws = make_bytes(lhs, warpctct_logmm_workspace_bytes(B, M, K, Nn));
    check_rc(warpctct_logmm_bwd_f32(
                 go.data_ptr<float>(), lhs_rows.data_ptr<float>(), lhs_rows.stride(0),
                 lhs_rows.stride(1), lhs_rows.stride(2), rhs.data_ptr<float>(), rhs.stride(0),
                 rhs.stride(1), rhs.stride(2), res.data_ptr<float>(), B, M, K, Nn, ws.data_ptr(),
                 ws.numel(), grad_input_mask[0] ? grad_lhs.data_ptr<float>() : nullptr,
                 (long)M * K, (long)K, 1L,
                 grad_input_mask[1] ? grad_rhs.data_ptr<float>() : nullptr, (long)K * Nn, (long)Nn,
                 1L, current_stream()),
             "log_matmul_backward");
    return std::make_tuple(grad_lhs, grad_rhs);
}

// ---- the public losses as autograd functions -------------------------------
// One crossing from Python into this module per direction: the forward below
// is what warp_ctct.ctct_loss calls, and autograd calls the backward here
// without going through Python.  They are the counterpart of the reference's
// gather + CTCTLoss + reduction (warp_ctct/__init__.py:124-147), of its
// SimpleCTCTLoss / LogMMExp chain (:55-85, :36-52, :195-225) and of the caller's
// log_softmax in front of ctct_loss.

// labels and lengths as contiguous int32 (the reference casts with .int(),
// warp_ctct/__init__.py:135-136); tensors that already are cost nothing
torch::Tensor as_int32(const torch::Tensor &t) {
    if (t.scalar_type() == at::ScalarType::Int && t.is_contiguous()) return t;
    return t.to(at::ScalarType::Int).contiguous();
}

torch::Tensor upstream(const torch::Tensor &grad_output) {
    return grad_output.reshape({-1}).to(at::ScalarType::Float).contiguous();
}

using torch::autograd::AutogradContext;
using torch::autograd::tensor_list;

class JointLoss : public torch::autograd::Function<JointLoss> {
   public:
    static torch::Tensor forward(AutogradContext *ctx, const torch::Tensor &joint,
                                 const torch::Tensor &ys, const torch::Tensor &lx,
                                 const torch::Tensor &ly, const bool requires_grad,
                                 const int64_t reduction, const bool average_frames,
                                 const bool clear_in_forward) {
        auto out = ctct_loss_joint_fwd(joint, ys, lx, ly, requires_grad, reduction, average_frames,
                                       requires_grad && clear_in_forward);
        if (requires_grad) {
            ctx->save_for_backward({std::get<1>(out), ys, lx, ly});
            // the buffer of the dense gradient, cleared beside the lattices: it
            // serves the first backward; a later one (retained graph) clears its own
            ctx->saved_data["dense"] = std::get<2>(out);
            ctx->saved_data["like"] = torch::empty({0}, joint.options());
            ctx->saved_data["sizes"] = joint.sizes().vec();
            ctx->saved_data["scale"] = reduction == 2 ? 1.0 / static_cast<double>(joint.size(0)) : 1.0;
            ctx->saved_data["average_frames"] = average_frames;
        }
        return std::get<0>(out);
    }

    static tensor_list backward(AutogradContext *ctx, tensor_list grad_outputs) {
        const auto saved = ctx->get_saved_variables();
        const auto sizes = ctx->saved_data["sizes"].toIntVector();
        torch::Tensor dense = ctx->saved_data["dense"].toTensor();
        ctx->saved_data["dense"] = torch::empty({0}, dense.options());
        if (dense.numel() == 0 && sizes[0] * sizes[1] * sizes[2] * sizes[3] > 0)
            dense = dense_zero_fill(ctx->saved_data["like"].toTensor(), sizes[0], sizes[1], sizes[2],
                                    sizes[3]);
        else if (dense.numel() == 0)
            dense = torch::empty(sizes, dense.options());
        dense_patch_lattice(saved[0], saved[1], saved[2], saved[3], upstream(grad_outputs[0]),
                            ctx->saved_data["scale"].toDouble(),
                            ctx->saved_data["average_frames"].toBool(), dense);
        return {dense, torch::Tensor(), torch::Tensor(), torch::Tensor(), torch::Tensor(),
                torch::Tensor(), torch::Tensor(), torch::Tensor()};
    }
};

torch::Tensor ctct_loss_op(const torch::Tensor &joint, const torch::Tensor &labels,
                           const torch::Tensor &frames_lengths, const torch::Tensor &labels_lengths,
                           const int64_t reduction, const bool average_frames,
                           const bool clear_in_forward) {
    const bool requires_grad = joint.requires_grad() && at::GradMode::is_enabled();
    return JointLoss::apply(joint, as_int32(labels), as_int32(frames_lengths),
                            as_int32(labels_lengths), requires_grad, reduction, average_frames,
                            clear_in_forward);
}

class LogitsLoss : public torch::autograd::Function<LogitsLoss> {
   public:
    static torch::Tensor forward(AutogradContext *ctx, const torch::Tensor &logits,
                                 const torch::Tensor &ys, const torch::Tensor &lx,
                                 const torch::Tensor &ly, const bool requires_grad,
                                 const int64_t reduction, const bool average_frames) {
        auto out = ctct_loss_logits_fwd(logits, ys, lx, ly, requires_grad, reduction, average_frames);
        if (requires_grad) {
            ctx->save_for_backward({std::get<1>(out), logits, ys, lx, ly});
            ctx->saved_data["scale"] = reduction == 2 ? 1.0 / static_cast<double>(logits.size(0)) : 1.0;
            ctx->saved_data["average_frames"] = average_frames;
        }
        return std::get<0>(out);
    }

    static tensor_list backward(AutogradContext *ctx, tensor_list grad_outputs) {
        const auto saved = ctx->get_saved_variables();
        auto grad = ctct_loss_logits_bwd(saved[0], saved[1], saved[2], saved[3], saved[4],
                                         upstream(grad_outputs[0]),
                                         ctx->saved_data["scale"].toDouble(),
                                         ctx->saved_data["average_frames"].toBool());
        return {grad, torch::Tensor(), torch::Tensor(), torch::Tensor(), torch::Tensor(),
                torch::Tensor(), torch::Tensor()};
    }
};

torch::Tensor ctct_loss_with_logits_op(const torch::Tensor &logits, const torch::Tensor &labels,
                                       const torch::Tensor &frames_lengths,
                                       const torch::Tensor &labels_lengths, const int64_t reduction,
                                       const bool average_frames) {
    const bool requires_grad = logits.requires_grad() && at::GradMode::is_enabled();
    return LogitsLoss::apply(logits.contiguous(), as_int32(labels), as_int32(frames_lengths),
                             as_int32(labels_lengths), requires_grad, reduction, average_frames);
}

// ctct_simple_loss on the un-gathered f (N,T,V), g (N,U+1,V).
class JoinerLoss : public torch::autograd::Function<JoinerLoss> {
   public:
    static torch::Tensor forward(AutogradContext *ctx, const torch::Tensor &f,
                                 const torch::Tensor &g, const torch::Tensor &ys,
                                 const torch::Tensor &lx, const torch::Tensor &ly,
                                 const bool normalized, const bool track_f, const bool track_g,
                                 const int64_t reduction, const bool average_frames) {
        const bool need_grad = track_f || track_g;
        auto out = ctct_simple_fwd(f, g, ys, lx, ly, normalized, need_grad, reduction, average_frames);
        if (need_grad) {
            // f, g, labels, lengths; the compact gradients; den and what the
            // log-matmul keeps for its backward (normalised variant only)
            tensor_list keep = {f, g, ys, lx, ly, std::get<3>(out), std::get<4>(out)};
            if (normalized) {
                keep.push_back(std::get<1>(out));
                keep.push_back(std::get<5>(out));
                for (const auto &t : std::get<2>(out)) keep.push_back(t);
            }
            ctx->save_for_backward(keep);
            ctx->saved_data["normalized"] = normalized;
            ctx->saved_data["track_f"] = track_f;
            ctx->saved_data["track_g"] = track_g;
            ctx->saved_data["scale"] = reduction == 2 ? 1.0 / static_cast<double>(f.size(0)) : 1.0;
            ctx->saved_data["average_frames"] = average_frames;
        }
        return std::get<0>(out);
    }

    static tensor_list backward(AutogradContext *ctx, tensor_list grad_outputs) {
        const auto s = ctx->get_saved_variables();
        const bool normalized = ctx->saved_data["normalized"].toBool();
        c10::optional<torch::Tensor> den, grad_den;
        std::vector<torch::Tensor> shifted;
        if (normalized) {
            den = s[7];
            grad_den = s[8];
            shifted.assign(s.begin() + 9, s.end());
        }
        auto dense = ctct_simple_bwd(s[0], s[1], den, shifted, s[5], s[6], grad_den, s[2], s[3], s[4],
                                     upstream(grad_outputs[0]),
                                     ctx->saved_data["track_f"].toBool(),
                                     ctx->saved_data["track_g"].toBool(),
                                     ctx->saved_data["scale"].toDouble(),
                                     ctx->saved_data["average_frames"].toBool());
        return {std::get<0>(dense), std::get<1>(dense), torch::Tensor(), torch::Tensor(),
                torch::Tensor(), torch::Tensor(), torch::Tensor(), torch::Tensor(),
                torch::Tensor(), torch::Tensor()};
    }
};

torch::Tensor ctct_simple_loss_op(const torch::Tensor &f, const torch::Tensor &g,
                                  const torch::Tensor &labels, const torch::Tensor &frames_lengths,
                                  const torch::Tensor &labels_lengths, const bool normalized,
                                  const int64_t reduction, const bool average_frames) {
    const bool grad_mode = at::GradMode::is_enabled();
    const bool track_f = f.requires_grad() && grad_mode, track_g = g.requires_grad() && grad_mode;
    auto as_float = [](const torch::Tensor &t) {
        return (t.scalar_type() == at::ScalarType::Float && t.is_contiguous())
                   ? t
                   : t.to(at::ScalarType::Float).contiguous();
    };
    return JoinerLoss::apply(as_float(f), as_float(g), as_int32(labels), as_int32(frames_lengths),
                             as_int32(labels_lengths), normalized, track_f, track_g, reduction,
                             average_frames);
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
    m.def("ctct_loss", &ctct_loss_op,
          "warp_ctct.ctct_loss: the un-gathered joint in, the reduced loss out, differentiable.",
          pybind11::arg("log_probs"), pybind11::arg("labels"), pybind11::arg("frames_lengths"),
          pybind11::arg("labels_lengths"), pybind11::arg("reduction"),
          pybind11::arg("average_frames"), pybind11::arg("clear_in_forward"));
    m.def("ctct_loss_with_logits", &ctct_loss_with_logits_op,
          "ctct_loss(logits.log_softmax(-1), ...) in one pass over the logits, differentiable.",
          pybind11::arg("logits"), pybind11::arg("labels"), pybind11::arg("frames_lengths"),
          pybind11::arg("labels_lengths"), pybind11::arg("reduction"),
          pybind11::arg("average_frames"));
    m.def("ctct_simple_loss", &ctct_simple_loss_op,
          "warp_ctct.ctct_simple_loss on un-gathered f and g: the reduced loss, differentiable.",
          pybind11::arg("f"), pybind11::arg("g"), pybind11::arg("labels"),
          pybind11::arg("frames_lengths"), pybind11::arg("labels_lengths"),
          pybind11::arg("normalized"), pybind11::arg("reduction") = 0,
          pybind11::arg("average_frames") = false);
    m.def("ctct_loss_fwd", &ctct_loss_fwd, "CTC-Transducer loss on gathered units (forward).",
          pybind11::arg("log_probs"), pybind11::arg("ys"), pybind11::arg("lx"),
          pybind11::arg("ly"), pybind11::arg("requires_grad"));
    m.def("ctct_loss_joint_fwd", &ctct_loss_joint_fwd,
          "CTC-Transducer loss on the un-gathered joint (forward).", pybind11::arg("log_probs"),
          pybind11::arg("ys"), pybind11::arg("lx"), pybind11::arg("ly"),
          pybind11::arg("requires_grad"), pybind11::arg("reduction") = 0,
          pybind11::arg("average_frames") = false, pybind11::arg("clear_gradient") = false);
    m.def("ctct_loss_compact_fwd", &ctct_loss_compact_fwd,
          "Costs and compact unit gradients from the un-gathered joint.",
          pybind11::arg("log_probs"), pybind11::arg("ys"), pybind11::arg("lx"),
          pybind11::arg("ly"));
    m.def("ctct_loss_logits_fwd", &ctct_loss_logits_fwd,
          "CTC-Transducer loss on logits, log_softmax inside (forward).", pybind11::arg("logits"),
          pybind11::arg("ys"), pybind11::arg("lx"), pybind11::arg("ly"),
          pybind11::arg("requires_grad"), pybind11::arg("reduction") = 0,
          pybind11::arg("average_frames") = false);
    m.def("ctct_loss_logits_bwd", &ctct_loss_logits_bwd, "Gradient wrt the logits.",
          pybind11::arg("workspace"), pybind11::arg("logits"), pybind11::arg("ys"),
          pybind11::arg("lx"), pybind11::arg("ly"), pybind11::arg("grad_out"),
          pybind11::arg("scale"), pybind11::arg("average_frames"));
    m.def("ctct_loss_joint_bwd", &ctct_loss_joint_bwd,
          "Dense gradient wrt the joint from unit gradients.", pybind11::arg("unit_grads"),
          pybind11::arg("ys"), pybind11::arg("lx"), pybind11::arg("ly"),
          pybind11::arg("grad_out"), pybind11::arg("V"));
    m.def("dense_zero_fill", &dense_zero_fill, "Zero-filled (N,T,U+1,V) gradient tensor.",
          pybind11::arg("like"), pybind11::arg("N"), pybind11::arg("T"), pybind11::arg("U1"),
          pybind11::arg("V"));
    m.def("dense_patch_lattice", &dense_patch_lattice,
          "Write the non-zero entries of the dense gradient from the lattice workspace.",
          pybind11::arg("workspace"), pybind11::arg("ys"), pybind11::arg("lx"),
          pybind11::arg("ly"), pybind11::arg("grad_out"), pybind11::arg("scale"),
          pybind11::arg("average_frames"), pybind11::arg("dense"));
    m.def("ctct_loss_simple_fwd", &ctct_loss_simple_fwd,
          "CTC-Transducer loss with the log-add joiner on gathered operands (forward).",
          pybind11::arg("f"), pybind11::arg("g"), pybind11::arg("ys"), pybind11::arg("den"),
          pybind11::arg("lx"), pybind11::arg("ly"), pybind11::arg("requires_grad"));
    m.def("ctct_simple_fwd", &ctct_simple_fwd,
          "CTC-Transducer loss with the log-add joiner on un-gathered f, g (forward).",
          pybind11::arg("f"), pybind11::arg("g"), pybind11::arg("ys"), pybind11::arg("lx"),
          pybind11::arg("ly"), pybind11::arg("normalized"), pybind11::arg("requires_grad"),
          pybind11::arg("reduction") = 0, pybind11::arg("average_frames") = false);
    m.def("ctct_simple_bwd", &ctct_simple_bwd, "Dense gradients wrt f and g.", pybind11::arg("f"),
          pybind11::arg("g"), pybind11::arg("den"), pybind11::arg("shifted"),
          pybind11::arg("grad_f"),
          pybind11::arg("grad_g"), pybind11::arg("grad_den"), pybind11::arg("ys"),
          pybind11::arg("lx"), pybind11::arg("ly"), pybind11::arg("grad_out"),
          pybind11::arg("want_f"), pybind11::arg("want_g"), pybind11::arg("scale") = 1.0,
          pybind11::arg("average_frames") = false);
    m.def("log_matmul", &log_matmul, "Log matrix multiplication", pybind11::arg("lhs"),
          pybind11::arg("rhs"));
    m.def("log_matmul_backward", &log_matmul_backward, "Log matrix multiplication backward",
          pybind11::arg("grad_out"), pybind11::arg("lhs"), pybind11::arg("rhs"),
          pybind11::arg("res"), pybind11::arg("grad_masks"));
    m.def("library_version", []() { return std::string(warpctct_version()); });
    m.def(
        "joiner_linear_lattice", [](const int from_frames) { return warpctct_joiner_linear_lattice(from_frames); },
        "From how many frames on the fused joiner forward sweeps in the linear domain (0: never, 1: always, "
        "negative: the defaults); returns the previous setting.",
        pybind11::arg("from_frames"));
    m.def(
        "status",
        [](const bool clear) {
            unsigned bits = 0;
            check_rc(warpctct_status(&bits, clear ? 1 : 0), "status");
            return static_cast<int64_t>(bits);
        },
        "Sticky status bits of the current device (synchronises with it).",
        pybind11::arg("clear") = true);
}
