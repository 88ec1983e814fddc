"""Every stage entry point of the C ABI called directly (ctypes, device
pointers) and compared with the float64 oracle: the dense-gradient pair that
works from ready-made unit gradients, the stages of the log-add joiner path
(units from gathered and from un-gathered operands, reductions, scatter), the
scaling of already gathered units, and the *_f32 forms of the orchestrators.

Tolerances: gathered / summed inputs exact where the kernel only moves or
adds float64 values, loss relative error <= 1e-5, gradient absolute error
<= 1e-4 (scaled by the largest upstream weight)."""
import ctypes

import numpy as np
import pytest
import torch

import hip_lib
from ctct_cases import make_joint_case, make_simple_case
from oracle import ctct_oracle as O

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
GRAD_ATOL = 1e-4
LOG2E = np.float64(1.4426950408889634074)


def dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def nan_like(*shape, dtype=torch.float32):
    return torch.full(shape, float("nan"), dtype=dtype, device="cuda")


DENSE_CASES = [
    # name, seed, N, T, U, V, lx, ly
    ("odd_vocab_element_stores", 201, 3, 17, 5, 37, [17, 9, 12], [5, 2, 4]),
    ("line_sized_rows", 202, 2, 14, 8, 96, [14, 12], [8, 7]),
    ("vocab_1024", 203, 2, 21, 6, 1024, [21, 13], [6, 3]),
]


@pytest.mark.parametrize("case", DENSE_CASES, ids=[c[0] for c in DENSE_CASES])
def test_dense_gradient_from_unit_gradients(case):
    """warpctct_dense_grad_f32, warpctct_zero_fill_f32 + warpctct_dense_patch_f32
    and _C.ctct_loss_joint_bwd: zeros + grad_out[n] * unit gradient at columns
    0, y[u-1], y[u]; a repeated label (two units in one column) and a label
    equal to the blank index (a unit in column 0) must add."""
    from warp_ctct import _C
    lib = hip_lib.lib()
    _, seed, N, T, U, V, lx, ly = case
    joint, ys, lx, ly = make_joint_case(seed, N, T, U, V, lx=lx, ly=ly, force_repeat=False)
    ys[0, 1] = ys[0, 0]                      # coincident columns y[u-1] == y[u] at u = 1
    ys[1, 0] = 0                             # a label on the blank's column
    if V > 64:
        ys[0, 3] = V - 1                     # last column of the row
        ys[1, 1] = 33                        # second 128-byte line of a float row
    lx = np.maximum(lx, ly + 1).astype(np.int32)
    lp3 = O.gather_units(joint, ys)
    _, ug = O.ctct_loss_fwd(lp3, ys, lx, ly)
    ug32 = ug.astype(np.float32)
    w = np.random.default_rng(seed).standard_normal(N).astype(np.float32)
    ref = O.scatter_units(ug32.astype(np.float64) * w.astype(np.float64)[:, None, None, None], ys, V)
    assert np.any(ref[0, :, 1, ys[0, 0]] != 0) and np.any(ref[1, :, 1, 0] != 0)
    p, s = hip_lib.ptr, hip_lib.stream_ptr()
    d_ug, d_ys, d_lx, d_ly, d_w = dev(ug32), dev(ys), dev(lx), dev(ly), dev(w)
    scale = max(1.0, float(np.abs(w).max()))

    def check(dense, what):
        got = dense.cpu().numpy().astype(np.float64)
        np.testing.assert_allclose(got, ref, atol=1e-6 * scale, rtol=1e-6, err_msg=what)
        assert np.all(got[ref == 0] == 0), what + ": non-zero where the oracle has a structural zero"

    dense = nan_like(N, T, U + 1, V)
    hip_lib.check(lib.warpctct_dense_grad_f32(p(d_ug), p(d_ys), p(d_lx), p(d_ly), p(d_w), p(dense),
                                              N, T, U, V, s))
    torch.cuda.synchronize()
    check(dense, "warpctct_dense_grad_f32")
    # the two halves on their own
    dense2 = nan_like(N, T, U + 1, V)
    hip_lib.check(lib.warpctct_zero_fill_f32(p(dense2), ctypes.c_size_t(dense2.numel()), s))
    torch.cuda.synchronize()
    assert bool((dense2 == 0).all())
    hip_lib.check(lib.warpctct_dense_patch_f32(p(d_ug), p(d_ys), p(d_lx), p(d_ly), p(d_w),
                                               p(dense2), N, T, U, V, s))
    torch.cuda.synchronize()
    check(dense2, "warpctct_zero_fill_f32 + warpctct_dense_patch_f32")
    # grad_out NULL = ones
    dense3 = nan_like(N, T, U + 1, V)
    hip_lib.check(lib.warpctct_dense_grad_f32(p(d_ug), p(d_ys), p(d_lx), p(d_ly), p(None),
                                              p(dense3), N, T, U, V, s))
    torch.cuda.synchronize()
    ones = O.scatter_units(ug32.astype(np.float64), ys, V)
    np.testing.assert_allclose(dense3.cpu().numpy(), ones, atol=1e-6, rtol=1e-6)
    # the torch operator over the same entry point
    check(_C.ctct_loss_joint_bwd(d_ug, d_ys, d_lx, d_ly, d_w, V), "_C.ctct_loss_joint_bwd")
    # a tensor that does not start on a 128-byte boundary takes the element-wise stores
    if (V * 4) % 128 == 0:
        raw = nan_like(N * T * (U + 1) * V + 4)
        off = raw[1:1 + N * T * (U + 1) * V]
        assert off.data_ptr() % 128 != 0
        hip_lib.check(lib.warpctct_dense_grad_f32(p(d_ug), p(d_ys), p(d_lx), p(d_ly), p(d_w),
                                                  p(off), N, T, U, V, s))
        torch.cuda.synchronize()
        check(off.view(N, T, U + 1, V), "warpctct_dense_grad_f32, unaligned tensor")
        assert torch.isnan(raw[0]) and bool(torch.isnan(raw[1 + N * T * (U + 1) * V:]).all())


def test_scale_units_and_orchestrators_in_float32_form():
    """warpctct_scale_units_f32 (already gathered natural-log units -> work
    buffer), then warpctct_loss_lattice_f32, warpctct_dense_grad_lattice_f32 and
    warpctct_zero_fill + warpctct_dense_patch_lattice_f32 against the oracle."""
    lib = hip_lib.lib()
    N, T, U, V = 3, 19, 6, 40
    joint, ys, lx, ly = make_joint_case(211, N, T, U, V, lx=[19, 11, 14], ly=[6, 3, 5])
    p, s = hip_lib.ptr, hip_lib.stream_ptr()
    P = lib.warpctct_padded_contexts(U)
    lp3 = O.gather_units(joint, ys).astype(np.float32)
    units = nan_like(N, T, P, 3, dtype=torch.float64)
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    d_lp3 = dev(lp3)                          # (kept alive until the kernel has run)
    hip_lib.check(lib.warpctct_scale_units_f32(p(d_lp3), p(d_lx), p(d_ly), p(units), N, T, U, s))
    torch.cuda.synchronize()
    got = units.cpu().numpy()
    for n in range(N):
        t, u = int(lx[n]), int(ly[n])
        exp = lp3[n, :t, :u + 1].astype(np.float64) * LOG2E
        np.testing.assert_array_equal(got[n, :t, :u + 1, :2], exp[..., :2])
        np.testing.assert_array_equal(got[n, :t, :u, 2], exp[:, :u, 2])
        assert np.all(np.isneginf(got[n, :t, u, 2]))
        assert np.all(got[n, :t, u + 1:, :2] == 0) and np.all(np.isneginf(got[n, :t, u + 1:, 2]))
        assert np.all(np.isnan(got[n, t:]))
    # orchestrators, float32 form
    w = np.array([0.5, -1.5, 2.0], np.float32)
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="none", grad_output=w)
    need = lib.warpctct_workspace_bytes(N, T, U)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    costs = nan_like(N)
    d_joint, d_w = dev(joint), dev(w)
    hip_lib.check(lib.warpctct_loss_lattice_f32(p(d_joint), p(d_ys), p(d_lx), p(d_ly), N, T, U, V,
                                                p(ws), ctypes.c_size_t(need), p(costs), 1, s))
    torch.cuda.synchronize()
    np.testing.assert_allclose(costs.cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
    one = ctypes.c_float(1.0)
    dense = nan_like(N, T, U + 1, V)
    hip_lib.check(lib.warpctct_dense_grad_lattice_f32(p(ws), ctypes.c_size_t(need), p(d_ys), p(d_lx),
                                                      p(d_ly), p(d_w), 1, one, 0, p(dense), N, T, U,
                                                      V, s))
    torch.cuda.synchronize()
    np.testing.assert_allclose(dense.cpu().numpy(), ref_dense, atol=GRAD_ATOL * 2, rtol=0)
    assert np.all(dense.cpu().numpy()[ref_dense == 0] == 0)
    dense2 = nan_like(N, T, U + 1, V)
    hip_lib.check(lib.warpctct_zero_fill(p(dense2), ctypes.c_size_t(dense2.numel() * 4), s))
    hip_lib.check(lib.warpctct_dense_patch_lattice_f32(p(ws), ctypes.c_size_t(need), p(d_ys),
                                                       p(d_lx), p(d_ly), p(d_w), 1, one, 0,
                                                       p(dense2), N, T, U, V, s))
    torch.cuda.synchronize()
    assert torch.equal(dense2, dense)
    # beta-only mode (want_alpha = 0): same costs
    costs2 = nan_like(N)
    hip_lib.check(lib.warpctct_loss_lattice_f32(p(d_joint), p(d_ys), p(d_lx), p(d_ly), N, T, U, V,
                                                p(ws), ctypes.c_size_t(need), p(costs2), 0, s))
    torch.cuda.synchronize()
    assert torch.equal(costs2, costs)


def test_forward_that_clears_the_gradient_buffer_beside_the_lattices():
    """warpctct_loss_lattice_clearing + warpctct_dense_patch_lattice against
    warpctct_loss_lattice + warpctct_dense_grad_lattice: same costs and the same
    dense gradient bit for bit, on a buffer that held NaNs, for a narrow and for
    a two-wavefront lattice, with and without a buffer to clear, for a strided
    joint."""
    lib = hip_lib.lib()
    p, s = hip_lib.ptr, hip_lib.stream_ptr()
    one = ctypes.c_float(1.0)
    for seed, N, T, U, V, lx, ly in [(231, 4, 37, 9, 1024, [37, 20, 31, 9], [9, 4, 7, 1]),
                                     (232, 2, 21, 70, 48, [21, 15], [70, 33])]:
        joint, ys, lx, ly = make_joint_case(seed, N, T, U, V, lx=lx, ly=ly)
        w = np.random.default_rng(seed).standard_normal(N).astype(np.float32)
        _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="none", grad_output=w)
        need = lib.warpctct_workspace_bytes(N, T, U)
        d_ys, d_lx, d_ly, d_w = dev(ys), dev(lx), dev(ly), dev(w)
        # the joint stored as (N, U+1, T, V): the entry point sees it through strides
        stored = dev(np.ascontiguousarray(joint.transpose(0, 2, 1, 3)))
        view = stored.transpose(1, 2)
        strides = (ctypes.c_long * 4)(*view.stride())
        ws_a = torch.empty(need, dtype=torch.uint8, device="cuda")
        ws_b = torch.empty(need, dtype=torch.uint8, device="cuda")
        costs_a, costs_b, costs_c = nan_like(N), nan_like(N), nan_like(N)
        dense_a, dense_b = nan_like(N, T, U + 1, V), nan_like(N, T, U + 1, V)
        nbytes = ctypes.c_size_t(dense_a.numel() * 4)
        hip_lib.check(lib.warpctct_loss_lattice_strided(p(stored), 0, strides, p(d_ys), p(d_lx),
                                                        p(d_ly), N, T, U, V, p(ws_a),
                                                        ctypes.c_size_t(need), p(costs_a), 1, 0, 0,
                                                        None, s))
        hip_lib.check(lib.warpctct_dense_grad_lattice(p(ws_a), ctypes.c_size_t(need), p(d_ys),
                                                      p(d_lx), p(d_ly), p(d_w), 1, one, 0,
                                                      p(dense_a), 0, N, T, U, V, s))
        hip_lib.check(lib.warpctct_loss_lattice_clearing(p(stored), 0, strides, p(d_ys), p(d_lx),
                                                         p(d_ly), N, T, U, V, p(ws_b),
                                                         ctypes.c_size_t(need), p(costs_b), 1, 0, 0,
                                                         None, p(dense_b), nbytes, s))
        # work queued on the caller's stream afterwards sees the cleared buffer
        cleared = dense_b.clone()
        hip_lib.check(lib.warpctct_dense_patch_lattice(p(ws_b), ctypes.c_size_t(need), p(d_ys),
                                                       p(d_lx), p(d_ly), p(d_w), 1, one, 0,
                                                       p(dense_b), 0, N, T, U, V, s))
        # nothing to clear: the plain forward
        hip_lib.check(lib.warpctct_loss_lattice_clearing(p(stored), 0, strides, p(d_ys), p(d_lx),
                                                         p(d_ly), N, T, U, V, p(ws_b),
                                                         ctypes.c_size_t(need), p(costs_c), 1, 0, 0,
                                                         None, None, ctypes.c_size_t(0), s))
        torch.cuda.synchronize()
        assert torch.count_nonzero(cleared).item() == 0 and not torch.isnan(cleared).any()
        assert torch.equal(costs_b, costs_a) and torch.equal(costs_c, costs_a)
        assert torch.equal(dense_b, dense_a)
        np.testing.assert_allclose(costs_b.cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
        scale = max(1.0, float(np.abs(w).max()))
        np.testing.assert_allclose(dense_b.cpu().numpy(), ref_dense, atol=GRAD_ATOL * scale, rtol=0)


SIMPLE_STAGE_CASES = [
    # name, seed, N, T, U, V, lx, ly, normalized
    ("normalized", 221, 3, 23, 7, 29, [23, 12, 17], [7, 3, 5], True),
    ("unnormalized", 222, 3, 23, 7, 29, [23, 12, 17], [7, 3, 5], False),
    ("two_wavefronts", 223, 2, 110, 80, 21, [110, 97], [80, 71], True),
]


@pytest.mark.parametrize("case", SIMPLE_STAGE_CASES, ids=[c[0] for c in SIMPLE_STAGE_CASES])
def test_log_add_joiner_stages(case):
    """The joiner path stage by stage: units from gathered operands
    (warpctct_simple_units_f32) and from un-gathered ones
    (warpctct_simple_gather_units_f32), lattice + unit gradients on them,
    warpctct_simple_reduce_f32 and warpctct_simple_scatter_f32."""
    lib = hip_lib.lib()
    _, seed, N, T, U, V, lx, ly, normalized = case
    f, g, ys, lx, ly = make_simple_case(seed, N, T, U, V, lx=lx, ly=ly, normalized=normalized)
    U1 = U + 1
    f_g, g_g = O.gather_separate(f, g, ys)
    den = O.log_matmul(f, np.swapaxes(g, 1, 2)).astype(np.float32) if normalized else None
    lp3 = O.simple_units(f_g, g_g, den)                      # float64, natural log
    p, s = hip_lib.ptr, hip_lib.stream_ptr()
    P = lib.warpctct_padded_contexts(U)
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    d_den = dev(den) if normalized else None

    def check_units(units, band_only, what):
        got = units.cpu().numpy()
        for n in range(N):
            t, u = int(lx[n]), int(ly[n])
            exp = lp3[n, :t, :u + 1] * LOG2E
            tt, uu = np.meshgrid(np.arange(t), np.arange(u + 1), indexing="ij")
            inside = (tt >= uu) & (t - tt >= u - uu) if band_only else np.ones_like(tt, bool)
            x = got[n, :t, :u + 1]
            np.testing.assert_allclose(x[..., 0][inside], exp[..., 0][inside], rtol=1e-14, atol=0,
                                       err_msg=what)
            m1 = inside & (uu >= 1)
            np.testing.assert_allclose(x[..., 1][m1], exp[..., 1][m1], rtol=1e-14, atol=0, err_msg=what)
            m2 = inside & (uu < u)
            np.testing.assert_allclose(x[..., 2][m2], exp[..., 2][m2], rtol=1e-14, atol=0, err_msg=what)
            assert np.all(np.isneginf(x[:, u, 2])), what
            # cells that no complete alignment reaches and padding contexts: neutral units
            out = ~inside
            assert np.all(x[..., 0][out] == 0) and np.all(np.isneginf(x[..., 2][out])), what
            pad = got[n, :t, u + 1:]
            assert np.all(pad[..., :2] == 0) and np.all(np.isneginf(pad[..., 2])), what
            assert np.all(np.isnan(got[n, t:])), what

    units_a = nan_like(N, T, P, 3, dtype=torch.float64)
    d_fg, d_gg = dev(f_g), dev(g_g)
    hip_lib.check(lib.warpctct_simple_units_f32(p(d_fg), p(d_gg), p(d_den), p(d_lx), p(d_ly),
                                                p(units_a), N, T, U, s))
    units_b = nan_like(N, T, P, 3, dtype=torch.float64)
    d_f, d_g = dev(f), dev(g)
    hip_lib.check(lib.warpctct_simple_gather_units_f32(p(d_f), p(d_g), p(d_den), p(d_ys), p(d_lx),
                                                       p(d_ly), p(units_b), N, T, U, V, s))
    torch.cuda.synchronize()
    check_units(units_a, False, "warpctct_simple_units_f32")
    check_units(units_b, True, "warpctct_simple_gather_units_f32")

    # lattice + unit gradients on either set of units: same costs and gradients
    costs_ref, ug_ref = O.ctct_loss_fwd(lp3, ys, lx, ly)
    results = []
    for units in (units_a, units_b):
        alphas = nan_like(N, T + 1, P, 2, dtype=torch.float64)
        betas = nan_like(N, T + 1, P, 2, dtype=torch.float64)
        costs = nan_like(N)
        ug = nan_like(N, T, U1, 3)
        lib.warpctct_lattice_relay_bytes.restype = ctypes.c_size_t
        relay_bytes = lib.warpctct_lattice_relay_bytes(N, T, U)
        relay = torch.empty(max(relay_bytes, 8), dtype=torch.uint8, device="cuda")
        hip_lib.check(lib.warpctct_lattice_f32(p(units), p(d_ys), p(d_lx), p(d_ly), p(alphas),
                                               p(betas), p(costs), N, T, U, 0, p(relay),
                                               ctypes.c_size_t(relay_bytes), s))
        hip_lib.check(lib.warpctct_unit_grads_f32(p(units), p(d_ys), p(d_lx), p(d_ly), p(alphas),
                                                  p(betas), p(ug), N, T, U, s))
        torch.cuda.synchronize()
        np.testing.assert_allclose(costs.cpu().numpy(), costs_ref, rtol=LOSS_RTOL)
        np.testing.assert_allclose(ug.cpu().numpy(), ug_ref, atol=GRAD_ATOL, rtol=0)
        assert np.all(ug.cpu().numpy()[ug_ref == 0] == 0)
        results.append(ug)

    # reductions of the unit gradients (csrc/binding.cpp:198-219 of the reference)
    ug = results[0]
    ug64 = ug.cpu().numpy().astype(np.float64)
    gf_ref, gg_ref, gd_ref = O.simple_unit_grad_reduce(ug64, normalized)
    grad_f, grad_g = nan_like(N, T, U1), nan_like(N, U1, 3)
    grad_den = nan_like(N, T, U1) if normalized else None
    hip_lib.check(lib.warpctct_simple_reduce_f32(p(ug), p(grad_f), p(grad_g), p(grad_den), N, T, U, s))
    torch.cuda.synchronize()
    np.testing.assert_allclose(grad_f.cpu().numpy(), gf_ref, atol=1e-6, rtol=1e-6)
    np.testing.assert_allclose(grad_g.cpu().numpy(), gg_ref, atol=2e-6, rtol=1e-5)
    if normalized:
        np.testing.assert_allclose(grad_den.cpu().numpy(), gd_ref, atol=1e-6, rtol=1e-6)

    # backward of the two gathers: scatter-add, scaled per sample
    w = np.linspace(-1.0, 2.0, N).astype(np.float32)
    gf32, gg32 = grad_f.cpu().numpy().astype(np.float64), grad_g.cpu().numpy().astype(np.float64)
    exp_f = np.zeros((N, T, V))
    exp_g = np.zeros((N, U1, V))
    gi = O.gather_index(ys, U1)
    for n in range(N):
        cols = np.concatenate([[0], ys[n]])
        for t in range(int(lx[n])):
            np.add.at(exp_f[n, t], cols[:ly[n] + 1], gf32[n, t, :ly[n] + 1] * w[n])
        for u in range(int(ly[n]) + 1):
            ks = [0] + ([1] if u >= 1 else []) + ([2] if u < ly[n] else [])
            np.add.at(exp_g[n, u], gi[n, u, ks], gg32[n, u, ks] * w[n])
    dense_f = torch.zeros(N, T, V, device="cuda")
    dense_g = torch.zeros(N, U1, V, device="cuda")
    d_w = dev(w)
    hip_lib.check(lib.warpctct_simple_scatter_f32(p(grad_f), p(grad_g), p(d_ys), p(d_lx), p(d_ly),
                                                  p(d_w), p(dense_f), p(dense_g), N, T, U, V, s))
    torch.cuda.synchronize()
    np.testing.assert_allclose(dense_f.cpu().numpy(), exp_f, atol=2e-6, rtol=1e-5)
    np.testing.assert_allclose(dense_g.cpu().numpy(), exp_g, atol=2e-6, rtol=1e-5)
    # either output alone
    only_g = torch.zeros(N, U1, V, device="cuda")
    hip_lib.check(lib.warpctct_simple_scatter_f32(p(None), p(grad_g), p(d_ys), p(d_lx), p(d_ly),
                                                  p(None), p(None), p(only_g), N, T, U, V, s))
    torch.cuda.synchronize()
    np.testing.assert_allclose(only_g.cpu().numpy(), _scatter_g(gg32, gi, ly, np.ones(N), U1, V),
                               atol=2e-6, rtol=1e-5)


FUSED_JOINER_CASES = [
    # name, seed, N, T, U, V, lx, ly, normalized
    ("normalized", 231, 3, 23, 7, 29, [23, 12, 17], [7, 3, 5], True),
    ("unnormalized", 232, 3, 23, 7, 29, [23, 12, 17], [7, 3, 5], False),
    ("matrix_core_kernels", 233, 2, 136, 20, 512, [136, 129], [20, 11], True),
    ("chain_of_workgroups", 234, 2, 90, 70, 40, [90, 77], [70, 64], False),
]


@pytest.mark.parametrize("case", FUSED_JOINER_CASES, ids=[c[0] for c in FUSED_JOINER_CASES])
@pytest.mark.parametrize("reduction,average_frames", [(0, 0), (1, 1), (2, 0), (2, 1)])
def test_fused_joiner_entry_points_with_reduction(case, reduction, average_frames):
    """warpctct_simple_forward_reduced_f32 and warpctct_simple_backward_weighted_f32 called
    directly: un-gathered f and g in, costs / reduced loss out, dense gradients
    for an upstream gradient that is one scalar (sum, mean) or one value per
    sample (no reduction), against the float64 oracle."""
    lib = hip_lib.lib()
    _, seed, N, T, U, V, lx, ly, normalized = case
    f, g, ys, lx, ly = make_simple_case(seed, N, T, U, V, lx=lx, ly=ly, normalized=normalized)
    U1 = U + 1
    p, s = hip_lib.ptr, hip_lib.stream_ptr()
    for fn in ("warpctct_simple_workspace_bytes", "warpctct_simple_backward_workspace_bytes"):
        getattr(lib, fn).restype = ctypes.c_size_t
    Vp = lib.warpctct_logmm_padded_reduction(V)
    d_f, d_g, d_ys, d_lx, d_ly = dev(f), dev(g), dev(ys), dev(lx), dev(ly)
    ws = torch.empty(lib.warpctct_simple_workspace_bytes(N, T, U), dtype=torch.uint8, device="cuda")
    den = nan_like(N, T, U1) if normalized else None
    fmax = nan_like(N, T) if normalized else None
    gmax = nan_like(N, U1) if normalized else None
    keeps = lib.warpctct_simple_needs_fexp(p(d_f), T, U, V) != 0
    fexp = nan_like(N, T, Vp) if normalized and keeps else None
    gexp = nan_like(N, U1, Vp) if normalized else None
    costs, reduced = nan_like(N), nan_like(1)
    grad_f, grad_g = nan_like(N, T, U1), nan_like(N, U1, 3)
    grad_den = nan_like(N, T, U1) if normalized else None
    hip_lib.check(lib.warpctct_simple_forward_reduced_f32(
        p(d_f), p(d_g), p(d_ys), p(d_lx), p(d_ly), N, T, U, V, int(normalized), p(ws),
        ctypes.c_size_t(ws.numel()), p(den), p(fmax), p(gmax), p(fexp), p(gexp), p(costs),
        p(grad_f), p(grad_g), p(grad_den), reduction, average_frames,
        p(reduced) if reduction else p(None), s))
    torch.cuda.synchronize()

    rng = np.random.default_rng(seed)
    up = rng.uniform(-1.5, 2.0, size=N if reduction == 0 else 1).astype(np.float32)
    per_sample = np.broadcast_to(up, (N,)).astype(np.float64)
    if average_frames:
        per_sample = per_sample / lx
    if reduction == 2:
        per_sample = per_sample / N
    name = {0: "none", 1: "sum", 2: "mean"}[reduction]
    loss, gf, gg, costs_ref = O.ctct_simple_loss(f, g, ys, lx, ly, reduction=name,
                                                 average_frames=bool(average_frames),
                                                 normalized=normalized, grad_output=per_sample)
    per_cost = costs_ref / lx if average_frames else costs_ref
    np.testing.assert_allclose(costs.cpu().numpy(), per_cost, rtol=LOSS_RTOL)
    if reduction:
        np.testing.assert_allclose(float(reduced.cpu()), loss, rtol=LOSS_RTOL)
    else:
        assert np.isnan(float(reduced.cpu()))   # untouched

    bws = torch.empty(max(lib.warpctct_simple_backward_workspace_bytes(N, T, U), 8),
                      dtype=torch.uint8, device="cuda")
    dense_f, dense_g = nan_like(N, T, V), nan_like(N, U1, V)
    weights = nan_like(N)
    d_up = dev(up)
    scale = ctypes.c_float(1.0 / N if reduction == 2 else 1.0)

    def backward(grad_out, stride, scale_arg, avg, weights_arg):
        return lib.warpctct_simple_backward_weighted_f32(
            p(d_f), p(d_g), p(den), p(fmax), p(gmax), p(fexp), p(gexp), p(grad_f), p(grad_g),
            p(grad_den), p(d_ys), p(d_lx), p(d_ly), p(grad_out), stride, scale_arg, avg,
            p(weights_arg), N, T, U, V, p(bws), ctypes.c_size_t(bws.numel()), p(dense_f), p(dense_g), s)

    hip_lib.check(backward(d_up, 1 if reduction == 0 else 0, scale, average_frames, weights))
    torch.cuda.synchronize()
    np.testing.assert_allclose(dense_f.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(dense_g.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)
    # arguments (1 = WARPCTCT_EINVAL): a stride other than 0 or 1, no scratch where the
    # weights need one, a reduction that does not exist, a reduction without its output
    assert backward(d_up, 2, scale, average_frames, weights) == 1
    if normalized and (reduction != 0 or average_frames):
        assert backward(d_up, 1 if reduction == 0 else 0, scale, average_frames, None) == 1
    assert lib.warpctct_simple_forward_reduced_f32(
        p(d_f), p(d_g), p(d_ys), p(d_lx), p(d_ly), N, T, U, V, int(normalized), p(ws),
        ctypes.c_size_t(ws.numel()), p(den), p(fmax), p(gmax), p(fexp), p(gexp), p(costs),
        p(grad_f), p(grad_g), p(grad_den), 3, 0, p(reduced), s) == 1
    assert lib.warpctct_simple_forward_reduced_f32(
        p(d_f), p(d_g), p(d_ys), p(d_lx), p(d_ly), N, T, U, V, int(normalized), p(ws),
        ctypes.c_size_t(ws.numel()), p(den), p(fmax), p(gmax), p(fexp), p(gexp), p(costs),
        p(grad_f), p(grad_g), p(grad_den), 1, 0, p(None), s) == 1


def _scatter_g(gg, gi, ly, w, U1, V):
    N = gg.shape[0]
    out = np.zeros((N, U1, V))
    for n in range(N):
        for u in range(int(ly[n]) + 1):
            ks = [0] + ([1] if u >= 1 else []) + ([2] if u < ly[n] else [])
            np.add.at(out[n, u], gi[n, u, ks], gg[n, u, ks] * w[n])
    return out
