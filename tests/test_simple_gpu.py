"""GPU parity tests of the log-add joiner path: log-semiring matmul (forward
and backward), the reference's _C.ctct_loss_simple_fwd surface, and the public
ctct_simple_loss with its autograd, against the float64 oracle.

Tolerances: loss relative error <= 1e-5, gradient absolute error <= 1e-4."""
import numpy as np
import pytest
import torch

from ctct_cases import make_joint_case, make_simple_case
from oracle import c_oracle as C
from oracle import ctct_oracle as O

import hip_lib

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
GRAD_ATOL = 1e-4


@pytest.fixture(autouse=True, params=["log_lattices", "linear_lattices"])
def lattice_domain(request):
    """Every test of this file runs twice: with the joiner's lattices swept in the
    log domain only, and with the linear sweeps (checked, with the log domain as
    their fall-back) used for every input, not just for long ones."""
    import warp_ctct
    lib = hip_lib.lib()
    before = lib.warpctct_joiner_linear_lattice(1 if request.param == "linear_lattices" else 0)
    warp_ctct.status(reset=True)
    yield request.param
    lib.warpctct_joiner_linear_lattice(before)
    # the linear sweeps must hold on their own: a test whose input is meant to
    # send them back to the log domain says so (the fall-back would hide a
    # mistake in them from every comparison with the oracle)
    fell_back = warp_ctct.status(reset=True) & warp_ctct.STATUS_LINEAR_FELL_BACK
    if request.node.get_closest_marker("may_fall_back") is None:
        assert not fell_back, "the linear lattices were given up on input that they should take"


def dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


# ------------------------------------------------------------------ log matmul
@pytest.mark.parametrize("B,M,K,Nn", [
    (1, 1, 1, 1), (2, 5, 7, 3), (3, 70, 100, 33), (2, 130, 257, 81),
    # long reductions: the form that keeps a slab of the right operand in LDS
    # (512 <= K rounded up to 32 <= 2048): whole and partial slabs, one to three
    # column tiles, fewer rows than a row block and a ragged last block
    (2, 37, 512, 81), (1, 130, 777, 100), (2, 21, 2048, 200), (1, 5, 1500, 3), (3, 16, 1024, 64),
    # and just beyond it
    (1, 9, 2049, 7)])
@pytest.mark.parametrize("layout", ["contiguous", "transposed_view"])
def test_log_matmul_forward(B, M, K, Nn, layout):
    from warp_ctct import _C
    rng = np.random.default_rng(B * 1000 + M)
    lhs = (rng.standard_normal((B, M, K)) * 3).astype(np.float32)
    rhs = (rng.standard_normal((B, K, Nn)) * 3).astype(np.float32)
    ref = C.log_matmul(lhs, rhs)
    d_lhs = dev(lhs)
    if layout == "contiguous":
        d_rhs = dev(rhs)
    else:   # what ctct_simple_loss passes: g (B,Nn,K) viewed as (B,K,Nn)
        d_rhs = dev(np.ascontiguousarray(rhs.transpose(0, 2, 1))).transpose(1, 2)
        assert not d_rhs.is_contiguous() or K == 1 or Nn == 1
    out = _C.log_matmul(d_lhs, d_rhs)
    assert out.shape == (B, M, Nn) and out.is_contiguous()
    np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=1e-5, atol=1e-5)


def test_log_matmul_infinities_and_far_apart_maxima():
    from warp_ctct import _C
    rng = np.random.default_rng(3)
    B, M, K, Nn = 2, 9, 40, 6
    lhs = rng.standard_normal((B, M, K)).astype(np.float32)
    rhs = rng.standard_normal((B, K, Nn)).astype(np.float32)
    lhs[0, 1, :] = -np.inf            # whole row -inf -> -inf outputs
    rhs[1, :, 2] = -np.inf            # whole column -inf
    lhs[0, 3, 5:] = -np.inf           # partly -inf
    # row maximum at k=0, column maximum at k=7, 300 apart: the shifted sum
    # underflows and the exact path must take over
    lhs[1, 4, 0] = 300.0
    rhs[1, 7, 4] = 300.0
    ref = C.log_matmul(lhs, rhs)
    out = _C.log_matmul(dev(lhs), dev(rhs)).cpu().numpy()
    assert np.all(np.isneginf(out[0, 1])) and np.all(np.isneginf(out[1, :, 2]))
    assert np.array_equal(np.isneginf(out), np.isneginf(ref))
    fin = np.isfinite(ref)
    np.testing.assert_allclose(out[fin], ref[fin], rtol=1e-5, atol=1e-5)
    assert abs(out[1, 4, 4] - ref[1, 4, 4]) < 1e-3 and ref[1, 4, 4] > 290
    # backward over the same operands: -inf rows have no gradient, and the pair
    # (4,4) whose maxima are 300 apart takes the exact per-term path
    go = rng.standard_normal((B, M, Nn)).astype(np.float32)
    gl, gr = O.log_matmul_backward(go, lhs, rhs, ref)
    d_lhs, d_rhs = dev(lhs), dev(rhs)
    d_res = _C.log_matmul(d_lhs, d_rhs)
    out_l, out_r = _C.log_matmul_backward(dev(go), d_lhs, d_rhs, d_res, [True, True])
    np.testing.assert_allclose(out_l.cpu().numpy(), gl, atol=2e-5, rtol=1e-4)
    np.testing.assert_allclose(out_r.cpu().numpy(), gr, atol=2e-5, rtol=1e-4)
    assert abs(gl[1, 4, 0]) + abs(gl[1, 4, 7]) > 1e-3      # the far-apart pair carries gradient


def test_log_matmul_far_apart_maxima_in_a_long_reduction():
    """The pairs left to the exact per-term pass, in the shapes that take the
    slab-resident kernels (reduction of 512, whole and ragged row blocks)."""
    from warp_ctct import _C
    rng = np.random.default_rng(5)
    for B, M, K, Nn in ((2, 32, 512, 40), (1, 21, 300, 9), (2, 140, 512, 40)):
        lhs = rng.standard_normal((B, M, K)).astype(np.float32)
        rhs = rng.standard_normal((B, K, Nn)).astype(np.float32)
        lhs[0, 4, 0] = 300.0              # row maximum at k = 0
        rhs[0, 7, 3] = 300.0              # column maximum at k = 7: pair (4, 3) underflows
        lhs[B - 1, M - 1, K - 1] = 250.0
        rhs[B - 1, 2, Nn - 1] = 250.0
        ref = C.log_matmul(lhs, rhs)
        d_lhs, d_rhs = dev(lhs), dev(rhs)
        d_res = _C.log_matmul(d_lhs, d_rhs)
        np.testing.assert_allclose(d_res.cpu().numpy(), ref, rtol=1e-5, atol=1e-4)
        go = rng.standard_normal((B, M, Nn)).astype(np.float32)
        gl, gr = O.log_matmul_backward(go, lhs, rhs, ref)
        out_l, out_r = _C.log_matmul_backward(dev(go), d_lhs, d_rhs, d_res, [True, True])
        np.testing.assert_allclose(out_l.cpu().numpy(), gl, atol=2e-5, rtol=1e-4)
        np.testing.assert_allclose(out_r.cpu().numpy(), gr, atol=2e-5, rtol=1e-4)
        assert abs(gl[0, 4, 0]) + abs(gl[0, 4, 7]) > 1e-3


def test_log_matmul_rejects_bad_arguments():
    from warp_ctct import _C
    a = torch.zeros(2, 3, 4, device="cuda")
    with pytest.raises(RuntimeError):
        _C.log_matmul(a, torch.zeros(2, 5, 3, device="cuda"))      # inner sizes differ
    with pytest.raises(RuntimeError):
        _C.log_matmul(a.double(), torch.zeros(2, 4, 3, device="cuda").double())
    with pytest.raises(RuntimeError):
        _C.log_matmul(a.cpu(), torch.zeros(2, 4, 3))
    with pytest.raises(RuntimeError):
        _C.log_matmul(a[0], torch.zeros(4, 3, device="cuda"))


@pytest.mark.parametrize("B,M,K,Nn", [
    (2, 5, 7, 3), (2, 45, 130, 40), (1, 33, 65, 17),
    # reductions of 256 and more with at most 96 columns: the gradient of lhs keeps
    # a slab of the right operand in LDS; one, two and three chunks of columns,
    # ragged and whole row blocks, ragged and whole slabs
    (2, 37, 300, 81), (1, 48, 512, 33), (2, 20, 260, 7), (3, 64, 384, 96),
    # 128 and more rows as well: the gradient of rhs keeps its sums in registers and
    # streams lhs once; one to six blocks of 16 columns, ragged chunks of rows
    (2, 150, 300, 81), (1, 400, 512, 96), (2, 129, 260, 7), (1, 200, 777, 33), (1, 128, 256, 50)])
@pytest.mark.parametrize("mask", [(True, True), (True, False), (False, True)])
def test_log_matmul_backward(B, M, K, Nn, mask):
    from warp_ctct import _C
    rng = np.random.default_rng(M + K)
    lhs = rng.standard_normal((B, M, K)).astype(np.float32)
    rhs_t = rng.standard_normal((B, Nn, K)).astype(np.float32)
    rhs = rhs_t.transpose(0, 2, 1)
    go = rng.standard_normal((B, M, Nn)).astype(np.float32)       # signed
    go[0, 0, :] = 0.0
    res = O.log_matmul(lhs, rhs)
    gl, gr = O.log_matmul_backward(go, lhs, rhs, res)
    d_rhs = dev(rhs_t).transpose(1, 2)
    d_res = _C.log_matmul(dev(lhs), d_rhs)
    out_l, out_r = _C.log_matmul_backward(dev(go), dev(lhs), d_rhs, d_res, list(mask))
    if mask[0]:
        assert out_l.shape == lhs.shape
        np.testing.assert_allclose(out_l.cpu().numpy(), gl, atol=2e-5, rtol=1e-4)
    else:
        assert out_l is None
    if mask[1]:
        assert out_r.shape == (B, K, Nn)
        np.testing.assert_allclose(out_r.cpu().numpy(), gr, atol=2e-5, rtol=1e-4)
    else:
        assert out_r is None


def test_log_matmul_with_a_shared_right_operand():
    """A size-1 batch of rhs is shared by all batch entries of lhs: the forward
    broadcasts it, the backward sums its gradient over the batch (the reference
    undoes the broadcast with a reduction, csrc/binding.cpp:283-296).  Checked
    against torch.logsumexp and its autograd with the operand expanded."""
    import warp_ctct
    rng = np.random.default_rng(88)
    B, M, K, Nn = 5, 37, 70, 11
    lhs = torch.tensor(rng.standard_normal((B, M, K)), dtype=torch.float32, device="cuda", requires_grad=True)
    rhs = torch.tensor(rng.standard_normal((1, K, Nn)), dtype=torch.float32, device="cuda", requires_grad=True)
    w = torch.tensor(rng.standard_normal((B, M, Nn)), dtype=torch.float32, device="cuda")
    out = warp_ctct.LogMMExp.apply(lhs, rhs)
    ref = torch.logsumexp(lhs[:, :, :, None] + rhs.expand(B, K, Nn)[:, None, :, :], dim=2)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)
    gl, gr = torch.autograd.grad((out * w).sum(), (lhs, rhs))
    rl, rr = torch.autograd.grad((ref * w).sum(), (lhs, rhs))
    assert gl.shape == lhs.shape and gr.shape == rhs.shape
    torch.testing.assert_close(gl, rl, rtol=1e-4, atol=2e-5)
    torch.testing.assert_close(gr, rr, rtol=1e-4, atol=5e-5)
    # the same with lhs given as a view whose batch entries are not adjacent rows
    base = torch.tensor(rng.standard_normal((M, B, K)), dtype=torch.float32, device="cuda")
    view = base.transpose(0, 1).detach().requires_grad_(True)
    out2 = warp_ctct.LogMMExp.apply(view, rhs)
    ref2 = torch.logsumexp(view[:, :, :, None] + rhs.expand(B, K, Nn)[:, None, :, :], dim=2)
    g2 = torch.autograd.grad((out2 * w).sum(), (view, rhs))
    r2 = torch.autograd.grad((ref2 * w).sum(), (view, rhs))
    torch.testing.assert_close(g2[0], r2[0], rtol=1e-4, atol=2e-5)
    torch.testing.assert_close(g2[1], r2[1], rtol=1e-4, atol=5e-5)


def test_log_matmul_empty_extents():
    """Empty reductions and empty operands: logsumexp over nothing is -inf,
    its gradient zero; empty outputs stay empty."""
    from warp_ctct import _C
    z = lambda *shape: torch.zeros(*shape, device="cuda")
    out = _C.log_matmul(z(2, 3, 0), z(2, 0, 4))
    assert out.shape == (2, 3, 4) and bool(torch.isneginf(out).all())
    assert _C.log_matmul(z(2, 0, 5), z(2, 5, 4)).shape == (2, 0, 4)
    assert _C.log_matmul(z(2, 3, 5), z(2, 5, 0)).shape == (2, 3, 0)
    assert _C.log_matmul(z(0, 3, 5), z(0, 5, 4)).shape == (0, 3, 4)
    # backward: no rows on one side -> the other side's gradient is all zeros
    gl, gr = _C.log_matmul_backward(z(2, 0, 4), z(2, 0, 5), z(2, 5, 4), z(2, 0, 4), [True, True])
    assert gl.shape == (2, 0, 5) and gr.shape == (2, 5, 4) and bool((gr == 0).all())
    lhs = torch.randn(2, 3, 5, device="cuda")
    gl, gr = _C.log_matmul_backward(z(2, 3, 0), lhs, z(2, 5, 0), z(2, 3, 0), [True, True])
    assert gr.shape == (2, 5, 0) and gl.shape == (2, 3, 5) and bool((gl == 0).all())
    gl, gr = _C.log_matmul_backward(z(2, 3, 4), z(2, 3, 0), z(2, 0, 4), z(2, 3, 4), [True, True])
    assert gl.shape == (2, 3, 0) and gr.shape == (2, 0, 4)


def test_reference_autograd_classes_on_gathered_operands():
    """warp_ctct.LogMMExp / CTCTLoss / SimpleCTCTLoss, the reference's
    module-level autograd functions (warp_ctct/__init__.py:20-85), for code
    that imports them by name: LogMMExp against torch.logsumexp and its
    autograd, the two loss functions against the oracle on gathered operands."""
    import warp_ctct
    rng = np.random.default_rng(77)
    lhs = torch.tensor(rng.standard_normal((2, 9, 21)), dtype=torch.float32, device="cuda", requires_grad=True)
    rhs_t = torch.tensor(rng.standard_normal((2, 6, 21)), dtype=torch.float32, device="cuda", requires_grad=True)
    w = torch.tensor(rng.standard_normal((2, 9, 6)), dtype=torch.float32, device="cuda")
    out = warp_ctct.LogMMExp.apply(lhs, rhs_t.transpose(1, 2))
    ref = torch.logsumexp(lhs[:, :, :, None] + rhs_t.transpose(1, 2)[:, None, :, :], dim=2)
    torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)
    gl, gr = torch.autograd.grad((out * w).sum(), (lhs, rhs_t))
    rl, rr = torch.autograd.grad((ref * w).sum(), (lhs, rhs_t))
    torch.testing.assert_close(gl, rl, rtol=1e-4, atol=2e-5)
    torch.testing.assert_close(gr, rr, rtol=1e-4, atol=2e-5)
    only_l = warp_ctct.LogMMExp.apply(lhs, rhs_t.transpose(1, 2), True, False)
    (g_only,) = torch.autograd.grad((only_l * w).sum(), (lhs,))
    torch.testing.assert_close(g_only, rl, rtol=1e-4, atol=2e-5)

    f, g, ys, lx, ly = make_simple_case(78, 3, 14, 4, 11, lx=[14, 9, 12], ly=[4, 2, 3])
    f_g, g_g = O.gather_separate(f, g, ys)
    den = O.log_matmul(f, np.swapaxes(g, 1, 2)).astype(np.float32)
    costs, gf, gg, gd = O.ctct_loss_simple_fwd(f_g, g_g, ys, den, lx, ly)
    tf, tg, td = (dev(a).requires_grad_(True) for a in (f_g, g_g, den))
    wn = np.array([0.5, 2.0, -1.0])
    c = warp_ctct.SimpleCTCTLoss.apply(tf, tg, td, dev(ys), dev(lx), dev(ly), True, True)
    np.testing.assert_allclose(c.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    (c * dev(wn, torch.float32)).sum().backward()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf * wn[:, None, None], atol=2 * GRAD_ATOL)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg * wn[:, None, None], atol=2 * GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(td.grad.cpu().numpy(), gd * wn[:, None, None], atol=2 * GRAD_ATOL)
    # unnormalised, gradient wanted for g only
    costs_u, _, gg_u, _ = O.ctct_loss_simple_fwd(f_g, g_g, ys, None, lx, ly)
    tg2 = dev(g_g).requires_grad_(True)
    c_u = warp_ctct.SimpleCTCTLoss.apply(dev(f_g), tg2, None, dev(ys), dev(lx), dev(ly), False, True)
    np.testing.assert_allclose(c_u.detach().cpu().numpy(), costs_u, rtol=LOSS_RTOL)
    c_u.sum().backward()
    np.testing.assert_allclose(tg2.grad.cpu().numpy(), gg_u, atol=2 * GRAD_ATOL, rtol=1e-5)

    joint, ys, lx, ly = make_joint_case(79, 3, 12, 4, 9, lx=[12, 8, 10], ly=[4, 3, 2])
    lp3 = O.gather_units(joint, ys)
    costs3, ug = C.ctct_loss_fwd(lp3, ys, lx, ly, dtype=np.float64)
    t3 = dev(lp3.astype(np.float32)).requires_grad_(True)
    c3 = warp_ctct.CTCTLoss.apply(t3, dev(ys), dev(lx), dev(ly), True)
    np.testing.assert_allclose(c3.detach().cpu().numpy(), costs3, rtol=LOSS_RTOL)
    (c3 * dev(wn, torch.float32)).sum().backward()
    np.testing.assert_allclose(t3.grad.cpu().numpy(), ug * wn[:, None, None, None], atol=2 * GRAD_ATOL)


# ------------------------------------------------ reference operator surface
SIMPLE_CASES = [
    # name, seed, N, T, U, V, lx, ly
    ("small", 1, 3, 12, 4, 9, [12, 9, 7], [4, 2, 3]),
    ("ragged", 2, 5, 40, 11, 33, range(20, 41), range(3, 12)),
    ("two_contexts_per_lane", 3, 2, 140, 90, 50, [140, 120], [90, 70]),
    ("single_label", 4, 2, 5, 1, 6, [5, 2], [1, 1]),
    # shapes that take the other log-matmul gradient kernels: more than 96
    # contexts (no resident slab), and a frame count that tiles better by 96
    ("wide_contexts", 5, 2, 130, 110, 40, [130, 125], [110, 100]),
    ("ninety_frames", 6, 3, 90, 20, 70, [90, 81, 66], [20, 17, 9]),
    # shapes whose log-matmul kernels read f itself (at least 128 frames, at most 96
    # contexts, a vocabulary of 512..2048 in whole chunks of 32): one block of 16
    # contexts and four, a vocabulary that ends inside a slab, ragged lengths
    ("reads_f_itself_few_contexts", 7, 2, 160, 5, 512, [160, 131], [5, 3]),
    ("reads_f_itself_partial_slab", 8, 2, 130, 60, 800, [130, 128], [60, 33]),
    # the remaining instances of the joiner's gradient kernels: two and five
    # blocks of 16 contexts, with f read itself and with a vocabulary too long
    # for that (2049..4096 and 4097..8192 entries: the row kernels of the shifted
    # exponentials for 16 and 32 vectors per lane)
    ("reads_f_itself_five_blocks", 9, 2, 130, 70, 800, [130, 128], [70, 41]),
    ("reads_f_itself_two_blocks", 11, 2, 128, 20, 512, [128, 128], [20, 9]),
    ("long_vocabulary_two_blocks", 10, 2, 144, 20, 2304, [144, 129], [20, 11]),
    ("long_vocabulary_five_blocks", 12, 2, 144, 66, 4352, [144, 140], [66, 50]),
]


@pytest.mark.parametrize("case", SIMPLE_CASES, ids=[c[0] for c in SIMPLE_CASES])
@pytest.mark.parametrize("normalized", [True, False])
def test_operator_surface_simple_fwd(case, normalized):
    """_C.ctct_loss_simple_fwd(f_g, g_g, ys, den, lx, ly, requires_grad)."""
    from warp_ctct import _C
    name, seed, N, T, U, V, lx, ly = case
    f, g, ys, lx, ly = make_simple_case(seed, N, T, U, V, lx=lx, ly=ly, normalized=normalized)
    f_g, g_g = O.gather_separate(f, g, ys)
    den = O.log_matmul(f, np.swapaxes(g, 1, 2)).astype(np.float32) if normalized else None
    costs, gf, gg, gd = O.ctct_loss_simple_fwd(f_g, g_g, ys, den, lx, ly)
    d_den = dev(den) if normalized else torch.empty(1)       # the reference's own stand-in
    out = _C.ctct_loss_simple_fwd(dev(f_g), dev(g_g), dev(ys), d_den, dev(lx), dev(ly), True)
    np.testing.assert_allclose(out[0].cpu().numpy(), costs, rtol=LOSS_RTOL)
    np.testing.assert_allclose(out[1].cpu().numpy(), gf, atol=GRAD_ATOL, rtol=0)
    # grad_g sums T gradients: scale the bound by what was summed
    np.testing.assert_allclose(out[2].cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)
    if normalized:
        np.testing.assert_allclose(out[3].cpu().numpy(), gd, atol=GRAD_ATOL, rtol=0)
    else:
        assert out[3] is None
    nog = _C.ctct_loss_simple_fwd(dev(f_g), dev(g_g), dev(ys), d_den, dev(lx), dev(ly), False)
    np.testing.assert_array_equal(nog[0].cpu().numpy(), out[0].cpu().numpy())
    assert nog[1] is None and nog[2] is None and nog[3] is None


# ----------------------------------------------------------------- public API
@pytest.mark.parametrize("case", SIMPLE_CASES, ids=[c[0] for c in SIMPLE_CASES])
@pytest.mark.parametrize("normalized", [True, False])
def test_public_simple_loss_and_grads(case, normalized):
    import warp_ctct
    name, seed, N, T, U, V, lx, ly = case
    f, g, ys, lx, ly = make_simple_case(seed, N, T, U, V, lx=lx, ly=ly, normalized=normalized)
    w = np.random.default_rng(seed).standard_normal(N)
    loss, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none",
                                             normalized=normalized, grad_output=w)
    tf = dev(f).requires_grad_(True)
    tg = dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                     normalized=normalized)
    np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    (out * dev(w, torch.float32)).sum().backward()
    scale = max(1.0, float(np.abs(w).max()))
    # dense gradients sum up to T (resp. U+1) unit gradients per entry
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL * scale, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL * scale, rtol=1e-5)
    assert tf.grad.shape == f.shape and tg.grad.shape == g.shape
    for n in range(N):
        assert np.all(tf.grad[n, lx[n]:].cpu().numpy() == 0)
        assert np.all(tg.grad[n, ly[n] + 1:].cpu().numpy() == 0)


@pytest.mark.parametrize("normalized", [True, False])
def test_simple_loss_without_a_single_frame(normalized):
    """T = 0: a sample without labels costs 0, one with labels is infeasible
    (+inf); the gradients have the operands' shapes, that of g all zeros."""
    import warp_ctct
    ys = np.array([[1, 2], [3, 4], [2, 2]], dtype=np.int32)
    lx = np.zeros(3, dtype=np.int32)
    for ly in ([0, 0, 0], [0, 1, 0]):
        ly = np.array(ly, dtype=np.int32)
        _, _, _, costs = O.ctct_simple_loss(np.zeros((3, 0, 5)), np.zeros((3, 3, 5)), ys, lx, ly,
                                            reduction="none", normalized=normalized)
        tf = torch.zeros(3, 0, 5, device="cuda", requires_grad=True)
        tg = torch.zeros(3, 3, 5, device="cuda", requires_grad=True)
        out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                         normalized=normalized)
        np.testing.assert_array_equal(out.detach().cpu().numpy(), costs.astype(np.float32))
        if np.all(np.isfinite(costs)):
            out.sum().backward()
            assert tf.grad.shape == tf.shape and tg.grad.shape == tg.shape
            assert np.all(tg.grad.cpu().numpy() == 0)


@pytest.mark.parametrize("normalized", [True, False])
def test_simple_loss_replays_from_a_hip_graph(normalized):
    """A captured ctct_simple_loss step (log-matmul, lattice, scatter) replays
    with the eager results of the same inputs; the scatter adds atomically, so
    gradients are compared within float32 rounding, the loss exactly."""
    import warp_ctct
    f, g, ys, lx, ly = make_simple_case(31, 3, 21, 6, 48, lx=range(12, 22), ly=range(2, 7),
                                        normalized=normalized)
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    sf, sg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            torch.autograd.grad(warp_ctct.ctct_simple_loss(sf, sg, d_ys, d_lx, d_ly,
                                                           normalized=normalized), (sf, sg))
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        s_loss = warp_ctct.ctct_simple_loss(sf, sg, d_ys, d_lx, d_ly, normalized=normalized)
        s_gf, s_gg = torch.autograd.grad(s_loss, (sf, sg))
    rng = np.random.default_rng(32)
    for replay in range(3):
        with torch.no_grad():
            sf.copy_(dev(rng.standard_normal(f.shape).astype(np.float32)))
            sg.copy_(dev(rng.standard_normal(g.shape).astype(np.float32)))
        graph.replay()
        torch.cuda.synchronize()
        got = (s_loss.clone(), s_gf.clone(), s_gg.clone())
        xf = sf.detach().clone().requires_grad_(True)
        xg = sg.detach().clone().requires_grad_(True)
        loss = warp_ctct.ctct_simple_loss(xf, xg, d_ys, d_lx, d_ly, normalized=normalized)
        gf, gg = torch.autograd.grad(loss, (xf, xg))
        torch.cuda.synchronize()
        assert torch.equal(got[0], loss), "replay %d" % replay
        torch.testing.assert_close(got[1], gf, rtol=1e-5, atol=1e-6)
        torch.testing.assert_close(got[2], gg, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("track", [(True, False), (False, True), (False, False)])
def test_simple_loss_partial_tracking_and_reduction(track):
    import warp_ctct
    f, g, ys, lx, ly = make_simple_case(7, 3, 15, 5, 12, lx=[15, 11, 8], ly=[5, 3, 4])
    loss, gf, gg, _ = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="mean", average_frames=True)
    tf = dev(f).requires_grad_(track[0])
    tg = dev(g).requires_grad_(track[1])
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys).long(), dev(lx).long(), dev(ly).long(),
                                     reduction="mean", average_frames=True)
    np.testing.assert_allclose(float(out.detach()), loss, rtol=LOSS_RTOL)
    if not any(track):
        assert not out.requires_grad
        return
    out.backward()
    if track[0]:
        np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    else:
        assert tf.grad is None
    if track[1]:
        np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)
    else:
        assert tg.grad is None


@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
@pytest.mark.parametrize("average_frames", [False, True])
@pytest.mark.parametrize("shape", [(5, 24, 7, 19), (70, 9, 3, 6), (3, 136, 20, 512)],
                         ids=["ragged", "batch_beyond_one_wavefront", "matrix_core_kernels"])
def test_simple_loss_reduction_inside_the_kernels(shape, average_frames, reduction, normalized):
    """reduction and average_frames of ctct_simple_loss (warp_ctct/__init__.py:138-147
    of the reference) are applied by the lattice kernel in the forward and by the
    per-sample weights of the backward: loss and both dense gradients against the
    float64 oracle, with an upstream gradient other than one."""
    import warp_ctct
    N, T, U, V = shape
    f, g, ys, lx, ly = make_simple_case(41 + N, N, T, U, V, lx=range(max(U + 2, T // 2), T + 1),
                                        ly=range(1, U + 1), normalized=normalized)
    rng = np.random.default_rng(N)
    w = rng.uniform(-1.5, 2.0, size=N) if reduction == "none" else np.array(-0.75)
    # the oracle takes the weight of every sample's cost in the differentiated scalar
    per_sample = np.broadcast_to(w, (N,)).astype(np.float64)
    if average_frames:
        per_sample = per_sample / lx
    if reduction == "mean":
        per_sample = per_sample / N
    loss, gf, gg, _ = O.ctct_simple_loss(f, g, ys, lx, ly, reduction=reduction,
                                         average_frames=average_frames, normalized=normalized,
                                         grad_output=per_sample)
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction=reduction,
                                     average_frames=average_frames, normalized=normalized)
    assert out.shape == ((N,) if reduction == "none" else ())
    np.testing.assert_allclose(out.detach().cpu().numpy(), loss, rtol=LOSS_RTOL)
    (out * dev(w, torch.float32)).sum().backward()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)


@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("case", [(3, 15, 5, 12, [15, 11, 8], [5, 3, 4]),
                                  (2, 140, 80, 9, [140, 125], [80, 70]),       # chains of two
                                  (2, 9, 4, 7, [9, 1], [4, 0])])
def test_simple_loss_repeated_labels_weighted_and_backward_twice(case, normalized):
    """Every other label repeats its neighbour (their columns of the dense gradients
    coincide and add), per-sample weights, and a second backward over a retained
    graph, which must give the same gradients again."""
    import warp_ctct
    N, T, U, V, lx, ly = case
    f, g, ys, lx, ly = make_simple_case(17, N, T, U, V, lx=lx, ly=ly, normalized=normalized)
    k = ys[:, 1::2].shape[1]
    ys[:, 1::2] = ys[:, 0::2][:, :k]
    w = np.linspace(0.5, 2.0, N)
    _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none",
                                          normalized=normalized, grad_output=w)
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                     normalized=normalized)
    fin = np.isfinite(costs)
    np.testing.assert_allclose(out.detach().cpu().numpy()[fin], costs[fin], rtol=LOSS_RTOL)
    assert fin.all()
    (out * dev(w, torch.float32)).sum().backward(retain_graph=True)
    first = (tf.grad.clone(), tg.grad.clone())
    tf.grad, tg.grad = None, None
    (out * dev(w, torch.float32)).sum().backward()
    for a, b in zip(first, (tf.grad, tg.grad)):
        torch.testing.assert_close(a, b, atol=1e-6, rtol=1e-6)
    np.testing.assert_allclose(first[0].cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(first[1].cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)


def test_simple_normalized_labels_crowded_into_few_columns():
    """All 40 labels of one sample (with repeats) lie in columns 1..99 of a
    512-column vocabulary, those of the other are spread out: the gradient through
    the gathers lands on a few columns of the dense gradient wrt f, on top of the
    gradient through the normaliser, in a shape that takes the matrix-core kernels
    (T a multiple of 16 >= 128, V a multiple of 128 >= 512)."""
    import warp_ctct
    N, T, U, V = 2, 144, 40, 512
    f, g, ys, lx, ly = make_simple_case(23, N, T, U, V, lx=[144, 130], ly=[40, 33], normalized=True)
    rng = np.random.default_rng(23)
    ys[0] = rng.integers(1, 100, U)
    ys[0, 1::2] = ys[0, 0::2]
    w = np.array([1.5, -0.5])
    _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none", normalized=True,
                                          grad_output=w)
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                     normalized=True)
    np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    (out * dev(w, torch.float32)).sum().backward()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)


def test_simple_normalized_reads_f_itself_edge_values():
    """Shapes whose log-matmul kernels read f itself (T >= 128, 512 <= V <= 2048 in
    whole chunks of 32), at their edges: no label dimension at all (one context),
    a sample whose lengths are zero beside a full one, vocabulary entries that are
    -inf in f, in g, and in both (their exponentials are 0 in every kernel that
    forms them), a whole 256-column slab of f at -inf, and a zero weight."""
    import warp_ctct
    rng = np.random.default_rng(31)
    # U = 0
    N, T, V = 2, 128, 512
    f = np.log(rng.dirichlet(np.ones(V), (N, T))).astype(np.float32)
    g = np.log(rng.dirichlet(np.ones(V), (N, 1))).astype(np.float32)
    ys = np.zeros((N, 0), np.int32)
    lx, ly = np.array([128, 77], np.int32), np.zeros(N, np.int32)
    w = np.array([1.0, 0.0])
    _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none", normalized=True,
                                          grad_output=w)
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none", normalized=True)
    np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    (out * dev(w, torch.float32)).sum().backward()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)
    # -inf entries; labels avoid the masked columns, blank (0) stays finite
    N, T, U, V = 2, 136, 6, 1024
    f, g, ys, lx, ly = make_simple_case(32, N, T, U, V, lx=[136, 129], ly=[6, 4], normalized=True)
    ys[:] = rng.integers(1, 200, ys.shape)
    f[:, :, 300:400] = -np.inf          # in f only
    g[:, :, 380:500] = -np.inf          # in g only, and 380..399 in both
    f[0, 5:40, 512:768] = -np.inf       # a whole slab of the reduction for some frames
    _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none", normalized=True,
                                          grad_output=np.ones(N))
    assert np.isfinite(costs).all()
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none", normalized=True)
    np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    out.sum().backward()
    assert torch.isfinite(tf.grad).all() and torch.isfinite(tg.grad).all()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)


@pytest.mark.parametrize("normalized", [True, False])
def test_simple_loss_edge_shapes(normalized):
    """No label dimension at all (g holds the one start context), samples
    without labels beside samples with labels, a single frame, an empty batch."""
    import warp_ctct
    rng = np.random.default_rng(71)
    # U = 0: only the all-blank path
    f = rng.standard_normal((3, 7, 6)).astype(np.float32)
    g = rng.standard_normal((3, 1, 6)).astype(np.float32)
    ys = np.zeros((3, 0), np.int32)
    lx, ly = np.array([7, 4, 1], np.int32), np.zeros(3, np.int32)
    loss, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none",
                                             normalized=normalized, grad_output=np.ones(3))
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                     normalized=normalized)
    np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    out.sum().backward()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)
    # zero-label samples inside a batch with labels, one of them a single frame
    f, g, ys, lx, ly = make_simple_case(72, 4, 9, 3, 8, lx=[9, 5, 1, 3], ly=[3, 0, 1, 0],
                                        normalized=normalized)
    loss, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none",
                                             normalized=normalized, grad_output=np.ones(4))
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                     normalized=normalized)
    np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    out.sum().backward()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)
    # empty batch
    ef = torch.zeros(0, 5, 4, device="cuda", requires_grad=True)
    eg = torch.zeros(0, 3, 4, device="cuda", requires_grad=True)
    ei = torch.zeros(0, 2, dtype=torch.int32, device="cuda")
    el = torch.zeros(0, dtype=torch.int32, device="cuda")
    assert tuple(warp_ctct.ctct_simple_loss(ef, eg, ei, el, el, reduction="none",
                                            normalized=normalized).shape) == (0,)
    s_ = warp_ctct.ctct_simple_loss(ef, eg, ei, el, el, reduction="sum", normalized=normalized)
    assert s_.item() == 0.0
    s_.backward()
    assert tuple(ef.grad.shape) == (0, 5, 4) and tuple(eg.grad.shape) == (0, 3, 4)


@pytest.mark.parametrize("normalized", [True, False])
def test_simple_loss_vocabulary_beyond_one_lds_row(normalized):
    """V = 20000: a row of f no longer fits the 64 KiB that the whole-row
    builder of the unnormalised dense gradient stages in LDS (zero-fill plus
    atomic adds take over), and the log-matmul reduces over 625 chunks."""
    import warp_ctct
    f, g, ys, lx, ly = make_simple_case(73, 2, 7, 3, 20000, lx=[7, 5], ly=[3, 2], normalized=normalized)
    ys[0] = [19999, 19999, 17000]                     # last column, a repeat
    lx[0] = 7
    w = np.array([0.5, -2.0])
    loss, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none",
                                             normalized=normalized, grad_output=w)
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                     normalized=normalized)
    np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
    (out * dev(w, torch.float32)).sum().backward()
    np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=2 * GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=2 * GRAD_ATOL, rtol=1e-5)


def test_simple_loss_assertions():
    import warp_ctct
    f, g, ys, lx, ly = make_simple_case(8, 2, 6, 2, 5)
    with pytest.raises(AssertionError):
        warp_ctct.ctct_simple_loss(dev(f), dev(g)[:, :2], dev(ys), dev(lx), dev(ly))
    with pytest.raises(AssertionError):
        warp_ctct.ctct_simple_loss(dev(f)[0], dev(g), dev(ys), dev(lx), dev(ly))
    with pytest.raises(AssertionError):
        warp_ctct.ctct_simple_loss(dev(f), dev(g), dev(ys), dev(lx), dev(ly), reduction="max")


def _identity_check(N, T, U, V, lx_rng, ly_rng, normalized, seed):
    """ctct_simple_loss(f, g) == ctct_loss(joiner(f, g)) with the joint
    materialised on the GPU, losses and gradients (through torch autograd of
    the broadcast add / log_softmax)."""
    import warp_ctct
    rng = np.random.default_rng(seed)
    gen = torch.Generator(device="cuda").manual_seed(seed)
    f = torch.randn(N, T, V, device="cuda", generator=gen)
    g = torch.randn(N, U + 1, V, device="cuda", generator=gen)
    if normalized:
        f = f.log_softmax(-1)
        g = g.log_softmax(-1)
    lx = rng.integers(lx_rng[0], lx_rng[1] + 1, N).astype(np.int32)
    ly = rng.integers(ly_rng[0], ly_rng[1] + 1, N).astype(np.int32)
    lx[0], ly[-1] = lx_rng[1], ly_rng[1]
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    ys[:, 5] = ys[:, 4]
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    w = torch.tensor(rng.standard_normal(N), dtype=torch.float32, device="cuda")
    f1 = f.clone().requires_grad_(True)
    g1 = g.clone().requires_grad_(True)
    c1 = warp_ctct.ctct_simple_loss(f1, g1, d_ys, d_lx, d_ly, reduction="none",
                                    normalized=normalized)
    (c1 * w).sum().backward()
    f2 = f.clone().requires_grad_(True)
    g2 = g.clone().requires_grad_(True)
    joint = f2[:, :, None, :] + g2[:, None, :, :]
    if normalized:
        joint = joint.log_softmax(-1)
    c2 = warp_ctct.ctct_loss(joint, d_ys, d_lx, d_ly, reduction="none")
    (c2 * w).sum().backward()
    np.testing.assert_allclose(c1.detach().cpu().numpy(), c2.detach().cpu().numpy(), rtol=LOSS_RTOL)
    scale = max(1.0, float(w.abs().max()))
    # torch sums fp32 gradients over u (resp. t) in the reference side: allow for that
    np.testing.assert_allclose(f1.grad.cpu().numpy(), f2.grad.cpu().numpy(),
                               atol=2 * GRAD_ATOL * scale, rtol=1e-4)
    np.testing.assert_allclose(g1.grad.cpu().numpy(), g2.grad.cpu().numpy(),
                               atol=2 * GRAD_ATOL * scale, rtol=1e-4)
    return c1


def test_full_size_log_add_joiner_normalized():
    """N=32, T<=400, U<=80, V=2048, normalized."""
    c = _identity_check(32, 400, 80, 2048, (300, 400), (50, 80), True, 404)
    assert torch.isfinite(c).all()


def test_full_size_log_add_joiner_against_the_float64_oracle():
    """N=32, T<=400, U<=80, V=2048, normalized: the shapes that select the
    production tiles of the three matrix-core kernels.  den, the loss and the
    dense gradients wrt f and g of two batch entries (one of them the longest)
    against the float64 oracle at the gate itself: loss 1e-5 relative,
    gradients 1e-4 absolute."""
    import warp_ctct
    from warp_ctct import _C
    N, T, U, V = 32, 400, 80, 2048
    rng = np.random.default_rng(414)
    gen = torch.Generator(device="cuda").manual_seed(414)
    f = torch.randn(N, T, V, device="cuda", generator=gen).log_softmax(-1)
    g = torch.randn(N, U + 1, V, device="cuda", generator=gen).log_softmax(-1)
    lx = rng.integers(300, 401, N).astype(np.int32)
    ly = rng.integers(50, 81, N).astype(np.int32)
    lx[0], ly[0] = 400, 80
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    ys[:, 5] = ys[:, 4]
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    w = rng.standard_normal(N)
    w[0], w[9] = 1.25, -0.75
    f.requires_grad_(True)
    g.requires_grad_(True)
    costs = warp_ctct.ctct_simple_loss(f, g, d_ys, d_lx, d_ly, reduction="none")
    (costs * dev(w, torch.float32)).sum().backward()
    den = _C.ctct_simple_fwd(f.detach(), g.detach(), d_ys, d_lx, d_ly, True, False)[1]
    for n in (0, 9):
        fn = f[n:n + 1].detach().cpu().numpy()
        gn = g[n:n + 1].detach().cpu().numpy()
        t, u = int(lx[n]), int(ly[n])
        den_ref = O.log_matmul(fn[:, :t], np.swapaxes(gn[:, :u + 1], 1, 2))
        np.testing.assert_allclose(den[n, :t, :u + 1].cpu().numpy(), den_ref[0], rtol=1e-5, atol=1e-5)
        loss, gf, gg, c_ref = O.ctct_simple_loss(fn, gn, ys[n:n + 1], lx[n:n + 1], ly[n:n + 1],
                                                 reduction="none", grad_output=w[n:n + 1])
        np.testing.assert_allclose(costs[n].item(), c_ref[0], rtol=LOSS_RTOL)
        # an entry of these gradients is a sum over up to 400 frames (81 contexts)
        # of terms that are each within the bound; where it reaches the hundreds,
        # one unit in the last place of float32 is 3e-5: 1e-6 relative on top
        np.testing.assert_allclose(f.grad[n].cpu().numpy(), gf[0], atol=GRAD_ATOL, rtol=1e-6)
        np.testing.assert_allclose(g.grad[n].cpu().numpy(), gg[0], atol=GRAD_ATOL, rtol=1e-6)
        assert np.all(f.grad[n, t:].cpu().numpy() == 0) and np.all(g.grad[n, u + 1:].cpu().numpy() == 0)


def test_full_size_normalized_joiner_invariants():
    """N=32, T<=400, U<=80, V=2048, normalized: properties that hold at any size.
    The normalised loss sees f and g only through log_softmax(f + g): adding a
    constant to every vocabulary entry of a frame of f (of a context of g) changes
    neither the costs nor the gradients; for the same reason the gradient wrt f
    sums to zero over the vocabulary in every frame, and likewise that wrt g;
    frames beyond lx and contexts beyond ly take no gradient; and the gradients
    are linear in the weights of the samples."""
    import warp_ctct
    N, T, U, V = 32, 400, 80, 2048
    rng = np.random.default_rng(515)
    gen = torch.Generator(device="cuda").manual_seed(515)
    f = torch.randn(N, T, V, device="cuda", generator=gen)
    g = torch.randn(N, U + 1, V, device="cuda", generator=gen)
    lx = rng.integers(300, 401, N).astype(np.int32)
    ly = rng.integers(50, 81, N).astype(np.int32)
    lx[3], ly[3] = 400, 80
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    w = torch.randn(N, device="cuda", generator=gen)

    def run(ff, gg, weights):
        ff = ff.clone().requires_grad_(True)
        gg = gg.clone().requires_grad_(True)
        costs = warp_ctct.ctct_simple_loss(ff, gg, d_ys, d_lx, d_ly, reduction="none", normalized=True)
        (costs * weights).sum().backward()
        return costs.detach(), ff.grad, gg.grad

    c0, gf0, gg0 = run(f, g, w)
    assert torch.isfinite(c0).all()
    # shifts per frame and per context, of the size of the values themselves
    sf = 3.0 * torch.randn(N, T, 1, device="cuda", generator=gen)
    sg = 3.0 * torch.randn(N, U + 1, 1, device="cuda", generator=gen)
    c1, gf1, gg1 = run(f + sf, g + sg, w)
    torch.testing.assert_close(c1, c0, rtol=2e-5, atol=1e-3)
    scale = float(w.abs().max())
    torch.testing.assert_close(gf1, gf0, rtol=1e-4, atol=2 * GRAD_ATOL * scale)
    torch.testing.assert_close(gg1, gg0, rtol=1e-4, atol=2 * GRAD_ATOL * scale)
    # zero sum over the vocabulary (each row sums 2048 terms of either sign)
    assert float(gf0.sum(-1).abs().max()) < 1e-3 * scale
    assert float(gg0.double().sum(-1).abs().max()) < 2e-2 * scale    # entries reach the hundreds
    # nothing beyond the lengths
    t_idx = torch.arange(T, device="cuda")[None, :] >= d_lx[:, None]
    u_idx = torch.arange(U + 1, device="cuda")[None, :] > d_ly[:, None]
    assert float(gf0[t_idx].abs().max()) == 0.0 and float(gg0[u_idx].abs().max()) == 0.0
    # linear in the weights
    c2, gf2, gg2 = run(f, g, -2.0 * w)
    torch.testing.assert_close(c2, c0, rtol=0, atol=0)
    torch.testing.assert_close(gf2, -2.0 * gf0, rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(gg2, -2.0 * gg0, rtol=1e-5, atol=1e-5)


def test_deep_lattice_unnormalized():
    """The long-utterance shape (T<=1500, U<=300) at a vocabulary that lets the
    joint be materialised for the identity check."""
    c = _identity_check(2, 1500, 300, 256, (1200, 1500), (250, 300), False, 505)
    assert torch.isfinite(c).all()


def test_full_size_unnormalized_stress_against_c_oracle():
    """N=4, T<=1500, U<=300, V=8192 raw scores: costs and compact gradients
    against the C oracle in float64 on the gathered operands; dense gradients
    through their scatter structure."""
    import warp_ctct
    from warp_ctct import _C
    N, T, U, V = 4, 1500, 300, 8192
    rng = np.random.default_rng(606)
    gen = torch.Generator(device="cuda").manual_seed(606)
    f = torch.randn(N, T, V, device="cuda", generator=gen)
    g = torch.randn(N, U + 1, V, device="cuda", generator=gen)
    lx = rng.integers(1200, 1501, N).astype(np.int32)
    ly = rng.integers(250, 301, N).astype(np.int32)
    lx[1], ly[2] = 1500, 300
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    ys[:, 9] = ys[:, 8]
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    f.requires_grad_(True)
    g.requires_grad_(True)
    costs = warp_ctct.ctct_simple_loss(f, g, d_ys, d_lx, d_ly, reduction="none", normalized=False)
    costs.sum().backward()
    # oracle on gathered operands
    fi = torch.zeros(N, T, U + 1, dtype=torch.long, device="cuda")
    fi[..., 1:] = d_ys.long()[:, None, :]
    gi = torch.zeros(N, U + 1, 3, dtype=torch.long, device="cuda")
    gi[:, 1:, 1] = d_ys
    gi[:, :U, 2] = d_ys
    f_g = f.detach().gather(-1, fi).cpu().numpy()
    g_g = g.detach().gather(-1, gi).cpu().numpy()
    lp3 = O.simple_units(f_g, g_g, None)
    c_ref, ug = C.ctct_loss_fwd(lp3, ys, lx, ly, dtype=np.float64)
    np.testing.assert_allclose(costs.detach().cpu().numpy(), c_ref, rtol=LOSS_RTOL)
    gf_ref, gg_ref, _ = O.simple_unit_grad_reduce(ug, False)
    # dense grad_f at the gathered columns: labels repeat, so compare column sums
    dense_f = f.grad
    exp_f = torch.zeros_like(dense_f, dtype=torch.float64)
    exp_f.scatter_add_(-1, fi, torch.as_tensor(gf_ref).cuda())
    np.testing.assert_allclose(dense_f.cpu().numpy(), exp_f.cpu().numpy(), atol=GRAD_ATOL, rtol=1e-5)
    exp_g = torch.zeros_like(g.grad, dtype=torch.float64)
    exp_g.scatter_add_(-1, gi, torch.as_tensor(gg_ref).cuda())
    np.testing.assert_allclose(g.grad.cpu().numpy(), exp_g.cpu().numpy(), atol=GRAD_ATOL, rtol=1e-5)


# ------------------------------------------------- lattices in the linear domain
def _launched_kernels(run):
    """Names of the library's kernels that `run` launches (its timing hook)."""
    import ctypes
    lib = hip_lib.lib()
    torch.cuda.synchronize()
    assert lib.warpctct_profile(1) == 0
    try:
        run()
        torch.cuda.synchronize()
    finally:
        lib.warpctct_profile(0)
    name, us = ctypes.c_char_p(), ctypes.c_float()
    names = []
    for i in range(lib.warpctct_profile_count()):
        if lib.warpctct_profile_read(i, ctypes.byref(name), ctypes.byref(us)) == 0:
            names.append(name.value.decode())
    return names


def _loss_and_grads(f, g, ys, lx, ly, normalized, reduction="none", w=None):
    import warp_ctct
    tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
    out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction=reduction,
                                     normalized=normalized)
    (out * dev(w, torch.float32)).sum().backward() if w is not None else out.sum().backward()
    return out.detach(), tf.grad, tg.grad


@pytest.mark.parametrize("normalized", [True, False])
def test_linear_lattices_are_used_for_long_inputs_and_hold_on_ordinary_input(normalized, lattice_domain):
    """With the default setting the fused forward sweeps in the linear domain from
    768 frames on, from 384 with normalisation (lattice_lin_kernel is launched, the
    log-domain kernels behind it return at once: the fall-back bit stays clear),
    and below that in the log domain; both agree with the oracle.  A chain of two
    workgroups per lattice."""
    import warp_ctct
    lib = hip_lib.lib()
    lib.warpctct_joiner_linear_lattice(-1)
    for T, linear in (((400, True), (380, False)) if normalized else ((780, True), (760, False))):
        N, U, V = 2, 70, 24
        f, g, ys, lx, ly = make_simple_case(60 + T, N, T, U, V, lx=[T, T - 37], ly=[U, 41],
                                            normalized=normalized)
        w = np.array([0.7, -1.3])
        _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none", normalized=normalized,
                                              grad_output=w)
        warp_ctct.status(reset=True)
        got = {}
        names = _launched_kernels(lambda: got.update(r=_loss_and_grads(f, g, ys, lx, ly, normalized, w=w)))
        assert any("lattice_lin_kernel" in k for k in names) == linear, names
        assert not (warp_ctct.status(reset=True) & warp_ctct.STATUS_LINEAR_FELL_BACK)
        out, df, dg = got["r"]
        np.testing.assert_allclose(out.cpu().numpy(), costs, rtol=LOSS_RTOL)
        np.testing.assert_allclose(df.cpu().numpy(), gf, atol=GRAD_ATOL * 1.3, rtol=1e-5)
        np.testing.assert_allclose(dg.cpu().numpy(), gg, atol=GRAD_ATOL * 1.3, rtol=1e-5)


@pytest.mark.parametrize("what", ["unit_out_of_range", "infeasible_sample", "mass_beyond_the_range"])
def test_linear_lattices_fall_back_to_the_log_domain(what, lattice_domain):
    """Input that the linear sweeps cannot take is computed again in the log
    domain, in the same call: the results are bit for bit those of a call with the
    linear sweeps switched off, and the status word says so.
    - a gathered unit above 2^80 (a frame whose scores are ~+60: twelve such frames
      in a row would leave the range of a double);
    - a sample with fewer frames than its labels need (cost +inf, NaN gradients);
    - all units in range, but the mass that counts far below the largest state of
      its 64 contexts: the one label can only be emitted in the first three frames
      (log 0 afterwards), and the blank behind it scores -50 per frame, while the
      blank before it scores 0 and keeps context 0 at mass 1: context 1 falls by
      2^-72 per frame, is gone from the linear sweep after 15 frames, and the
      total mass comes out as 0, which the check refuses."""
    import warp_ctct
    lib = hip_lib.lib()
    N, T, U, V = 2, 64, 6, 11
    f, g, ys, lx, ly = make_simple_case(77, N, T, U, V, lx=[T, T - 9], ly=[U, 4], normalized=False)
    if what == "unit_out_of_range":
        f[0, 20, :] = 60.0
    elif what == "infeasible_sample":
        lx[1] = 3
    else:
        N, T, U, V = 1, 400, 1, 4
        f = np.zeros((N, T, V), np.float32)
        g = np.zeros((N, U + 1, V), np.float32)
        ys = np.array([[2]], np.int32)
        lx, ly = np.array([T], np.int32), np.array([U], np.int32)
        f[0, 3:, 2] = -np.inf
        g[0, 1, 0] = -50.0
    results = []
    for frames in (0, 1):
        lib.warpctct_joiner_linear_lattice(frames)
        warp_ctct.status(reset=True)
        results.append(_loss_and_grads(f, g, ys, lx, ly, False))
        bits = warp_ctct.status(reset=True)
        assert bool(bits & warp_ctct.STATUS_LINEAR_FELL_BACK) == (frames == 1), (what, bits)
    for a, b in zip(*results):
        assert torch.equal(torch.nan_to_num(a, nan=7.0), torch.nan_to_num(b, nan=7.0)), what
    _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none", normalized=False)
    if what != "infeasible_sample":
        np.testing.assert_allclose(results[1][0].cpu().numpy(), costs, rtol=LOSS_RTOL)
        np.testing.assert_allclose(results[1][1].cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)


@pytest.mark.may_fall_back
def test_linear_lattices_give_up_a_hand_over_that_does_not_arrive(lattice_domain):
    """The bounded wait of the linear sweeps, forced from the host: with a wait
    limit of 0 a wavefront that finds its neighbour's values missing declares them
    lost at its first look (no kernel waits, every one of them exits), the status
    word says so and that the batch went to the log-domain kernels, whose own
    chains lose their hand-overs the same way.  The call after that, with the
    limit back, is right again: nothing of the lost call is left in the buffers."""
    import warp_ctct
    lib = hip_lib.lib()
    # chains of three workgroups, 24 wavefronts that receive (any one of them finding
    # its first values missing is enough); sample 2 has a lone wavefront
    N, T, U, V = 7, 180, 150, 40
    f, g, ys, lx, ly = make_simple_case(91, N, T, U, V, lx=[T, 160, 40, T, 170, T, 175],
                                        ly=[U, 130, 30, 140, 128, U, 135], normalized=False)
    _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none", normalized=False)
    assert np.all(np.isfinite(costs))               # (every sample has alignments)
    lib.warpctct_joiner_linear_lattice(1)
    warp_ctct.status(reset=True)
    default = lib.warpctct_lattice_wait_limit(0)
    try:
        got = _loss_and_grads(f, g, ys, lx, ly, False)
    finally:
        assert lib.warpctct_lattice_wait_limit(-1) == 0
    bits = warp_ctct.status(reset=True)
    assert default > 1000
    assert bits & warp_ctct.STATUS_LOST_HAND_OVER and bits & warp_ctct.STATUS_LINEAR_FELL_BACK, bits
    # (the lone wavefront of sample 2 needs no hand-over, in either domain)
    np.testing.assert_allclose(got[0].cpu().numpy()[2], costs[2], rtol=LOSS_RTOL)
    got = _loss_and_grads(f, g, ys, lx, ly, False)
    assert warp_ctct.status(reset=True) == 0
    np.testing.assert_allclose(got[0].cpu().numpy(), costs, rtol=LOSS_RTOL)
    np.testing.assert_allclose(got[1].cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(got[2].cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)



@pytest.mark.parametrize("normalized", [False, True])
def test_linear_lattices_hold_on_peaked_scores(normalized, lattice_domain):
    """What a trained model hands in: at every frame one entry of the vocabulary far
    above the others (the label due there, or blank), the others 40-150 below, so
    that most units are between 2^-60 and 2^-220 and the mass of nearly every
    alignment vanishes against the best one's.  The linear sweeps lose such states,
    which is harmless: their check must pass, and costs and gradients are the
    oracle's.  Chains of three workgroups, 300 frames."""
    import warp_ctct
    N, T, U, V = 2, 300, 130, 40
    rng = np.random.default_rng(5)
    f = (-40.0 - 110.0 * rng.random((N, T, V))).astype(np.float32)
    g = (0.1 * rng.standard_normal((N, U + 1, V))).astype(np.float32)
    ys = rng.integers(1, V, size=(N, U)).astype(np.int32)
    lx, ly = np.array([T, T - 23], np.int32), np.array([U, 101], np.int32)
    for n in range(N):
        # the labels spread evenly over the frames, blank between them
        at = np.linspace(2, lx[n] - 3, ly[n]).astype(int)
        f[n, :, 0] = 0.0
        f[n, at, 0] = -60.0
        f[n, at, ys[n, :ly[n]]] = 0.0
    _, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none", normalized=normalized)
    assert np.all(np.isfinite(costs))
    warp_ctct.status(reset=True)
    got = _loss_and_grads(f, g, ys, lx, ly, normalized)
    assert not (warp_ctct.status() & warp_ctct.STATUS_LINEAR_FELL_BACK)
    # (normalised, the best alignment has probability 1 within float32: a cost of 0)
    np.testing.assert_allclose(got[0].cpu().numpy(), costs, rtol=LOSS_RTOL, atol=1e-5 if normalized else 0)
    np.testing.assert_allclose(got[1].cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(got[2].cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)


@pytest.mark.parametrize("shape", [(600, 260, 50), (300, 200, 130)], ids=["lone_wavefronts", "chains_of_three"])
def test_linear_lattices_with_several_wavefronts_on_every_simd(shape, lattice_domain):
    """1200 or 1800 wavefronts of sweeps at once, more than one per SIMD: the state in which
    a store of a lattice row whose data registers the next instruction overwrote
    came out wrong now and then (the check then sent the whole call back to the
    log domain).  The linear sweeps must hold, twice in a row with the same results (and
    so must the log-domain sweeps, whose rows are stored the same way), agree with
    the log-domain sweeps on every sample and with the oracle on a few."""
    import warp_ctct
    if lattice_domain != "linear_lattices":
        pytest.skip("a test of the linear sweeps")
    lib = hip_lib.lib()
    (N, T, U), V = shape, 16
    rng = np.random.default_rng(11)
    lx = rng.integers(T - 40, T + 1, size=N).astype(np.int32)
    ly = rng.integers(U // 2, U + 1, size=N).astype(np.int32)
    f, g, ys, lx, ly = make_simple_case(77, N, T, U, V, lx=lx, ly=ly, normalized=False)
    w = rng.standard_normal(N)
    runs = []
    for domain in (1, 1, 0, 0):
        lib.warpctct_joiner_linear_lattice(domain)
        warp_ctct.status(reset=True)
        runs.append([x.cpu().numpy() for x in _loss_and_grads(f, g, ys, lx, ly, False, w=w)])
        fell_back = warp_ctct.status(reset=True) & warp_ctct.STATUS_LINEAR_FELL_BACK
        assert not fell_back, "the linear lattices were given up"
    lib.warpctct_joiner_linear_lattice(1)
    # (one wavefront per block of the gradient kernel adds in a fixed order; with
    # several, the sums over the contexts take the order in which they arrive)
    for first, second in ((runs[0], runs[1]), (runs[2], runs[3])):   # linear twice, log domain twice
        assert np.array_equal(first[0], second[0])
        for a, b in zip(first[1:], second[1:]):
            assert np.array_equal(a, b) if U < 62 else np.allclose(a, b, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(runs[0][0], runs[2][0], rtol=LOSS_RTOL)
    np.testing.assert_allclose(runs[0][1], runs[2][1], atol=GRAD_ATOL, rtol=1e-5)
    # (the gradient of g sums all frames)
    np.testing.assert_allclose(runs[0][2], runs[2][2], atol=GRAD_ATOL * 2, rtol=1e-4)
    some = [0, 255, 256, N - 1]
    _, gf, gg, costs = O.ctct_simple_loss(f[some], g[some], ys[some], lx[some], ly[some], reduction="none",
                                          normalized=False, grad_output=w[some])
    np.testing.assert_allclose(runs[0][0][some], costs, rtol=LOSS_RTOL)
    np.testing.assert_allclose(runs[0][1][some], gf, atol=GRAD_ATOL, rtol=1e-5)
    np.testing.assert_allclose(runs[0][2][some], gg, atol=GRAD_ATOL * 2, rtol=1e-4)


def test_linear_lattices_by_default_only_for_batches_bound_by_latency(lattice_domain):
    """With the default setting, long inputs are swept in the linear domain only
    up to 768 wavefronts of sweeps (256 where a lattice needs one per direction);
    a limit set by the caller holds for every batch."""
    import warp_ctct
    if lattice_domain != "linear_lattices":
        pytest.skip("a test of the linear sweeps")
    lib = hip_lib.lib()
    T, V = 780, 8
    for N, U, linear in ((128, 50, True), (129, 50, False), (192, 123, True), (193, 123, False)):
        f, g, ys, lx, ly = make_simple_case(N + U, N, T, U, V, normalized=False)
        for setting, expected in ((-1, linear), (700, True)):
            lib.warpctct_joiner_linear_lattice(setting)
            names = _launched_kernels(lambda: _loss_and_grads(f, g, ys, lx, ly, False))
            assert any("lattice_lin_kernel" in k for k in names) == expected, (N, U, setting, names)
    lib.warpctct_joiner_linear_lattice(1)
