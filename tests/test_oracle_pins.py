"""Pins for oracle/ctct_oracle.py: each check would fail for a plausible
mistake in the restatement (dropped arc, wrong context index, wrong skip
condition, sign, transposed operand).  None of them retypes the oracle's
formula: they use enumeration, library routines, closed forms or finite
differences."""
import numpy as np
import pytest
import torch

from oracle import ctct_oracle as O
from ctct_cases import brute_force, log_softmax, make_joint_case, make_simple_case

TINY = [
    # (T, labels)            — covers repeats, single label, lx == ly, skip arcs
    (3, [1]),
    (4, [1, 2]),
    (5, [1, 1]),
    (5, [2, 1, 2]),
    (6, [1, 1, 2]),
    (6, [3, 2, 2]),
    (7, [1, 2, 3]),
    (3, [1, 2, 3]),           # lx == ly: a single path
    (5, [1, 2, 1, 2]),
    (7, [1, 1, 1]),           # needs blanks between every pair
    (5, [1, 1, 1]),           # exactly feasible (T = U + repeats)
]


@pytest.mark.parametrize("T,labels", TINY)
def test_brute_force_cost_and_dense_grad(T, labels):
    rng = np.random.default_rng(100 + T + 7 * len(labels))
    U = len(labels)
    V = max(labels) + 2
    lp = log_softmax(rng.standard_normal((T, U + 1, V)) * 1.5)
    ys = np.array(labels)
    ll_bf, dense_bf = brute_force(lp, ys)
    loss, dense, costs = O.ctct_loss(lp[None], ys[None], [T], [U], reduction="none")
    assert np.isclose(costs[0], -ll_bf, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dense[0], dense_bf, rtol=1e-10, atol=1e-12)
    # alpha-side and beta-side likelihoods agree
    lp3 = O.gather_units(lp[None], ys[None])[0]
    _, ll_a = O.alpha_lattice(lp3, ys)
    _, ll_b = O.beta_lattice(lp3, ys)
    assert np.isclose(ll_a, ll_bf, rtol=1e-12)
    assert np.isclose(ll_b, ll_bf, rtol=1e-12)


def test_infeasible_lattice_is_inf():
    # two equal labels need 3 frames
    lp = log_softmax(np.random.default_rng(0).standard_normal((2, 3, 4)))
    ll_bf, _ = brute_force(lp, [1, 1])
    assert ll_bf == -np.inf
    costs, _ = O.ctct_loss_fwd(O.gather_units(lp[None], np.array([[1, 1]])), [[1, 1]], [2], [2], False)
    assert costs[0] == np.inf


def test_padded_batch_matches_per_sample_brute_force():
    rng = np.random.default_rng(5)
    N, T, U, V = 3, 6, 3, 4
    joint = log_softmax(rng.standard_normal((N, T, U + 1, V)))
    ys = np.array([[1, 2, 2], [3, 3, 1], [2, 1, 3]])
    lx = np.array([6, 5, 4])
    ly = np.array([3, 2, 1])
    _, dense, costs = O.ctct_loss(joint, ys, lx, ly, reduction="none")
    for n in range(N):
        ll, d = brute_force(joint[n, :lx[n], :ly[n] + 1], ys[n, :ly[n]])
        assert np.isclose(costs[n], -ll, rtol=1e-12)
        np.testing.assert_allclose(dense[n, :lx[n], :ly[n] + 1], d, rtol=1e-10, atol=1e-13)
        assert np.all(dense[n, lx[n]:] == 0)
        assert np.all(dense[n, :, ly[n] + 1:] == 0)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_reduces_to_ctc_loss(seed):
    """If the joint does not depend on u the model is plain CTC: compare with
    torch.nn.functional.ctc_loss, losses directly and gradients through
    log_softmax on both sides."""
    rng = np.random.default_rng(seed)
    N, T, U, V = 3, 12, 4, 6
    logits = torch.tensor(rng.standard_normal((N, T, V)), dtype=torch.float64, requires_grad=True)
    ys = rng.integers(1, V, size=(N, U))
    ys[0, 1] = ys[0, 0]
    lx = np.array([12, 10, 9])
    ly = np.array([4, 3, 2])
    lp = logits.log_softmax(-1)
    ctc = torch.nn.functional.ctc_loss(lp.transpose(0, 1), torch.tensor(ys), torch.tensor(lx),
                                       torch.tensor(ly), blank=0, reduction="none")
    w = torch.tensor([0.3, -1.2, 2.0], dtype=torch.float64)
    (ctc * w).sum().backward()
    joint = np.repeat(lp.detach().numpy()[:, :, None, :], U + 1, axis=2)
    _, dense, costs = O.ctct_loss(joint, ys, lx, ly, reduction="none", grad_output=w.numpy())
    np.testing.assert_allclose(costs, ctc.detach().numpy(), rtol=1e-12)
    g_lp = dense.sum(2)                                   # d/d lp[n,t,v]
    p = np.exp(lp.detach().numpy())
    g_logits = g_lp - p * g_lp.sum(-1, keepdims=True)     # log_softmax backward
    np.testing.assert_allclose(g_logits, logits.grad.numpy(), rtol=1e-9, atol=1e-12)


def test_closed_form_when_lx_equals_ly():
    rng = np.random.default_rng(3)
    T = U = 9
    V = 12
    lp = log_softmax(rng.standard_normal((T, U + 1, V)))
    ys = np.array([1, 2, 3, 4, 5, 6, 7, 8, 9])
    expect = -sum(lp[t, t, ys[t]] for t in range(T))
    _, _, costs = O.ctct_loss(lp[None], ys[None], [T], [U], reduction="none")
    assert np.isclose(costs[0], expect, rtol=1e-13)


def test_frame_mass_invariant_and_support():
    joint, ys, lx, ly = make_joint_case(11, 4, 20, 6, 9, lx=range(12, 21), ly=range(2, 7),
                                        dtype=np.float64)
    _, dense, _ = O.ctct_loss(joint, ys, lx, ly, reduction="none")
    for n in range(4):
        per_frame = dense[n].sum((1, 2))
        np.testing.assert_allclose(per_frame[:lx[n]], -1.0, rtol=1e-10)
        assert np.all(per_frame[lx[n]:] == 0)
    lp3 = O.gather_units(joint, ys)
    _, g = O.ctct_loss_fwd(lp3, ys, lx, ly)
    idx = np.broadcast_to(O.gather_index(ys, 7)[:, None], g.shape)
    assert np.count_nonzero(dense) <= np.count_nonzero(g)
    # every non-zero of the dense gradient sits on a gathered index
    mask = np.zeros_like(dense, dtype=bool)
    np.put_along_axis(mask, idx, True, axis=-1)
    assert np.all(dense[~mask] == 0)


def test_unit_grads_match_finite_differences():
    joint, ys, lx, ly = make_joint_case(21, 1, 7, 3, 5, dtype=np.float64)
    lp3 = O.gather_units(joint, ys)
    costs, g = O.ctct_loss_fwd(lp3, ys, lx, ly)
    eps = 1e-6
    U = 3
    for t in range(7):
        for u in range(U + 1):
            for k in range(3):
                if (k == 1 and u == 0) or (k == 2 and u == U):
                    assert g[0, t, u, k] == 0
                    continue
                p = lp3.copy()
                p[0, t, u, k] += eps
                m = lp3.copy()
                m[0, t, u, k] -= eps
                fd = (O.ctct_loss_fwd(p, ys, lx, ly, False)[0][0]
                      - O.ctct_loss_fwd(m, ys, lx, ly, False)[0][0]) / (2 * eps)
                assert abs(fd - g[0, t, u, k]) < 1e-8


def test_logits_variant_against_library_log_softmax_and_finite_differences():
    """ctct_loss_with_logits: the loss is ctct_loss of torch.log_softmax's
    output; the gradient is what torch's own log_softmax backward makes of the
    (already pinned) gradient wrt the log-probabilities, and it matches central
    differences of the loss wrt single logits (a dropped softmax term or a
    wrong sign of the row sum fails both)."""
    rng = np.random.default_rng(77)
    N, T, U, V = 2, 6, 3, 5
    logits = rng.standard_normal((N, T, U + 1, V)) * 2.0
    ys = np.array([[1, 1, 3], [4, 2, 2]])
    lx, ly = np.array([6, 5]), np.array([3, 2])
    w = np.array([0.7, 1.9])
    loss, grad, costs = O.ctct_loss_with_logits(logits, ys, lx, ly, "none", False, grad_output=w)
    x = torch.tensor(logits, requires_grad=True)
    lp = torch.log_softmax(x, dim=-1)
    ref_loss, G, ref_costs = O.ctct_loss(lp.detach().numpy(), ys, lx, ly, "none", False,
                                         grad_output=w)
    np.testing.assert_allclose(costs, ref_costs, rtol=1e-12)
    lp.backward(torch.tensor(G))
    np.testing.assert_allclose(grad, x.grad.numpy(), rtol=1e-10, atol=1e-13)
    assert np.all(grad[0, :, :, :][np.abs(G[0]).sum(-1) == 0] == 0)   # untouched rows stay zero
    eps = 1e-6
    for idx in [(0, 0, 0, 0), (0, 2, 1, 1), (0, 4, 2, 3), (1, 3, 1, 2), (1, 1, 0, 4)]:
        p, m = logits.copy(), logits.copy()
        p[idx] += eps
        m[idx] -= eps
        fd = (O.ctct_loss_with_logits(p, ys, lx, ly, "none")[2] @ w
              - O.ctct_loss_with_logits(m, ys, lx, ly, "none")[2] @ w) / (2 * eps)
        assert abs(fd - grad[idx]) < 1e-7
    # rows sum to zero: log_softmax removes the direction of constant shifts
    assert np.max(np.abs(grad.sum(-1))) < 1e-12


def test_gather_closed_form():
    joint, ys, _, _ = make_joint_case(4, 2, 5, 3, 7, dtype=np.float64, zero_pad=False)
    lp3 = O.gather_units(joint, ys)
    for n in range(2):
        for u in range(4):
            np.testing.assert_array_equal(lp3[n, :, u, 0], joint[n, :, u, 0])
            if u >= 1:
                np.testing.assert_array_equal(lp3[n, :, u, 1], joint[n, :, u, ys[n, u - 1]])
            else:
                np.testing.assert_array_equal(lp3[n, :, u, 1], joint[n, :, u, 0])
            if u < 3:
                np.testing.assert_array_equal(lp3[n, :, u, 2], joint[n, :, u, ys[n, u]])
            else:
                np.testing.assert_array_equal(lp3[n, :, u, 2], joint[n, :, u, 0])
    t_idx = torch.zeros(2, 4, 3, dtype=torch.long)
    t_idx[:, 1:, 1] = torch.tensor(ys, dtype=torch.long)
    t_idx[:, :3, 2] = torch.tensor(ys, dtype=torch.long)
    ref = torch.tensor(joint).gather(-1, t_idx[:, None].expand(-1, 5, -1, -1)).numpy()
    np.testing.assert_array_equal(lp3, ref)


def test_log_matmul_against_logsumexp_and_autograd():
    rng = np.random.default_rng(8)
    B, M, K, Nn = 2, 5, 7, 4
    lhs = rng.standard_normal((B, M, K)) * 3
    rhs = rng.standard_normal((B, K, Nn)) * 3
    lhs[0, 1, :] = -np.inf                # a whole row of -inf -> -inf result
    rhs[1, 2, :] = -np.inf                # some -inf terms
    res = O.log_matmul(lhs, rhs)
    tl = torch.tensor(lhs)
    tr = torch.tensor(rhs)
    ref = torch.logsumexp(tl[:, :, :, None] + tr[:, None, :, :], dim=2).numpy()
    np.testing.assert_allclose(res, ref, rtol=1e-13)
    assert np.all(res[0, 1] == -np.inf)
    # backward on finite inputs, signed grad_out
    lhs = rng.standard_normal((B, M, K))
    rhs = rng.standard_normal((B, K, Nn))
    go = rng.standard_normal((B, M, Nn))
    tl = torch.tensor(lhs, requires_grad=True)
    tr = torch.tensor(rhs, requires_grad=True)
    out = torch.logsumexp(tl[:, :, :, None] + tr[:, None, :, :], dim=2)
    out.backward(torch.tensor(go))
    gl, gr = O.log_matmul_backward(go, lhs, rhs, out.detach().numpy())
    np.testing.assert_allclose(gl, tl.grad.numpy(), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(gr, tr.grad.numpy(), rtol=1e-11, atol=1e-13)


@pytest.mark.parametrize("normalized", [True, False])
def test_simple_loss_equals_full_loss_on_materialised_joint(normalized):
    f, g, ys, lx, ly = make_simple_case(13, 3, 9, 4, 7, lx=[9, 8, 6], ly=[4, 2, 3],
                                        normalized=normalized, dtype=np.float64)
    w = np.array([0.7, -0.4, 1.9])
    loss, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none",
                                             normalized=normalized, grad_output=w)
    tf = torch.tensor(f, requires_grad=True)
    tg = torch.tensor(g, requires_grad=True)
    joint = tf[:, :, None, :] + tg[:, None, :, :]
    if normalized:
        joint = joint.log_softmax(-1)
    _, dense, costs_full = O.ctct_loss(joint.detach().numpy(), ys, lx, ly, reduction="none",
                                       grad_output=w)
    np.testing.assert_allclose(costs, costs_full, rtol=1e-12)
    joint.backward(torch.tensor(dense))
    np.testing.assert_allclose(gf, tf.grad.numpy(), rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(gg, tg.grad.numpy(), rtol=1e-9, atol=1e-12)


def test_simple_fwd_reductions_are_consistent():
    """grad_den = -sum_k, grad_g = sum_t, grad_f: blank summed over u, label
    columns from the two neighbouring contexts (binding.cpp:198-219), checked by
    finite differences on f_g, g_g and den."""
    f, g, ys, lx, ly = make_simple_case(17, 2, 6, 3, 5, lx=[6, 5], ly=[3, 2], dtype=np.float64)
    den = O.log_matmul(f, np.swapaxes(g, 1, 2))
    f_g, g_g = O.gather_separate(f, g, ys)
    costs, gf, gg, gd = O.ctct_loss_simple_fwd(f_g, g_g, ys, den, lx, ly)
    eps = 1e-6

    def total(fg, gg_, dn):
        return O.ctct_loss_simple_fwd(fg, gg_, ys, dn, lx, ly, False)[0].sum()

    rng = np.random.default_rng(0)
    for arr, grad, which in ((f_g, gf, 0), (g_g, gg, 1), (den, gd, 2)):
        for _ in range(25):
            i = tuple(int(rng.integers(0, s)) for s in arr.shape)
            if which == 1 and ((i[1] == 0 and i[2] == 1) or (i[1] == 3 and i[2] == 2)):
                continue
            args = [f_g, g_g, den]
            p = arr.copy(); p[i] += eps
            m = arr.copy(); m[i] -= eps
            args[which] = p
            up = total(*args)
            args[which] = m
            dn = total(*args)
            assert abs((up - dn) / (2 * eps) - grad[i]) < 1e-7, (which, i)


def test_reduction_modes():
    costs = np.array([2.0, 6.0])
    lx = np.array([2, 3])
    assert O.reduce_costs(costs, lx, "mean") == 4.0
    assert O.reduce_costs(costs, lx, "sum") == 8.0
    np.testing.assert_array_equal(O.reduce_costs(costs, lx, None), costs)
    np.testing.assert_array_equal(O.reduce_costs(costs, lx, "none", True), [1.0, 2.0])


# ---------------------------------------------------------------- C oracle
def test_c_oracle_matches_numpy_oracle_and_brute_force():
    from oracle import c_oracle as C
    joint, ys, lx, ly = make_joint_case(31, 5, 17, 5, 8, lx=range(9, 18), ly=range(1, 6),
                                        dtype=np.float64)
    lp3 = O.gather_units(joint, ys)
    costs, grads = O.ctct_loss_fwd(lp3, ys, lx, ly)
    c64, g64 = C.ctct_loss_fwd(lp3, ys, lx, ly, dtype=np.float64)
    np.testing.assert_allclose(c64, costs, rtol=1e-13)
    np.testing.assert_allclose(g64, grads, rtol=1e-9, atol=1e-14)
    c32, g32 = C.ctct_loss_fwd(lp3, ys, lx, ly, dtype=np.float32)
    np.testing.assert_allclose(c32, costs, rtol=1e-5)
    np.testing.assert_allclose(g32, grads, atol=1e-4)
    w = np.array([1.0, -2.0, 0.5, 3.0, 0.25])
    _, dense, _ = O.ctct_loss(joint, ys, lx, ly, reduction="none", grad_output=w)
    cd, dd = C.ctct_loss_dense(joint, ys, lx, ly, grad_out=w, dtype=np.float64)
    np.testing.assert_allclose(cd, costs, rtol=1e-13)
    np.testing.assert_allclose(dd, dense, rtol=1e-9, atol=1e-14)
    # directly against enumeration, including the no-grad (beta only) mode
    lp = log_softmax(np.random.default_rng(1).standard_normal((6, 4, 4)))
    y = np.array([[2, 2, 1]])
    ll, d = brute_force(lp, y[0])
    cd, dd = C.ctct_loss_dense(lp[None], y, [6], [3], dtype=np.float64)
    assert np.isclose(cd[0], -ll, rtol=1e-13)
    np.testing.assert_allclose(dd[0], d, rtol=1e-10, atol=1e-14)
    cn, _ = C.ctct_loss_fwd(O.gather_units(lp[None], y), y, [6], [3], requires_grad=False)
    assert np.isclose(cn[0], -ll, rtol=1e-13)


def test_c_oracle_log_matmul():
    from oracle import c_oracle as C
    rng = np.random.default_rng(2)
    lhs = rng.standard_normal((3, 6, 33)) * 4
    rhs = rng.standard_normal((3, 33, 5)) * 4
    lhs[1, 2] = -np.inf
    ref = torch.logsumexp(torch.tensor(lhs)[:, :, :, None] + torch.tensor(rhs)[:, None], dim=2).numpy()
    np.testing.assert_allclose(C.log_matmul(lhs, rhs), ref, rtol=1e-13)
    np.testing.assert_allclose(C.log_matmul(lhs, rhs, dtype=np.float32), ref, rtol=2e-6)


def test_oracle_against_committed_brute_force_vectors():
    """tests/golden/brute_force_cases.npz holds lattices whose log-likelihood
    and dense gradient were obtained by enumerating every alignment
    (tests/golden/make_brute_force_fixtures.py); the oracle must reproduce them."""
    import os
    from oracle import c_oracle as C
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                             "brute_force_cases.npz"))
    joint = z["joint"].astype(np.float64)
    _, dense, costs = O.ctct_loss(joint, z["ys"], z["lx"], z["ly"], reduction="none",
                                  grad_output=np.ones(len(z["lx"])))
    np.testing.assert_allclose(costs, -z["loglik"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dense, z["dense_grad"], rtol=0, atol=1e-12)
    c_costs, c_dense = C.ctct_loss_dense(z["joint"], z["ys"], z["lx"], z["ly"], dtype=np.float64)
    np.testing.assert_allclose(c_costs, -z["loglik"], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(c_dense, z["dense_grad"], rtol=0, atol=1e-12)
