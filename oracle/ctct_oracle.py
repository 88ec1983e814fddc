"""CPU oracle for the CTC-Transducer loss path.  TEST INFRASTRUCTURE ONLY.

This module restates, in float64 numpy, the arithmetic of the reference
(maxwellzh/warp-ctct).  It is the checker for the HIP kernels; nothing in the
shipped package imports it.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may use it.

Every function cites the reference lines it follows.  Coordinates are the
"natural" (time-synchronous) ones of ref_ctct.py:6-74, not the shifted band
storage of the CUDA kernels; the set of cells that carry probability mass is
the same (a cell outside the reference's band has alpha = -inf or beta = -inf,
hence contributes nothing to cost or gradient).

State numbering for one lattice with U labels y[0..U-1] (ref_ctct.py:26-27):
    s = 2u     "blank after u labels"          u in [0, U]
    s = 2u - 1 "inside label y[u-1]"           u in [1, U]
The per-cell log-probabilities are the three gathered entries
    LP[t, u, 0] = lp[t, u, blank]
    LP[t, u, 1] = lp[t, u, y[u-1]]   (u >= 1)   "current label"
    LP[t, u, 2] = lp[t, u, y[u]]     (u <  U)   "next label"
(warp_ctct/__init__.py:124-131, csrc/gather.cu:16-21).

Pins (see tests/test_oracle_pins.py): brute-force enumeration of every
alignment for T <= 7, reduction to torch.nn.functional.ctc_loss when the joint
does not depend on u, the closed form for lx == ly, finite differences, the
per-frame invariant sum(G[t]) == -1, and torch.logsumexp / its autograd for the
log-semiring matmul.
"""
import numpy as np

__all__ = [
    "gather_index", "gather_units", "gather_separate", "simple_units",
    "alpha_lattice", "beta_lattice", "unit_grads", "lattice_cost_and_grads",
    "scatter_units", "ctct_loss_fwd", "ctct_loss", "reduce_costs",
    "simple_unit_grad_reduce", "ctct_loss_simple_fwd", "log_matmul",
    "log_matmul_backward", "ctct_simple_loss",
]


# --------------------------------------------------------------------------
# gather stage
# --------------------------------------------------------------------------
def gather_index(ys, U1):
    """Index tensor (N, U+1, 3): [0, y[u-1], y[u]] with 0 where undefined.

    Follows warp_ctct/__init__.py:124-128 and ref_ctct.py:225-228.
    """
    ys = np.asarray(ys)
    N = ys.shape[0]
    idx = np.zeros((N, U1, 3), dtype=np.int64)
    idx[:, 1:, 1] = ys
    idx[:, :U1 - 1, 2] = ys
    return idx


def gather_units(joint, ys):
    """(N,T,U+1,V),(N,U) -> (N,T,U+1,3).  warp_ctct/__init__.py:129-131."""
    joint = np.asarray(joint)
    N, T, U1, _ = joint.shape
    idx = gather_index(ys, U1)
    idx = np.broadcast_to(idx[:, None], (N, T, U1, 3))
    return np.take_along_axis(joint, idx, axis=-1)


def gather_separate(f, g, ys):
    """f (N,T,V) -> (N,T,U+1) at [0, y0..y_{U-1}]; g (N,U+1,V) -> (N,U+1,3).

    Follows warp_ctct/__init__.py:204-215 and ref_ctct.py:206-220.
    """
    f = np.asarray(f)
    g = np.asarray(g)
    ys = np.asarray(ys)
    N, T, _ = f.shape
    U1 = g.shape[1]
    fi = np.zeros((N, T, U1), dtype=np.int64)
    fi[..., 1:] = ys[:, None, :]
    f_g = np.take_along_axis(f, fi, axis=-1)
    g_g = np.take_along_axis(g, gather_index(ys, U1), axis=-1)
    return f_g, g_g


def simple_units(f_g, g_g, den=None):
    """Per-cell log-probs of the log-add joiner, (N,T,U+1,3).

    LP[t,u,0] = f_g[t,0]   + g_g[u,0] - den[t,u]
    LP[t,u,k] = f_g[t,u+k-1] + g_g[u,k] - den[t,u]     k in {1,2}
    Follows csrc/simple.cu:20-26 (normalized) and csrc/simple_unnorm.cu:20-25
    (den omitted).  Entries the lattice never uses (u=0,k=1 and u=U,k=2) are
    set to 0.
    """
    f_g = np.asarray(f_g, dtype=np.float64)
    g_g = np.asarray(g_g, dtype=np.float64)
    N, T, U1 = f_g.shape
    lp = np.zeros((N, T, U1, 3), dtype=np.float64)
    lp[..., 0] = f_g[:, :, :1] + g_g[:, None, :, 0]
    lp[:, :, 1:, 1] = f_g[:, :, 1:] + g_g[:, None, 1:, 1]
    lp[:, :, :U1 - 1, 2] = f_g[:, :, 1:] + g_g[:, None, :U1 - 1, 2]
    if den is not None:
        lp -= np.asarray(den, dtype=np.float64)[..., None]
        lp[:, :, 0, 1] = 0.0
        lp[:, :, U1 - 1, 2] = 0.0
    return lp


# --------------------------------------------------------------------------
# one lattice
# --------------------------------------------------------------------------
def _skip_flags(ys, U):
    """skip[u] (u in [0,U]): state 2u-1 may be entered from state 2u-3.

    True iff u >= 2 and y[u-1] != y[u-2]  (ref_ctct.py:32).
    """
    skip = np.zeros(U + 1, dtype=bool)
    if U >= 2:
        skip[2:] = ys[1:U] != ys[:U - 1]
    return skip


def alpha_lattice(lp3, ys):
    """Forward variables of one lattice.

    lp3: (T, U+1, 3) float, ys: (U,) int.  Returns (alpha (T+1, 2U+1), loglik).
    alpha[t, s] = log-mass of all prefixes that consumed t frames and sit in
    state s.  Follows ref_ctct.py:6-37.
    """
    lp3 = np.asarray(lp3, dtype=np.float64)
    T, U1, _ = lp3.shape
    U = U1 - 1
    ys = np.asarray(ys)[:U]
    skip = _skip_flags(ys, U)
    a_e = np.full(U1, -np.inf)      # states 2u
    a_o = np.full(U1, -np.inf)      # states 2u-1 (index 0 unused)
    a_e[0] = 0.0                    # ref_ctct.py:16,20
    alpha = np.full((T + 1, 2 * U + 1), -np.inf)
    alpha[0, 0] = 0.0
    with np.errstate(invalid="ignore"):
        for t in range(1, T + 1):
            lp = lp3[t - 1]
            # s = 2u:  [alpha(t-1,2u) (+) alpha(t-1,2u-1)] + LP(t-1,u,0)   ref_ctct.py:28-31
            n_e = np.logaddexp(a_e, a_o) + lp[:, 0]
            # s = 2u-1: stay + LP(t-1,u,1)  (+)  from 2u-2 (+ skip from 2u-3) + LP(t-1,u-1,2)
            n_o = np.full(U1, -np.inf)
            if U >= 1:
                come = a_e[:-1].copy()
                come = np.where(skip[1:], np.logaddexp(come, a_o[:-1]), come)   # ref_ctct.py:32-36
                n_o[1:] = np.logaddexp(a_o[1:] + lp[1:, 1], come + lp[:-1, 2])
            a_e, a_o = n_e, n_o
            alpha[t, 0::2] = a_e
            alpha[t, 1::2] = a_o[1:]
    ll = alpha[T, 2 * U]
    if U >= 1:
        ll = np.logaddexp(ll, alpha[T, 2 * U - 1])                            # ref_ctct.py:37
    return alpha, ll


def beta_lattice(lp3, ys):
    """Backward variables of one lattice.

    Returns (beta (T+1, 2U+1), loglik = beta[0,0]).  beta[t, s] = log-mass of
    all completions from state s with frames t..T-1 still to emit.
    Follows ref_ctct.py:40-74.
    """
    lp3 = np.asarray(lp3, dtype=np.float64)
    T, U1, _ = lp3.shape
    U = U1 - 1
    ys = np.asarray(ys)[:U]
    skip = _skip_flags(ys, U)
    b_e = np.full(U1, -np.inf)
    b_o = np.full(U1, -np.inf)
    b_e[U] = 0.0                                                               # ref_ctct.py:52
    if U >= 1:
        b_o[U] = 0.0                                                           # ref_ctct.py:53
    beta = np.full((T + 1, 2 * U + 1), -np.inf)
    beta[T, 0::2] = b_e
    beta[T, 1::2] = b_o[1:]
    with np.errstate(invalid="ignore"):
        for t in range(T - 1, -1, -1):
            lp = lp3[t]
            nxt = np.full(U1, -np.inf)         # beta(t+1, 2u+1) + LP(t,u,2), u < U
            nxt[:-1] = b_o[1:] + lp[:-1, 2]
            stay_e = b_e + lp[:, 0]
            # s = 2u: ref_ctct.py:63-68 (even branch)
            n_e = np.logaddexp(stay_e, nxt)
            # s = 2u-1: ref_ctct.py:63-73 (odd branch): stay, to blank 2u, skip to 2u+1
            n_o = np.full(U1, -np.inf)
            if U >= 1:
                n_o[1:] = np.logaddexp(b_o[1:] + lp[1:, 1], stay_e[1:])
                sk = np.zeros(U1, dtype=bool)
                sk[1:U] = skip[2:]             # y[u-1] != y[u], u in [1, U-1]
                n_o = np.where(sk, np.logaddexp(n_o, nxt), n_o)
            b_e, b_o = n_e, n_o
            beta[t, 0::2] = b_e
            beta[t, 1::2] = b_o[1:]
    return beta, beta[0, 0]


def unit_grads(lp3, ys, alpha, beta, ll):
    """d(cost)/d(LP[t,u,k]) for one lattice, shape (T, U+1, 3); cost = -ll.

    Follows csrc/gather.cu:311-374 translated to natural coordinates:
      g0 = -exp(a(t,2u)+LP0+b(t+1,2u)-ll) - [u>=1] exp(a(t,2u-1)+LP0+b(t+1,2u)-ll)
      g1 = -exp(a(t,2u-1)+LP1+b(t+1,2u-1)-ll)                              (u>=1)
      g2 = -exp(a(t,2u)+LP2+b(t+1,2u+1)-ll)
           - [u>=1, y[u-1]!=y[u]] exp(a(t,2u-1)+LP2+b(t+1,2u+1)-ll)        (u<U)
    """
    lp3 = np.asarray(lp3, dtype=np.float64)
    T, U1, _ = lp3.shape
    U = U1 - 1
    ys = np.asarray(ys)[:U]
    skip = _skip_flags(ys, U)
    a_e = alpha[:T, 0::2]                       # (T, U+1)
    b_e = beta[1:, 0::2]
    a_o = np.full((T, U1), -np.inf)
    b_o = np.full((T, U1), -np.inf)
    a_o[:, 1:] = alpha[:T, 1::2]
    b_o[:, 1:] = beta[1:, 1::2]
    g = np.zeros((T, U1, 3))
    with np.errstate(invalid="ignore", over="ignore"):
        g[:, :, 0] = -np.exp(a_e + lp3[:, :, 0] + b_e - ll) \
                     - np.exp(a_o + lp3[:, :, 0] + b_e - ll)
        g[:, 1:, 1] = -np.exp(a_o[:, 1:] + lp3[:, 1:, 1] + b_o[:, 1:] - ll)
        if U >= 1:
            nb = b_o[:, 1:]                     # beta(t+1, 2u+1), u in [0,U-1]
            g[:, :U, 2] = -np.exp(a_e[:, :U] + lp3[:, :U, 2] + nb - ll)
            sk = np.zeros(U, dtype=bool)
            sk[1:] = skip[2:]
            g[:, :U, 2] -= np.where(sk[None, :],
                                    np.exp(a_o[:, :U] + lp3[:, :U, 2] + nb - ll), 0.0)
    return g


def lattice_cost_and_grads(lp3, ys, want_grad=True):
    """(cost, unit grads or None) of one trimmed lattice; cost = -beta(0,0)
    as in csrc/binding.cpp:86."""
    beta, ll = beta_lattice(lp3, ys)
    if not want_grad:
        return -ll, None
    alpha, _ = alpha_lattice(lp3, ys)
    return -ll, unit_grads(lp3, ys, alpha, beta, ll)


# --------------------------------------------------------------------------
# batched operator level (mirrors warp_ctct._C)
# --------------------------------------------------------------------------
def ctct_loss_fwd(lp3, ys, lx, ly, requires_grad=True):
    """Mirror of _C.ctct_loss_fwd (csrc/binding.cpp:31-100).

    lp3 (N,T,U+1,3), ys (N,U), lx (N,), ly (N,) -> costs (N,), grads
    (N,T,U+1,3) zero outside t<lx, u<=ly (binding.cpp:89 zeros_like +
    gather.cu:321 early return).
    """
    lp3 = np.asarray(lp3, dtype=np.float64)
    N, T, U1, _ = lp3.shape
    costs = np.zeros(N)
    grads = np.zeros_like(lp3) if requires_grad else None
    for n in range(N):
        t, u = int(lx[n]), int(ly[n])
        c, g = lattice_cost_and_grads(lp3[n, :t, :u + 1], np.asarray(ys[n])[:u], requires_grad)
        costs[n] = c
        if requires_grad:
            grads[n, :t, :u + 1] = g
    return costs, grads


def scatter_units(unit_g, ys, V):
    """Backward of the gather: dense (N,T,U+1,V) from unit grads (N,T,U+1,3).

    zeros + scatter_add along V with the gather index (autograd of
    warp_ctct/__init__.py:131); coincident indices add.
    """
    unit_g = np.asarray(unit_g, dtype=np.float64)
    N, T, U1, _ = unit_g.shape
    idx = gather_index(ys, U1)
    dense = np.zeros((N, T, U1, V))
    n_i, u_i = np.meshgrid(np.arange(N), np.arange(U1), indexing="ij")
    for k in range(3):
        # (N, U1) index into V, broadcast over T
        for t in range(T):
            np.add.at(dense[:, t], (n_i, u_i, idx[:, :, k]), unit_g[:, t, :, k])
    return dense


def reduce_costs(costs, lx, reduction="mean", average_frames=False):
    """warp_ctct/__init__.py:138-147 (same code at :227-236)."""
    costs = np.asarray(costs, dtype=np.float64)
    if average_frames:
        costs = costs / np.asarray(lx, dtype=np.float64)
    if reduction == "none" or reduction is None:
        return costs
    if reduction == "sum":
        return costs.sum()
    if reduction == "mean":
        return costs.mean()
    return costs


def ctct_loss(joint, ys, lx, ly, reduction="mean", average_frames=False, grad_output=None):
    """Public-API level oracle: loss and dense d(loss)/d(joint).

    warp_ctct/__init__.py:88-147 plus its autograd (CTCTLoss.backward :30-33,
    gather backward).  grad_output, if given, is d(final)/d(costs[n]) applied
    instead of the reduction's own weights.
    """
    joint = np.asarray(joint, dtype=np.float64)
    N, T, U1, V = joint.shape
    lp3 = gather_units(joint, ys)
    costs, g = ctct_loss_fwd(lp3, ys, lx, ly, True)
    loss = reduce_costs(costs, lx, reduction, average_frames)
    if grad_output is None:
        w = np.ones(N)
        if average_frames:
            w = w / np.asarray(lx, dtype=np.float64)
        if reduction == "mean":
            w = w / N
    else:
        w = np.asarray(grad_output, dtype=np.float64)
    dense = scatter_units(g * w[:, None, None, None], ys, V)
    return loss, dense, costs


# --------------------------------------------------------------------------
# simple (log-add joiner) path
# --------------------------------------------------------------------------
def ctct_loss_with_logits(logits, ys, lx, ly, reduction="mean", average_frames=False,
                          grad_output=None):
    """ctct_loss on log_softmax(logits) and its gradient wrt the logits.

    What a caller of the reference computes as
    warp_ctct.ctct_loss(logits.log_softmax(-1), ...) (warp_ctct/__init__.py:88-147)
    plus autograd through log_softmax: with G = d(loss)/d(log_probs),
    d(loss)/d(logits) = G - softmax(logits) * sum_v G.
    Returns (loss, grad_logits, costs).
    """
    logits = np.asarray(logits, dtype=np.float64)
    m = logits.max(axis=-1, keepdims=True)
    lse = m + np.log(np.exp(logits - m).sum(axis=-1, keepdims=True))
    log_probs = logits - lse
    loss, G, costs = ctct_loss(log_probs, ys, lx, ly, reduction, average_frames, grad_output)
    grad = G - np.exp(log_probs) * G.sum(axis=-1, keepdims=True)
    return loss, grad, costs


def simple_unit_grad_reduce(g, normalized):
    """Unit grads (N,T,U+1,3) -> (grad_f_g (N,T,U+1), grad_g_g (N,U+1,3),
    grad_den (N,T,U+1) or None).  Follows csrc/binding.cpp:198-219."""
    N, T, U1, _ = g.shape
    grad_den = -g.sum(3) if normalized else None
    grad_g = g.sum(1)
    grad_f = np.zeros((N, T, U1))
    grad_f[..., 0] = g[..., 0].sum(2)
    grad_f[..., 1:] = g[:, :, 1:, 1] + g[:, :, :U1 - 1, 2]
    return grad_f, grad_g, grad_den


def ctct_loss_simple_fwd(f_g, g_g, ys, den, lx, ly, requires_grad=True):
    """Mirror of _C.ctct_loss_simple_fwd (csrc/binding.cpp:103-222)."""
    normalized = den is not None and np.ndim(den) == 3
    lp3 = simple_units(f_g, g_g, den if normalized else None)
    costs, g = ctct_loss_fwd(lp3, ys, lx, ly, requires_grad)
    if not requires_grad:
        return costs, None, None, None
    gf, gg, gd = simple_unit_grad_reduce(g, normalized)
    return costs, gf, gg, gd


def log_matmul(lhs, rhs):
    """res[b,i,j] = logsumexp_k(lhs[b,i,k] + rhs[b,k,j]).

    csrc/logmatmul.cu:44-146; all -inf terms give -inf (:142-144).
    """
    lhs = np.asarray(lhs, dtype=np.float64)
    rhs = np.asarray(rhs, dtype=np.float64)
    B, M, K = lhs.shape
    Nn = rhs.shape[2]
    out = np.empty((B, M, Nn))
    with np.errstate(invalid="ignore", divide="ignore"):
        for b in range(B):
            for j in range(Nn):
                s = lhs[b] + rhs[b, :, j][None, :]            # (M, K)
                m = s.max(axis=1)
                ms = np.where(np.isfinite(m), m, 0.0)
                out[b, :, j] = np.log(np.exp(s - ms[:, None]).sum(axis=1)) + ms
                out[b, :, j] = np.where(m == -np.inf, -np.inf, out[b, :, j])
    return out


def log_matmul_backward(grad_out, lhs, rhs, res):
    """grad_lhs[b,i,k] = sum_j grad_out[b,i,j] exp(lhs[b,i,k]+rhs[b,k,j]-res[b,i,j]),
    grad_rhs[b,k,j] = sum_i (same term).  The value csrc/binding.cpp:247-324
    computes through its positive/negative log split."""
    grad_out = np.asarray(grad_out, dtype=np.float64)
    lhs = np.asarray(lhs, dtype=np.float64)
    rhs = np.asarray(rhs, dtype=np.float64)
    res = np.asarray(res, dtype=np.float64)
    B, M, K = lhs.shape
    gl = np.zeros_like(lhs)
    gr = np.zeros_like(rhs)
    with np.errstate(invalid="ignore", over="ignore"):
        for b in range(B):
            for i in range(M):
                # (K, Nn)
                w = np.exp(lhs[b, i][:, None] + rhs[b] - res[b, i][None, :])
                w = np.where(np.isfinite(w), w, 0.0) * grad_out[b, i][None, :]
                gl[b, i] = w.sum(1)
                gr[b] += w
    return gl, gr


def ctct_simple_loss(f, g, ys, lx, ly, reduction="mean", average_frames=False,
                     normalized=True, grad_output=None):
    """Public-API level oracle of ctct_simple_loss and its autograd:
    returns (loss, grad_f (N,T,V), grad_g (N,U+1,V), costs).
    warp_ctct/__init__.py:150-236 with SimpleCTCTLoss (:55-85), LogMMExp
    (:36-52) and the two gather backwards."""
    f = np.asarray(f, dtype=np.float64)
    g = np.asarray(g, dtype=np.float64)
    ys = np.asarray(ys)
    N, T, V = f.shape
    U1 = g.shape[1]
    den = log_matmul(f, np.swapaxes(g, 1, 2)) if normalized else None
    f_g, g_g = gather_separate(f, g, ys)
    costs, gf_g, gg_g, gden = ctct_loss_simple_fwd(f_g, g_g, ys, den, lx, ly, True)
    loss = reduce_costs(costs, lx, reduction, average_frames)
    if grad_output is None:
        w = np.ones(N)
        if average_frames:
            w = w / np.asarray(lx, dtype=np.float64)
        if reduction == "mean":
            w = w / N
    else:
        w = np.asarray(grad_output, dtype=np.float64)
    w3 = w[:, None, None]
    grad_f = np.zeros_like(f)
    grad_g = np.zeros_like(g)
    fi = np.zeros((N, T, U1), dtype=np.int64)
    fi[..., 1:] = ys[:, None, :]
    gi = gather_index(ys, U1)
    for n in range(N):
        for t in range(T):
            np.add.at(grad_f[n, t], fi[n, t], gf_g[n, t] * w[n])
        for u in range(U1):
            np.add.at(grad_g[n, u], gi[n, u], gg_g[n, u] * w[n])
    if normalized:
        gl, gr = log_matmul_backward(gden * w3, f, np.swapaxes(g, 1, 2), den)
        grad_f += gl
        grad_g += np.swapaxes(gr, 1, 2)
    return loss, grad_f, grad_g, costs
