"""Seeded synthetic inputs shared by the tests, plus a brute-force enumerator
that is independent of any lattice recursion."""
import itertools

import numpy as np


def log_softmax(x, axis=-1):
    x = np.asarray(x, dtype=np.float64)
    m = x.max(axis=axis, keepdims=True)
    return x - m - np.log(np.exp(x - m).sum(axis=axis, keepdims=True))


def make_joint_case(seed, N, T, U, V, lx=None, ly=None, sigma=1.0, force_repeat=True,
                    dtype=np.float32, zero_pad=True):
    """Joint log-probs (N,T,U+1,V) = log_softmax of N(0,sigma) logits, labels
    uniform in [1,V-1], lengths drawn from a Python range, or given explicitly."""
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((N, T, U + 1, V)) * sigma
    joint = log_softmax(logits).astype(dtype)
    ys = rng.integers(1, V, size=(N, U)).astype(np.int32)
    lx = _lengths(rng, lx, N, T)
    ly = _lengths(rng, ly, N, U)
    if force_repeat and U >= 2:
        for n in range(N):
            if ly[n] >= 2:
                p = int(rng.integers(0, ly[n] - 1))
                ys[n, p + 1] = ys[n, p]
    # feasibility: need lx >= ly + number of adjacent repeats
    for n in range(N):
        rep = int(np.sum(ys[n, 1:ly[n]] == ys[n, :ly[n] - 1])) if ly[n] >= 2 else 0
        if lx[n] < ly[n] + rep:
            lx[n] = min(T, ly[n] + rep)
            if lx[n] < ly[n] + rep:
                ly[n] = max(1, lx[n] - rep - 1)
    if zero_pad:
        for n in range(N):
            joint[n, lx[n]:] = 0
            joint[n, :, ly[n] + 1:] = 0
    return joint, ys, lx.astype(np.int32), ly.astype(np.int32)


def _lengths(rng, spec, N, full):
    """None -> all `full`; a Python range -> uniform draw from it with the
    maximum forced to appear once; anything else -> taken as the lengths."""
    if spec is None:
        return np.full(N, full, dtype=np.int64)
    if isinstance(spec, range):
        out = rng.integers(spec.start, spec.stop, size=N)
        out[int(rng.integers(0, N))] = spec.stop - 1
        return out
    return np.asarray(spec, dtype=np.int64).copy()


def make_simple_case(seed, N, T, U, V, lx=None, ly=None, normalized=True, dtype=np.float32):
    """f (N,T,V), g (N,U+1,V): log_softmax of N(0,1) if normalized else raw scores."""
    rng = np.random.default_rng(seed)
    f = rng.standard_normal((N, T, V))
    g = rng.standard_normal((N, U + 1, V))
    if normalized:
        f = log_softmax(f)
        g = log_softmax(g)
    ys = rng.integers(1, V, size=(N, U)).astype(np.int32)
    lx = _lengths(rng, lx, N, T)
    ly = _lengths(rng, ly, N, U)
    if U >= 2:
        for n in range(N):
            if ly[n] >= 2:
                p = int(rng.integers(0, ly[n] - 1))
                ys[n, p + 1] = ys[n, p]
    for n in range(N):
        rep = int(np.sum(ys[n, 1:ly[n]] == ys[n, :ly[n] - 1])) if ly[n] >= 2 else 0
        if lx[n] < ly[n] + rep:
            lx[n] = min(T, ly[n] + rep)
    return f.astype(dtype), g.astype(dtype), ys, lx.astype(np.int32), ly.astype(np.int32)


def collapse(z):
    """CTC collapse: merge repeats, then drop blanks (0)."""
    out = []
    prev = None
    for tok in z:
        if tok != prev and tok != 0:
            out.append(tok)
        prev = tok
    return out


def brute_force(lp, ys):
    """Enumerate every alignment of one lattice.

    lp: (T, U+1, V) log-probs, ys: (U,) labels.  An alignment is a token per
    frame whose CTC collapse equals ys; the token at frame t is scored with
    context u_t = number of labels started before frame t (README.md:4-13 of
    the reference: label context like RNN-T, frame alignment like CTC).
    Returns (loglik, dense d(-loglik)/d(lp)).
    """
    lp = np.asarray(lp, dtype=np.float64)
    T, U1, V = lp.shape
    ys = [int(v) for v in ys]
    alphabet = sorted(set(ys) | {0})
    total = 0.0
    mass = np.zeros_like(lp)
    for z in itertools.product(alphabet, repeat=T):
        if collapse(z) != ys:
            continue
        u = 0
        score = 0.0
        cells = []
        prev = None
        for t, tok in enumerate(z):
            score += lp[t, u, tok]
            cells.append((t, u, tok))
            if tok != 0 and tok != prev:
                u += 1
            prev = tok
        p = np.exp(score)
        total += p
        for c in cells:
            mass[c] += p
    if total == 0.0:
        return -np.inf, mass
    return np.log(total), -mass / total
