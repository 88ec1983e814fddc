"""GPU parity tests of the ctct_loss path: HIP kernels (through the C ABI and
through the warp_ctct Python API) against the float64 oracle on identical
seeded inputs.

Tolerances (from the build's north star): loss relative error <= 1e-5,
gradient absolute error <= 1e-4, both in fp32 against the float64 oracle.
Integer/structural facts (which cells are -inf, which gradient entries are
exactly zero) are compared exactly."""
import ctypes
import math

import numpy as np
import pytest
import torch

import hip_lib
from ctct_cases import make_joint_case
from oracle import c_oracle as C
from oracle import ctct_oracle as O

pytestmark = pytest.mark.gpu

LOSS_RTOL = 1e-5
GRAD_ATOL = 1e-4
LN2 = math.log(2.0)
LOG2E = np.float64(1.4426950408889634074)


def assert_support(got, ref, what, underflow=1e-30):
    """Structural zeros of the oracle are exact zeros here; an exact zero here
    is either structural or an underflow of a negligible value (below
    `underflow`: fp32's range by default)."""
    assert np.all(got[ref == 0] == 0), what + ": non-zero where the oracle has a structural zero"
    assert np.all(np.abs(ref[got == 0]) < underflow), what + ": zero where the oracle has mass"


def dev(a, dtype=None):
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def run_stages(joint, ys, lx, ly, beta_only=False):
    """Call every stage through the C ABI; returns numpy views of all buffers."""
    lib = hip_lib.lib()
    N, T, U1, V = joint.shape
    U = U1 - 1
    s = hip_lib.stream_ptr()
    d_joint, d_ys, d_lx, d_ly = dev(joint), dev(ys), dev(lx), dev(ly)
    f64 = dict(device="cuda", dtype=torch.float64)
    P = lib.warpctct_padded_contexts(U)           # contexts per frame in the work buffers
    assert P % 64 == 0 and U1 <= P < U1 + 64
    units = torch.full((N, T, P, 3), float("nan"), **f64)
    alphas = torch.full((N, T + 1, P, 2), float("nan"), **f64)
    betas = torch.full((N, T + 1, P, 2), float("nan"), **f64)
    costs = torch.full((N,), float("nan"), device="cuda")
    ug = torch.full((N, T, U1, 3), float("nan"), device="cuda")
    p = hip_lib.ptr
    hip_lib.check(lib.warpctct_gather_units_f32(p(d_joint), p(d_ys), p(d_lx), p(d_ly), p(units),
                                                N, T, U, V, s))
    lib.warpctct_lattice_relay_bytes.restype = ctypes.c_size_t
    relay_bytes = lib.warpctct_lattice_relay_bytes(N, T, U)
    relay = torch.empty(max(relay_bytes, 8), dtype=torch.uint8, device="cuda")
    hip_lib.check(lib.warpctct_lattice_f32(p(units), p(d_ys), p(d_lx), p(d_ly),
                                           p(None if beta_only else alphas), p(betas), p(costs),
                                           N, T, U, int(beta_only), p(relay),
                                           ctypes.c_size_t(relay_bytes), s))
    if not beta_only:
        hip_lib.check(lib.warpctct_unit_grads_f32(p(units), p(d_ys), p(d_lx), p(d_ly), p(alphas),
                                                  p(betas), p(ug), N, T, U, s))
    torch.cuda.synchronize()
    out = dict(units=units, alphas=alphas, betas=betas, costs=costs, unit_grads=ug)
    return {k: v.cpu().numpy() for k, v in out.items()}


def check_lattice(name, stored, ref, lx, ly):
    """stored (N,T+1,U+1,2) {o,e} in log2 units; ref[n] (lx+1, 2ly+1) natural
    log.  Same -inf cells ("identical lattice paths"), finite cells within
    2e-5 absolute (the values are O(1000))."""
    for n in range(stored.shape[0]):
        t, u = int(lx[n]), int(ly[n])
        got = np.full((t + 1, 2 * u + 1), np.nan)
        val = stored[n, :t + 1, :u + 1] * LN2
        got[:, 0::2] = val[:, :, 1]
        got[:, 1::2] = val[:, 1:, 0]
        assert np.all(np.isneginf(stored[n, :t + 1, 0, 0])), name + ": state -1 must be -inf"
        r = ref[n]
        assert np.array_equal(np.isneginf(got), np.isneginf(r)), name + ": live-cell pattern differs"
        fin = np.isfinite(r)
        np.testing.assert_allclose(got[fin], r[fin], rtol=0, atol=2e-5, err_msg=name)


CASES = [
    # name, seed, N, T, U, V, lx, ly, sigma
    ("c1_reference_config", 1, 2, 40, 10, 32, None, None, 1.0),
    ("ragged_small", 2, 5, 23, 7, 16, range(9, 24), range(1, 8), 1.0),
    ("single_label", 3, 3, 6, 1, 5, [6, 3, 1], [1, 1, 1], 1.0),
    ("lx_equals_ly", 4, 2, 9, 9, 12, [9, 9], [9, 9], 1.0),
    ("two_contexts_per_lane", 5, 3, 150, 100, 48, range(120, 151), range(64, 101), 1.0),
    ("three_contexts_per_lane", 6, 2, 200, 160, 24, range(180, 201), range(129, 161), 2.0),
    ("five_contexts_per_lane", 7, 2, 340, 300, 12, [340, 331], [300, 257], 1.0),
    ("odd_vocab_scalar_stores", 8, 3, 17, 5, 37, range(8, 18), range(2, 6), 1.0),
    ("vocab_1024_vector_stores", 9, 2, 30, 12, 1024, [30, 21], [12, 7], 1.0),
    ("peaky", 10, 4, 60, 20, 64, range(40, 61), range(10, 21), 4.0),
    # lattices of several wavefronts whose samples are short: fewer frames than
    # one hand-over chunk, a single partial chunk, one frame more than a chunk,
    # and samples with 0..2 labels (the upper wavefronts hold only padding)
    ("two_wavefronts_short_samples", 301, 6, 20, 100, 16, [1, 5, 8, 9, 17, 20], [0, 2, 1, 5, 2, 18], 1.0),
    ("three_wavefronts_short_samples", 302, 5, 17, 150, 8, [1, 5, 8, 9, 17], [1, 0, 2, 2, 1], 1.0),
    ("five_wavefronts_mixed_lengths", 303, 4, 310, 300, 8, [310, 1, 5, 9], [300, 0, 2, 1], 1.0),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_stages_against_oracle(case):
    name, seed, N, T, U, V, lx, ly, sigma = case
    joint, ys, lx, ly = make_joint_case(seed, N, T, U, V, lx=lx, ly=ly, sigma=sigma)
    got = run_stages(joint, ys, lx, ly)
    # gather: exact (the gathered fp32 value times log2(e), in double)
    lp3 = O.gather_units(joint, ys)
    for n in range(N):
        t, u = int(lx[n]), int(ly[n])
        exp = lp3[n, :t, :u + 1].astype(np.float64) * LOG2E
        g = got["units"][n, :t, :u + 1]
        np.testing.assert_array_equal(g[..., 0], exp[..., 0])
        np.testing.assert_array_equal(g[:, 1:, 1], exp[:, 1:, 1])
        np.testing.assert_array_equal(g[:, :u, 2], exp[:, :u, 2])
        # no label follows the last one; padding contexts are neutral; frames
        # beyond lx are never written
        assert np.all(np.isneginf(g[:, u, 2]))
        pad = got["units"][n, :t, u + 1:]
        assert np.all(pad[..., :2] == 0) and np.all(np.isneginf(pad[..., 2]))
        assert np.all(np.isnan(got["units"][n, t:]))
    # lattices
    ref_a, ref_b = [], []
    for n in range(N):
        t, u = int(lx[n]), int(ly[n])
        a, ll_a = O.alpha_lattice(lp3[n, :t, :u + 1], ys[n, :u])
        b, ll_b = O.beta_lattice(lp3[n, :t, :u + 1], ys[n, :u])
        ref_a.append(a)
        ref_b.append(b)
    check_lattice("alpha", got["alphas"], ref_a, lx, ly)
    check_lattice("beta", got["betas"], ref_b, lx, ly)
    # costs and unit gradients
    costs, grads = O.ctct_loss_fwd(lp3, ys, lx, ly)
    np.testing.assert_allclose(got["costs"], costs, rtol=LOSS_RTOL)
    np.testing.assert_allclose(got["unit_grads"], grads, atol=GRAD_ATOL, rtol=0)
    assert_support(got["unit_grads"], grads, "unit grads")
    # beta-only mode gives the same costs bit for bit
    again = run_stages(joint, ys, lx, ly, beta_only=True)
    np.testing.assert_array_equal(again["costs"], got["costs"])


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_public_api_loss_and_dense_grad(case):
    import warp_ctct
    name, seed, N, T, U, V, lx, ly, sigma = case
    joint, ys, lx, ly = make_joint_case(seed, N, T, U, V, lx=lx, ly=ly, sigma=sigma)
    rng = np.random.default_rng(seed)
    w = rng.standard_normal(N)
    ref_loss, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="none", grad_output=w)
    x = dev(joint).requires_grad_(True)
    costs = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="none")
    (costs * dev(w, torch.float32)).sum().backward()
    np.testing.assert_allclose(costs.detach().cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
    g = x.grad.cpu().numpy()
    assert g.shape == joint.shape and x.grad.dtype == torch.float32
    np.testing.assert_allclose(g, ref_dense, atol=GRAD_ATOL * max(1.0, np.abs(w).max()), rtol=0)
    assert_support(g, ref_dense, "dense gradient")


def test_repeated_label_columns_add():
    """y[u-1] == y[u]: units k=1 and k=2 of context u land in the same column."""
    joint, ys, lx, ly = make_joint_case(12, 1, 8, 3, 8, force_repeat=False)
    ys[0] = [3, 3, 5]
    import warp_ctct
    x = dev(joint).requires_grad_(True)
    loss = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="sum")
    loss.backward()
    _, dense, _ = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    lp3 = O.gather_units(joint, ys)
    _, ug = O.ctct_loss_fwd(lp3, ys, lx, ly)
    # context 1 has current label 3 and next label 3
    np.testing.assert_allclose(dense[0, :, 1, 3], ug[0, :, 1, 1] + ug[0, :, 1, 2], rtol=1e-12)
    assert np.any(ug[0, :, 1, 1] != 0) and np.any(ug[0, :, 1, 2] != 0)
    np.testing.assert_allclose(x.grad.cpu().numpy(), dense, atol=GRAD_ATOL, rtol=0)


@pytest.mark.parametrize("reduction", ["none", "sum", "mean", None])
@pytest.mark.parametrize("average_frames", [False, True])
def test_reduction_and_average_frames(reduction, average_frames):
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(13, 4, 19, 6, 11, lx=range(10, 20), ly=range(2, 7))
    ref_loss, ref_dense, _ = O.ctct_loss(joint, ys, lx, ly, reduction=reduction,
                                         average_frames=average_frames)
    x = dev(joint).requires_grad_(True)
    loss = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction=reduction,
                               average_frames=average_frames)
    np.testing.assert_allclose(loss.detach().cpu().numpy(), ref_loss, rtol=LOSS_RTOL)
    if reduction in ("none", None):
        assert loss.shape == (4,)
        loss.sum().backward()
    else:
        assert loss.dim() == 0
        loss.backward()
    np.testing.assert_allclose(x.grad.cpu().numpy(), ref_dense, atol=GRAD_ATOL, rtol=0)


def test_no_grad_and_int64_lengths_and_half_input():
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(14, 3, 21, 5, 9, lx=range(11, 22), ly=range(2, 6))
    _, _, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="none")
    x = dev(joint)
    c1 = warp_ctct.ctct_loss(x, dev(ys).long(), dev(lx).long(), dev(ly).long(), reduction="none")
    assert not c1.requires_grad
    np.testing.assert_allclose(c1.cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
    xr = dev(joint).requires_grad_(True)
    with torch.no_grad():
        c2 = warp_ctct.ctct_loss(xr, dev(ys), dev(lx), dev(ly), reduction="none")
    assert not c2.requires_grad
    np.testing.assert_array_equal(c2.cpu().numpy(), c1.cpu().numpy())
    # a half-precision joint is computed in fp32 and gets a half gradient back
    xh = dev(joint).half().requires_grad_(True)
    _, _, ref_h = O.ctct_loss(xh.detach().float().cpu().numpy(), ys, lx, ly, reduction="none")
    ch = warp_ctct.ctct_loss(xh, dev(ys), dev(lx), dev(ly), reduction="none")
    assert ch.dtype == torch.float32
    np.testing.assert_allclose(ch.detach().cpu().numpy(), ref_h, rtol=LOSS_RTOL)
    ch.sum().backward()
    assert xh.grad.dtype == torch.float16 and xh.grad.shape == xh.shape


HALF_TYPES = [
    # torch dtype, relative spacing of the type (one unit in the last place)
    (torch.float16, 2.0 ** -10),
    (torch.bfloat16, 2.0 ** -7),
]


@pytest.mark.parametrize("dtype,ulp", HALF_TYPES, ids=["float16", "bfloat16"])
@pytest.mark.parametrize("reduction", ["none", "mean"])
def test_half_precision_joint_is_read_and_written_natively(dtype, ulp, reduction):
    """A float16 / bfloat16 joint: the loss is that of the rounded inputs,
    computed in float32 (the reference casts after its gather,
    warp_ctct/__init__.py:135), and the gradient comes back in the input's
    type.  Every gradient element must be the float64 oracle's value rounded
    to the type: within one unit in the last place (half an ulp of rounding
    plus the fp32 error of the value), structural zeros exact.  Odd V makes
    rows start at 2-byte, not 4-byte, aligned addresses."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(31, 4, 26, 9, 33, lx=range(14, 27), ly=range(3, 10))
    xh = dev(joint).to(dtype).requires_grad_(True)
    rounded = xh.detach().double().cpu().numpy()
    w = np.linspace(0.5, 2.0, 4)
    ref_loss, ref_dense, _ = O.ctct_loss(rounded, ys, lx, ly, reduction=reduction,
                                         grad_output=w if reduction == "none" else None)
    loss = warp_ctct.ctct_loss(xh, dev(ys), dev(lx), dev(ly), reduction=reduction)
    assert loss.dtype == torch.float32
    np.testing.assert_allclose(loss.detach().cpu().numpy(), ref_loss, rtol=LOSS_RTOL)
    if reduction == "none":
        loss.backward(dev(w, torch.float32))
    else:
        loss.backward()
    assert xh.grad.dtype == dtype and xh.grad.shape == xh.shape
    got = xh.grad.double().cpu().numpy()
    tiny = 1e-7 if dtype == torch.float16 else 1e-30   # float16 subnormals end at 6e-8
    assert_support(got, ref_dense, "half dense gradient", underflow=tiny)
    assert np.all(np.abs(got - ref_dense) <= ulp * np.abs(ref_dense) + tiny)
    # and it is the float32 path's gradient, rounded once
    x32 = xh.detach().float().requires_grad_(True)
    loss32 = warp_ctct.ctct_loss(x32, dev(ys), dev(lx), dev(ly), reduction=reduction)
    if reduction == "none":
        loss32.backward(dev(w, torch.float32))
    else:
        loss32.backward()
    assert torch.equal(xh.grad, x32.grad.to(dtype))
    assert torch.equal(loss, loss32)


@pytest.mark.parametrize("dtype,V", [(torch.float32, 96), (torch.float32, 1024), (torch.bfloat16, 192),
                                     (torch.float16, 128), (torch.float32, 48)],
                         ids=["f32_3_lines", "f32_32_lines", "bf16_3_lines", "f16_2_lines", "f32_not_line_sized"])
def test_dense_gradient_rows_written_as_whole_lines(dtype, V):
    """The sparse pass of the dense gradient writes the 128-byte line around
    each non-zero element (rows that are not a whole number of lines: single
    elements).  Labels are placed so that a row's non-zero columns share the
    blank's line, share one other line, sit on both sides of a line boundary,
    and coincide (a repeated label); every element of the result, the zeros
    around the values included, must match the oracle."""
    import warp_ctct
    per_line = 128 // torch.empty(0, dtype=dtype).element_size()
    N, T, U = 2, 14, 8
    joint, ys, lx, ly = make_joint_case(81, N, T, U, V, lx=[14, 12], ly=[8, 7], force_repeat=False)
    edge = min(per_line, V - 2)
    ys[0] = [1, 2, edge - 1, edge, edge + 1, edge + 1, V - 1, 3]          # a repeat at positions 4, 5
    ys[1] = [V - 1, V - 2, edge, 1, edge - 1, 5, 5, 0][:U]
    ys[1, 7] = 1
    xh = dev(joint).to(dtype).requires_grad_(True)
    rounded = xh.detach().double().cpu().numpy()
    w = np.array([1.5, -0.75])
    _, ref_dense, ref_costs = O.ctct_loss(rounded, ys, lx, ly, reduction="none", grad_output=w)
    assert np.all(np.isfinite(ref_costs))
    loss = warp_ctct.ctct_loss(xh, dev(ys), dev(lx), dev(ly), reduction="none")
    loss.backward(dev(w, torch.float32))
    got = xh.grad.double().cpu().numpy()
    ulp = {torch.float32: 2.0 ** -23, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    tiny = 1e-7 if dtype == torch.float16 else 1e-30
    assert_support(got, ref_dense, "dense gradient", underflow=tiny)
    assert np.all(np.abs(got - ref_dense) <= ulp * np.abs(ref_dense) + max(tiny, 2e-6))


def test_double_joint_is_converted_like_the_reference():
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(32, 2, 12, 4, 7)
    xd = dev(joint).double().requires_grad_(True)
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    loss = warp_ctct.ctct_loss(xd, dev(ys), dev(lx), dev(ly), reduction="sum")
    np.testing.assert_allclose(loss.item(), ref_costs.sum(), rtol=LOSS_RTOL)
    loss.backward()
    assert xd.grad.dtype == torch.float64
    np.testing.assert_allclose(xd.grad.cpu().numpy(), ref_dense, atol=GRAD_ATOL, rtol=0)


def test_batch_reduction_is_deterministic_and_handles_large_batches():
    """The in-kernel sum over the batch adds in a fixed order: two calls give
    the same bits, for a batch larger than one wavefront too."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(33, 150, 9, 3, 6, lx=range(4, 10), ly=range(1, 4))
    _, _, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="none")
    x = dev(joint)
    for reduction, ref in (("sum", ref_costs.sum()), ("mean", ref_costs.mean())):
        a = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction=reduction)
        b = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction=reduction)
        assert a.dim() == 0 and torch.equal(a, b)
        np.testing.assert_allclose(a.item(), ref, rtol=LOSS_RTOL)
    af = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="mean", average_frames=True)
    np.testing.assert_allclose(af.item(), (ref_costs / lx).mean(), rtol=LOSS_RTOL)


LOGITS_CASES = [
    # name, seed, N, T, U, V, lx, ly, sigma, dtype
    ("small_f32", 41, 3, 17, 5, 37, range(8, 18), range(2, 6), 2.0, torch.float32),
    ("vector_rows_f32", 42, 2, 30, 12, 1024, [30, 21], [12, 7], 3.0, torch.float32),
    ("two_wavefronts_f32", 43, 2, 90, 70, 24, [90, 80], [70, 66], 1.0, torch.float32),
    ("bf16", 44, 3, 20, 6, 64, range(10, 21), range(2, 7), 2.0, torch.bfloat16),
    ("f16_odd_vocab", 45, 2, 14, 4, 33, [14, 9], [4, 3], 2.0, torch.float16),
    # rows of 2-byte elements read as 16-byte vectors: one vector, and more than
    # one round of 1024 elements with a partial last round
    ("f16_vector_rows", 48, 2, 14, 4, 8, [14, 9], [4, 3], 2.0, torch.float16),
    ("f16_vector_rows_two_rounds", 49, 2, 9, 3, 1096, [9, 6], [3, 2], 2.0, torch.float16),
    ("bf16_vector_rows_two_rounds", 50, 2, 9, 3, 1096, [9, 6], [3, 2], 2.0, torch.bfloat16),
    # a frame whose units do not fit the kernel's LDS staging (more than 2340
    # contexts): results stored row by row
    ("frame_wider_than_lds_f32", 47, 2, 36, 2400, 8, [36, 30], [24, 9], 1.5, torch.float32),
    ("frame_wider_than_lds_f16", 51, 2, 36, 2400, 16, [36, 30], [24, 9], 1.5, torch.float16),
    ("frame_wider_than_lds_bf16_odd_vocab", 52, 2, 36, 2400, 7, [36, 30], [24, 9], 1.5, torch.bfloat16),
]


@pytest.mark.parametrize("case", LOGITS_CASES, ids=[c[0] for c in LOGITS_CASES])
@pytest.mark.parametrize("reduction", ["none", "mean"])
def test_loss_with_logits(case, reduction):
    """ctct_loss_with_logits(x) == ctct_loss(log_softmax(x)): loss and
    d(loss)/d(logits) against the float64 oracle on the same (rounded)
    logits; rows of padding and rows outside the band get exact zeros."""
    import warp_ctct
    _, seed, N, T, U, V, lxs, lys, sigma, dtype = case
    _, ys, lx, ly = make_joint_case(seed, N, T, U, V, lx=lxs, ly=lys)
    rng = np.random.default_rng(seed)
    logits = (rng.standard_normal((N, T, U + 1, V)) * sigma + rng.standard_normal((N, T, U + 1, 1)) * 5)
    x = dev(logits.astype(np.float32)).to(dtype).requires_grad_(True)
    rounded = x.detach().double().cpu().numpy()
    w = np.linspace(0.5, 2.0, N)
    ref_loss, ref_grad, _ = O.ctct_loss_with_logits(
        rounded, ys, lx, ly, reduction, False, grad_output=w if reduction == "none" else None)
    loss = warp_ctct.ctct_loss_with_logits(x, dev(ys), dev(lx), dev(ly), reduction=reduction)
    assert loss.dtype == torch.float32
    np.testing.assert_allclose(loss.detach().cpu().numpy(), ref_loss, rtol=LOSS_RTOL)
    if reduction == "none":
        loss.backward(dev(w, torch.float32))
    else:
        loss.backward()
    assert x.grad.dtype == dtype and x.grad.shape == x.shape
    got = x.grad.double().cpu().numpy()
    ulp = {torch.float32: 0.0, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    assert np.all(np.abs(got - ref_grad) <= GRAD_ATOL + ulp * np.abs(ref_grad))
    dead = np.abs(ref_grad).sum(-1) == 0
    assert np.all(got[dead] == 0), "rows without gradient must be exact zeros"
    # the unfused route through torch.log_softmax gives the same loss
    with torch.no_grad():
        unfused = warp_ctct.ctct_loss(x.float().log_softmax(-1), dev(ys), dev(lx), dev(ly),
                                      reduction=reduction)
        fused = warp_ctct.ctct_loss_with_logits(x, dev(ys), dev(lx), dev(ly), reduction=reduction)
    assert not fused.requires_grad
    np.testing.assert_allclose(fused.cpu().numpy(), unfused.cpu().numpy(), rtol=LOSS_RTOL)


def test_loss_with_logits_average_frames_and_sum():
    import warp_ctct
    _, ys, lx, ly = make_joint_case(46, 4, 15, 4, 19, lx=range(7, 16), ly=range(1, 5))
    logits = np.random.default_rng(46).standard_normal((4, 15, 5, 19)).astype(np.float32) * 2
    x = dev(logits).requires_grad_(True)
    ref_loss, ref_grad, _ = O.ctct_loss_with_logits(logits, ys, lx, ly, "sum", True)
    loss = warp_ctct.ctct_loss_with_logits(x, dev(ys), dev(lx), dev(ly), reduction="sum",
                                           average_frames=True)
    np.testing.assert_allclose(loss.item(), ref_loss, rtol=LOSS_RTOL)
    loss.backward()
    np.testing.assert_allclose(x.grad.cpu().numpy(), ref_grad, atol=GRAD_ATOL, rtol=0)


def test_compact_hand_off_rebuilds_the_dense_gradient():
    """ctct_loss_compact: costs, unit gradients and the gather index; a
    scatter_add of the compact gradient is the dense gradient of the sum."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(51, 3, 19, 6, 23, lx=range(9, 20), ly=range(2, 7))
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    for dtype in (torch.float32, torch.bfloat16):
        x = dev(joint).to(dtype)
        if dtype != torch.float32:
            _, ref_dense, ref_costs = O.ctct_loss(x.double().cpu().numpy(), ys, lx, ly,
                                                  reduction="sum")
        costs, ug, index = warp_ctct.ctct_loss_compact(x, dev(ys), dev(lx), dev(ly))
        assert costs.dtype == ug.dtype == torch.float32 and index.dtype == torch.long
        assert tuple(ug.shape) == (3, 19, 7, 3) and tuple(index.shape) == (3, 7, 3)
        np.testing.assert_allclose(costs.cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
        np.testing.assert_array_equal(index.cpu().numpy(), O.gather_index(ys, 7))
        dense = torch.zeros(3, 19, 7, 23, device="cuda")
        dense.scatter_add_(3, index[:, None].expand_as(ug), ug)
        np.testing.assert_allclose(dense.cpu().numpy(), ref_dense, atol=GRAD_ATOL, rtol=0)


def test_edge_shapes_no_labels_single_frame_and_empty_batch():
    """U = 0 (no labels at all: only the all-blank path), samples without
    labels next to samples with labels, a single frame, and an empty batch."""
    import warp_ctct
    rng = np.random.default_rng(61)
    # no label dimension at all
    joint = np.log(rng.dirichlet(np.ones(6), size=(3, 7, 1))).astype(np.float32)
    ys = np.zeros((3, 0), np.int32)
    lx, ly = np.array([7, 4, 1], np.int32), np.zeros(3, np.int32)
    x = dev(joint).requires_grad_(True)
    c = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="none")
    ref = np.array([-joint[n, :lx[n], 0, 0].sum() for n in range(3)])   # blank on every frame
    np.testing.assert_allclose(c.detach().cpu().numpy(), ref, rtol=LOSS_RTOL)
    c.sum().backward()
    g = x.grad.cpu().numpy()
    for n in range(3):
        np.testing.assert_allclose(g[n, :lx[n], 0, 0], -1.0, atol=GRAD_ATOL)
        assert np.all(g[n, lx[n]:] == 0) and np.all(g[n, :, :, 1:] == 0)
    # samples with zero labels inside a batch that has labels; one frame only
    joint, ys, lx, ly = make_joint_case(62, 4, 9, 3, 8, lx=[9, 5, 1, 3], ly=[3, 0, 1, 0])
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    x = dev(joint).requires_grad_(True)
    c = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="none")
    np.testing.assert_allclose(c.detach().cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
    c.sum().backward()
    np.testing.assert_allclose(x.grad.cpu().numpy(), ref_dense, atol=GRAD_ATOL, rtol=0)
    # empty batch: nothing to launch, empty results, torch's reductions of empty tensors
    e = torch.zeros(0, 5, 3, 4, device="cuda", requires_grad=True)
    ei = torch.zeros(0, 2, dtype=torch.int32, device="cuda")
    el = torch.zeros(0, dtype=torch.int32, device="cuda")
    out = warp_ctct.ctct_loss(e, ei, el, el, reduction="none")
    assert tuple(out.shape) == (0,)
    s = warp_ctct.ctct_loss(e, ei, el, el, reduction="sum")
    assert s.item() == 0.0
    s.backward()
    assert tuple(e.grad.shape) == (0, 5, 3, 4)
    assert torch.isnan(warp_ctct.ctct_loss(e, ei, el, el, reduction="mean"))


@pytest.mark.parametrize("contexts", [512, 1024])
def test_wide_lattices_chains_of_many_wavefronts(contexts):
    """U + 1 = 512 and 1024 contexts: chains of 8 and 16 wavefronts per lattice
    and direction (the reference sets no limit on U: its grid is
    (sT/32, 2U+1, N), csrc/gather.cu:293-297).  One sample fills the lattice,
    the other is short, so most links of its chains hold only padding."""
    import warp_ctct
    U, V = contexts - 1, 6
    T = contexts + 20
    joint, ys, lx, ly = make_joint_case(63, 2, T, U, V, lx=[T, 90], ly=[U, 70], force_repeat=False,
                                        zero_pad=False)
    ys[:] = 1 + np.arange(U) % (V - 1)        # no adjacent repeats: all labels fit
    ys[0, 300] = ys[0, 299]                   # but one, in the fifth wavefront
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    x = dev(joint).requires_grad_(True)
    c = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="none")
    np.testing.assert_allclose(c.detach().cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
    c.sum().backward()
    got = x.grad.cpu().numpy()
    np.testing.assert_allclose(got, ref_dense, atol=GRAD_ATOL, rtol=0)
    assert_support(got, ref_dense, "dense gradient, %d contexts" % contexts)


def test_lost_hand_over_never_yields_a_plausible_number():
    """A workgroup of a chain whose wait for its neighbour's boundary values runs
    out stops and poisons what depends on it.  The wait limit is set to zero from
    the host (the first look decides), so consumers that have caught up with their
    producer give up at once and every kernel still runs to its end: each cost is
    then either NaN or the right number, the gradient of a sample with a NaN cost
    holds NaN, a sample whose lattice fits one wavefront is untouched, and with
    the default limit restored the same call is right again."""
    import warp_ctct
    lib = hip_lib.lib()
    N, T, U, V = 6, 200, 300, 6
    ly = [300, 290, 10, 280, 64, 200]
    joint, ys, lx, ly = make_joint_case(71, N, T, U, V, lx=[200, 190, 60, 200, 150, 180], ly=ly,
                                        force_repeat=False, zero_pad=False)
    ys[:] = 1 + np.arange(U) % (V - 1)
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)

    def run():
        x = dev(joint).requires_grad_(True)
        c = warp_ctct.ctct_loss(x, d_ys, d_lx, d_ly, reduction="none")
        c.sum().backward()
        torch.cuda.synchronize()
        return c.detach().cpu().numpy(), x.grad.cpu().numpy()

    warp_ctct.status(reset=True)
    default = lib.warpctct_lattice_wait_limit(0)
    try:
        assert default > 1000
        costs, grad = run()
    finally:
        assert lib.warpctct_lattice_wait_limit(-1) == 0
    # the status word tells these NaN from NaN that came in with the inputs
    assert warp_ctct.status() == warp_ctct.STATUS_LOST_HAND_OVER
    lost = np.isnan(costs)
    assert lost[[0, 1, 3, 4, 5]].any(), "no consumer ever caught up with its producer"
    assert not lost[2]                                   # 11 contexts: one wavefront, no hand-over
    np.testing.assert_allclose(costs[~lost], ref_costs[~lost], rtol=LOSS_RTOL)
    for n in range(N):
        if lost[n]:
            assert np.isnan(grad[n]).any()
        elif not np.isnan(grad[n]).any():
            # (a finite cost with NaN in the gradient: only the alpha chain lost its input)
            np.testing.assert_allclose(grad[n], ref_dense[n], atol=GRAD_ATOL, rtol=0)
    costs, grad = run()
    assert warp_ctct.status() == 0
    np.testing.assert_allclose(costs, ref_costs, rtol=LOSS_RTOL)
    np.testing.assert_allclose(grad, ref_dense, atol=GRAD_ATOL, rtol=0)


def test_wide_lattice_log_add_joiner_beyond_512_contexts():
    """ctct_simple_loss with 600 contexts: the compact gradients of the joiner
    path are reduced from the unit-gradient tensor instead of inside one
    workgroup per frame block."""
    import warp_ctct
    from ctct_cases import make_simple_case
    N, T, U, V = 2, 640, 599, 9
    f, g, ys, lx, ly = make_simple_case(64, N, T, U, V, lx=[640, 200], ly=[599, 130], normalized=False)
    ys[:] = 1 + np.arange(U) % (V - 1)
    for normalized in (False, True):
        if normalized:
            from ctct_cases import log_softmax
            f, g = log_softmax(f).astype(np.float32), log_softmax(g).astype(np.float32)
        loss, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction="none",
                                                 normalized=normalized, grad_output=np.ones(N))
        tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
        out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction="none",
                                         normalized=normalized)
        np.testing.assert_allclose(out.detach().cpu().numpy(), costs, rtol=LOSS_RTOL)
        out.sum().backward()
        np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL, rtol=1e-5)
        np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)


def test_forward_and_backward_replay_from_a_hip_graph():
    """Nothing in the path synchronises with the host or clears memory with a
    memset, so a training step can be captured once and replayed: every replay
    (with eager work and synchronisations in between, on fresh input values)
    must reproduce the eager result of the same inputs bit for bit."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(71, 6, 33, 9, 40, lx=range(20, 34), ly=range(3, 10))
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    static_in = dev(joint).requires_grad_(True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up outside the capture
        for _ in range(2):
            torch.autograd.grad(warp_ctct.ctct_loss(static_in, d_ys, d_lx, d_ly), static_in)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        static_loss = warp_ctct.ctct_loss(static_in, d_ys, d_lx, d_ly)
        static_grad, = torch.autograd.grad(static_loss, static_in)
    rng = np.random.default_rng(72)
    for replay in range(4):
        fresh = torch.log_softmax(dev(rng.standard_normal(joint.shape).astype(np.float32)), -1)
        with torch.no_grad():
            static_in.copy_(fresh)
        graph.replay()
        torch.cuda.synchronize()
        got_loss, got_grad = static_loss.clone(), static_grad.clone()
        x = fresh.clone().requires_grad_(True)           # eager work between the replays
        loss = warp_ctct.ctct_loss(x, d_ys, d_lx, d_ly)
        grad, = torch.autograd.grad(loss, x)
        torch.cuda.synchronize()
        assert torch.equal(got_loss, loss), "replay %d: loss differs from eager" % replay
        assert torch.equal(got_grad, grad), "replay %d: gradient differs from eager" % replay


def test_more_lattice_chains_than_the_gpu_holds_at_once():
    """1200 lattices of two workgroups per direction: 4800 single-wavefront
    workgroups that wait for one another, more than are resident at a time.
    A consumer is never dispatched before its producer (workgroup index order),
    so every wait ends: no NaN (the mark of a hand-over given up), and costs and
    gradients as the oracle's."""
    import warp_ctct
    N, T, U, V = 1200, 100, 70, 5
    joint, ys, lx, ly = make_joint_case(81, N, T, U, V, lx=range(96, 101), ly=range(64, 71))
    assert ly.min() >= 64 and 2 * N * 2 > 4096
    x = dev(joint).requires_grad_(True)
    out = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="none")
    out.sum().backward()
    got = out.detach().cpu().numpy()
    assert not np.any(np.isnan(got))
    _, ref_grad, costs = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    np.testing.assert_allclose(got, costs, rtol=LOSS_RTOL)
    np.testing.assert_allclose(x.grad.cpu().numpy(), ref_grad, atol=GRAD_ATOL, rtol=0)


@pytest.mark.parametrize("reduction", ["none", "sum", "mean"])
def test_no_frames_at_all(reduction):
    """A batch without a single frame (T = 0): no gather runs, the lattice
    launch still reduces over the batch; a sample without labels costs 0, one
    with labels is infeasible (+inf), as in the oracle."""
    import warp_ctct
    ys = np.array([[1, 2], [3, 4], [2, 2]], dtype=np.int32)
    lx = np.zeros(3, dtype=np.int32)
    for ly in ([0, 0, 0], [0, 1, 0]):
        ly = np.array(ly, dtype=np.int32)
        ref = O.ctct_loss(np.zeros((3, 0, 3, 5)), ys, lx, ly, reduction=reduction)[0]
        x = torch.zeros(3, 0, 3, 5, device="cuda", requires_grad=True)
        loss = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction=reduction)
        np.testing.assert_array_equal(loss.detach().cpu().numpy(), np.asarray(ref, dtype=np.float32))
        if np.all(np.isfinite(ref)):
            grad, = torch.autograd.grad(loss.sum(), x)
            assert grad.shape == x.shape
        logits = torch.zeros(3, 0, 3, 5, device="cuda")
        fused = warp_ctct.ctct_loss_with_logits(logits, dev(ys), dev(lx), dev(ly), reduction=reduction)
        np.testing.assert_array_equal(fused.cpu().numpy(), np.asarray(ref, dtype=np.float32))


def test_kernel_timing_records_stay_out_of_a_graph_capture():
    """The per-kernel timing of the library (warpctct_profile) brackets launches
    with events on their stream; a stream under capture takes none, so a
    capture made while the timing is on is as good as any other and leaves no
    error behind for the next call."""
    import warp_ctct
    lib = hip_lib.lib()
    joint, ys, lx, ly = make_joint_case(73, 3, 21, 6, 17, lx=range(12, 22), ly=range(2, 7))
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    static_in = dev(joint).requires_grad_(True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                       # warm-up outside the capture
        torch.autograd.grad(warp_ctct.ctct_loss(static_in, d_ys, d_lx, d_ly), static_in)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert lib.warpctct_profile(1) == 0
    try:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            static_loss = warp_ctct.ctct_loss(static_in, d_ys, d_lx, d_ly)
            static_grad, = torch.autograd.grad(static_loss, static_in)
        assert lib.warpctct_profile_count() == 0, "launches into the capture were bracketed"
        graph.replay()
        torch.cuda.synchronize()
        x = dev(joint).requires_grad_(True)
        loss = warp_ctct.ctct_loss(x, d_ys, d_lx, d_ly)      # eager: bracketed
        grad, = torch.autograd.grad(loss, x)
        torch.cuda.synchronize()
        assert lib.warpctct_profile_count() > 0
    finally:
        lib.warpctct_profile(0)
    assert torch.equal(static_loss, loss)
    assert torch.equal(static_grad, grad)


def test_operator_surface_on_gathered_units():
    """_C.ctct_loss_fwd keeps the reference's contract: gathered (N,T,U+1,3)
    input, (costs, grads) output, grads zero in padding, costs twice when
    requires_grad is False."""
    from warp_ctct import _C
    joint, ys, lx, ly = make_joint_case(15, 4, 26, 8, 13, lx=range(12, 27), ly=range(3, 9))
    lp3 = O.gather_units(joint, ys).astype(np.float32)
    costs_ref, grads_ref = O.ctct_loss_fwd(lp3, ys, lx, ly)
    costs, grads = _C.ctct_loss_fwd(dev(lp3), dev(ys), dev(lx), dev(ly), True)
    np.testing.assert_allclose(costs.cpu().numpy(), costs_ref, rtol=LOSS_RTOL)
    np.testing.assert_allclose(grads.cpu().numpy(), grads_ref, atol=GRAD_ATOL, rtol=0)
    assert_support(grads.cpu().numpy(), grads_ref, "unit grads")
    c2, same = _C.ctct_loss_fwd(dev(lp3), dev(ys), dev(lx), dev(ly), False)
    assert same.data_ptr() == c2.data_ptr()
    np.testing.assert_array_equal(c2.cpu().numpy(), costs.cpu().numpy())


def test_binding_rejects_bad_tensors():
    from warp_ctct import _C
    joint, ys, lx, ly = make_joint_case(16, 2, 6, 2, 5)
    lp3 = dev(O.gather_units(joint, ys).astype(np.float32))
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    with pytest.raises(RuntimeError):
        _C.ctct_loss_fwd(lp3.double(), d_ys, d_lx, d_ly, True)          # dtype
    with pytest.raises(RuntimeError):
        _C.ctct_loss_fwd(lp3, d_ys.long(), d_lx, d_ly, True)            # label dtype
    with pytest.raises(RuntimeError):
        _C.ctct_loss_fwd(lp3.cpu(), d_ys, d_lx, d_ly, True)             # device
    with pytest.raises(RuntimeError):
        _C.ctct_loss_fwd(lp3.transpose(1, 2), d_ys, d_lx, d_ly, True)   # layout
    with pytest.raises(RuntimeError):
        _C.ctct_loss_fwd(lp3[..., :2].contiguous(), d_ys, d_lx, d_ly, True)   # not gathered
    with pytest.raises(RuntimeError):
        _C.ctct_loss_fwd(lp3, d_ys, d_lx[:1], d_ly, True)               # batch mismatch
    import warp_ctct
    with pytest.raises(AssertionError):
        warp_ctct.ctct_loss(dev(joint), d_ys[:, :1], d_lx, d_ly)
    with pytest.raises(AssertionError):
        warp_ctct.ctct_loss(dev(joint), d_ys, d_lx, d_ly, reduction="avg")


def test_autograd_plumbing_views_non_leaf_and_repeated_backward():
    """The joint as a non-contiguous view and as a non-leaf, backward twice
    over a retained graph, and a loss that is only part of the objective."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(93, 3, 11, 4, 10, lx=[11, 7, 9], ly=[4, 2, 3])
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="none", grad_output=np.ones(3))
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    # stored as (N, U+1, T, V); the loss sees the transposed view
    base = dev(np.ascontiguousarray(joint.transpose(0, 2, 1, 3))).requires_grad_(True)
    view = base.transpose(1, 2)
    assert not view.is_contiguous()
    c = warp_ctct.ctct_loss(view, d_ys, d_lx, d_ly, reduction="none")
    np.testing.assert_allclose(c.detach().cpu().numpy(), ref_costs, rtol=LOSS_RTOL)
    c.sum().backward(retain_graph=True)
    first = base.grad.clone()
    np.testing.assert_allclose(first.transpose(1, 2).cpu().numpy(), ref_dense, atol=GRAD_ATOL, rtol=0)
    base.grad = None
    c.sum().backward()                                  # the saved lattices serve a second backward
    assert torch.equal(base.grad, first)
    # non-leaf input and an objective with another term: d/dx [2 * loss(x) + sum(x)]
    x = dev(joint).requires_grad_(True)
    loss = warp_ctct.ctct_loss(x * 1.0, d_ys, d_lx, d_ly, reduction="sum")
    (2.0 * loss + x.sum()).backward()
    np.testing.assert_allclose(x.grad.cpu().numpy(), 2.0 * ref_dense + 1.0, atol=2 * GRAD_ATOL, rtol=0)
    with torch.no_grad():
        quiet = warp_ctct.ctct_loss(x, d_ys, d_lx, d_ly, reduction="sum")
    assert quiet.grad_fn is None and not quiet.requires_grad
    np.testing.assert_allclose(quiet.item(), ref_costs.sum(), rtol=LOSS_RTOL)


def test_losses_under_autocast_and_with_int64_lengths():
    """The reference computes under autocast(enabled=False) after casting to
    float (warp_ctct/__init__.py:134-136): inside an autocast region the losses
    and their gradients are what they are outside it, for all three entry
    points, and int64 labels / lengths are cast as the reference casts them."""
    import warp_ctct
    from ctct_cases import make_simple_case
    joint, ys, lx, ly = make_joint_case(91, 3, 21, 6, 24, lx=[21, 13, 17], ly=[6, 2, 5])
    f, g, sys_, slx, sly = make_simple_case(92, 3, 19, 5, 40, lx=[19, 12, 15], ly=[5, 3, 4])

    def run(autocast, wide):
        cast = (lambda a: dev(a).long()) if wide else dev
        out = []
        with torch.autocast("cuda", dtype=torch.bfloat16, enabled=autocast):
            x = dev(joint).requires_grad_(True)
            warp_ctct.ctct_loss(x, cast(ys), cast(lx), cast(ly)).backward()
            out.append(x.grad)
            z = dev(joint).requires_grad_(True)
            warp_ctct.ctct_loss_with_logits(z, cast(ys), cast(lx), cast(ly), reduction="sum").backward()
            out.append(z.grad)
            tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
            loss = warp_ctct.ctct_simple_loss(tf, tg, cast(sys_), cast(slx), cast(sly))
            assert loss.dtype == torch.float32
            loss.backward()
            out += [tf.grad, tg.grad]
        return out

    plain = run(False, False)
    for autocast, wide in ((True, False), (False, True), (True, True)):
        for a, b in zip(plain, run(autocast, wide)):
            assert a.dtype == torch.float32 and torch.equal(a, b)


def test_gradient_buffer_cleared_in_the_forward_or_in_the_backward():
    """ctct_loss clears the joint's gradient beside the lattices in the forward
    (warp_ctct.CLEAR_GRADIENT_IN_FORWARD) or, with the switch off, in the
    backward: losses and gradients are the same bit for bit, for float32 and
    bfloat16 joints; without a gradient no buffer is made."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(95, 5, 41, 12, 96, lx=[41, 30, 22, 41, 7], ly=[12, 5, 9, 1, 3])
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="sum", grad_output=np.ones(5))
    assert warp_ctct.CLEAR_GRADIENT_IN_FORWARD
    try:
        for dtype in (torch.float32, torch.bfloat16):
            got = []
            for switch in (True, False):
                warp_ctct.CLEAR_GRADIENT_IN_FORWARD = switch
                x = dev(joint).to(dtype).requires_grad_(True)
                loss = warp_ctct.ctct_loss(x, d_ys, d_lx, d_ly, reduction="sum")
                loss.backward()
                got.append((loss.detach().clone(), x.grad.clone()))
            assert torch.equal(got[0][0], got[1][0]) and torch.equal(got[0][1], got[1][1])
            if dtype == torch.float32:
                np.testing.assert_allclose(got[0][0].item(), ref_costs.sum(), rtol=LOSS_RTOL)
                np.testing.assert_allclose(got[0][1].cpu().numpy(), ref_dense, atol=GRAD_ATOL, rtol=0)
    finally:
        warp_ctct.CLEAR_GRADIENT_IN_FORWARD = True


def test_label_range_check_is_opt_in():
    """Labels outside [0, V) are clamped by the kernels (no fault, a finite loss);
    with warp_ctct.CHECK_LABEL_RANGE the call raises as torch.gather does in the
    reference (warp_ctct/__init__.py:131)."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(77, 2, 9, 4, 7)
    ys[0, 1] = 7                              # == V
    ys[1, 0] = -1
    x, d_ys, d_lx, d_ly = dev(joint), dev(ys), dev(lx), dev(ly)
    warp_ctct.status(reset=True)
    assert torch.isfinite(warp_ctct.ctct_loss(x, d_ys, d_lx, d_ly, reduction="none")).all()
    # without any synchronisation in the loss: the clamped labels are on record
    assert warp_ctct.label_range_violated(reset=False)
    assert warp_ctct.status(reset=True) & warp_ctct.STATUS_LABEL_RANGE
    assert not warp_ctct.label_range_violated()
    for bad, fn in ((7, warp_ctct.ctct_loss), (-1, warp_ctct.ctct_loss_with_logits)):
        one = ys.copy()
        one[0, 1], one[1, 0] = 1, 1
        one[1, 2] = bad
        fn(x, dev(one), d_lx, d_ly)
        assert warp_ctct.label_range_violated(), (bad, fn.__name__)
        assert not warp_ctct.label_range_violated()
    one = ys.copy()
    one[0, 1], one[1, 0] = 7, 1
    warp_ctct.ctct_simple_loss(x[:, :, 0], x[:, 0], dev(one), d_lx, d_ly)
    assert warp_ctct.label_range_violated()
    # labels inside the range, also in the padding of short samples, leave no mark
    one[0, 1] = 6
    for fn in (warp_ctct.ctct_loss, warp_ctct.ctct_loss_with_logits):
        fn(x, dev(one), d_lx, d_ly)
    warp_ctct.ctct_simple_loss(x[:, :, 0], x[:, 0], dev(one), d_lx, d_ly)
    assert warp_ctct.status() == 0
    warp_ctct.CHECK_LABEL_RANGE = True
    try:
        with pytest.raises(IndexError):
            warp_ctct.ctct_loss(x, d_ys, d_lx, d_ly)
        with pytest.raises(IndexError):
            warp_ctct.ctct_loss_with_logits(x, d_ys, d_lx, d_ly)
        with pytest.raises(IndexError):
            warp_ctct.ctct_simple_loss(x[:, :, 0], x[:, 0], d_ys, d_lx, d_ly)
        ys[0, 1], ys[1, 0] = 6, 0
        assert torch.isfinite(warp_ctct.ctct_loss(x, dev(ys), d_lx, d_ly, reduction="none")).all()
    finally:
        warp_ctct.CHECK_LABEL_RANGE = False


def test_nan_input_is_reported_and_acts_as_log_zero():
    """A NaN among the gathered log-probabilities: the unit counts as log 0
    (the lattice's maximum drops NaN operands), so the cost is that of the same
    joint with -inf in its place, and the status word says that it happened."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(78, 2, 9, 4, 7)
    t, u = 3, 2
    col = int(ys[0, u - 1])
    poisoned, masked = joint.copy(), joint.copy()
    poisoned[0, t, u, col] = np.nan
    masked[0, t, u, col] = -np.inf
    warp_ctct.status(reset=True)
    got = warp_ctct.ctct_loss(dev(poisoned), dev(ys), dev(lx), dev(ly), reduction="none")
    ref = warp_ctct.ctct_loss(dev(masked), dev(ys), dev(lx), dev(ly), reduction="none")
    assert warp_ctct.status(reset=False) & warp_ctct.STATUS_NAN_INPUT
    assert warp_ctct.status() & warp_ctct.STATUS_NAN_INPUT and warp_ctct.status() == 0
    np.testing.assert_array_equal(got.cpu().numpy(), ref.cpu().numpy())
    _, _, want = O.ctct_loss(masked, ys, lx, ly, reduction="none")
    np.testing.assert_allclose(got.cpu().numpy(), want, rtol=LOSS_RTOL)
    # a NaN outside the gathered columns is never read
    poisoned = joint.copy()
    free = [v for v in range(1, 7) if v not in (int(ys[0, u - 1]), int(ys[0, u]))][0]
    poisoned[0, t, u, free] = np.nan
    warp_ctct.ctct_loss(dev(poisoned), dev(ys), dev(lx), dev(ly))
    assert warp_ctct.status() == 0


def test_infeasible_sample_has_infinite_cost():
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(17, 2, 6, 3, 5, force_repeat=False)
    ys[0] = [2, 2, 2]
    lx = np.array([4, 6], dtype=np.int32)          # sample 0 needs 5 frames
    ly = np.array([3, 3], dtype=np.int32)
    c = warp_ctct.ctct_loss(dev(joint), dev(ys), dev(lx), dev(ly), reduction="none").cpu().numpy()
    _, _, ref = O.ctct_loss(joint, ys, lx, ly, reduction="none")
    assert np.isposinf(c[0]) and np.isposinf(ref[0])
    np.testing.assert_allclose(c[1], ref[1], rtol=LOSS_RTOL)
    # Its gradient is NaN, as the reference's (csrc/gather.cu:339-340: the
    # exponent holds -inf - (-inf) once the log-likelihood is -inf): at every
    # gathered column of the cells that complete alignments could pass through,
    # and nowhere else; the feasible sample beside it is not touched by that.
    x = dev(joint).requires_grad_(True)
    warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="sum").backward()
    got = x.grad.cpu().numpy()
    _, ref_dense, _ = O.ctct_loss(joint, ys, lx, ly, reduction="sum")
    np.testing.assert_allclose(got[1], ref_dense[1], atol=GRAD_ATOL, rtol=0)
    expect_nan = np.zeros(got[0].shape, dtype=bool)
    Tn, Un = int(lx[0]), int(ly[0])
    for t in range(Tn):
        for u in range(Un + 1):
            if t < u or Tn - t < Un - u:          # outside the band: exactly zero
                continue
            expect_nan[t, u, 0] = True
            if u >= 1:
                expect_nan[t, u, ys[0, u - 1]] = True
            if u < Un:
                expect_nan[t, u, ys[0, u]] = True
    assert expect_nan.any()
    assert np.all(np.isnan(got[0][expect_nan])), "infeasible sample: gradient must be NaN"
    assert np.all(got[0][~expect_nan] == 0)
    assert np.all(np.isnan(ref_dense[0][expect_nan]))      # the float64 oracle agrees


def test_committed_brute_force_vectors():
    """The HIP path against tests/golden/brute_force_cases.npz: lattices whose
    log-likelihood and dense gradient come from enumerating every alignment
    (no lattice recursion involved), including no labels at all, a single
    frame, and lx = ly."""
    import os
    import warp_ctct
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden",
                             "brute_force_cases.npz"))
    x = dev(z["joint"]).requires_grad_(True)
    c = warp_ctct.ctct_loss(x, dev(z["ys"]), dev(z["lx"]), dev(z["ly"]), reduction="none")
    np.testing.assert_allclose(c.detach().cpu().numpy(), -z["loglik"], rtol=LOSS_RTOL)
    c.sum().backward()
    got = x.grad.cpu().numpy()
    np.testing.assert_allclose(got, z["dense_grad"], atol=GRAD_ATOL, rtol=0)
    assert_support(got, z["dense_grad"], "dense gradient")
    # the same through the logits entry: log_softmax of log-probabilities is the identity
    # up to rounding, its backward subtracts softmax * sum(G) = exp(joint) * (-1 per frame)
    x2 = dev(z["joint"]).requires_grad_(True)
    c2 = warp_ctct.ctct_loss_with_logits(x2, dev(z["ys"]), dev(z["lx"]), dev(z["ly"]), reduction="none")
    np.testing.assert_allclose(c2.detach().cpu().numpy(), -z["loglik"], rtol=1e-4)


def test_minus_infinity_entries_on_the_paths():
    """Log-probabilities of -inf (masked tokens) at cells that alignments would
    use: those alignments drop out, the rest is scored as usual; the gradient at
    a -inf entry is 0, never NaN."""
    import warp_ctct
    joint, ys, lx, ly = make_joint_case(91, 4, 22, 6, 12, lx=range(14, 23), ly=range(3, 7), zero_pad=False)
    rng = np.random.default_rng(92)
    N, T, U1, V = joint.shape
    for n in range(N):
        for t in range(T):
            for u in range(U1):
                r = rng.random()
                if r < 0.10:
                    joint[n, t, u, 0] = -np.inf                       # blank masked
                elif r < 0.20 and u < ly[n]:
                    joint[n, t, u, ys[n, u]] = -np.inf                # next label masked
                elif r < 0.25 and u >= 1:
                    joint[n, t, u, ys[n, u - 1]] = -np.inf            # label repeat masked
    joint[3, :, :, 0] = -np.inf                                       # sample 3: no blank anywhere
    _, ref_dense, ref_costs = O.ctct_loss(joint, ys, lx, ly, reduction="none", grad_output=np.ones(N))
    x = dev(joint).requires_grad_(True)
    c = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="none")
    got = c.detach().cpu().numpy()
    fin = np.isfinite(ref_costs)
    assert fin.sum() >= 2, "the case should leave feasible samples"
    assert np.array_equal(np.isposinf(got), np.isposinf(ref_costs))
    np.testing.assert_allclose(got[fin], ref_costs[fin], rtol=LOSS_RTOL)
    c[torch.as_tensor(fin).cuda()].sum().backward()
    g = x.grad.cpu().numpy()
    assert np.all(np.isfinite(g[fin]))
    np.testing.assert_allclose(g[fin], ref_dense[fin], atol=GRAD_ATOL, rtol=0)
    assert np.all(g[fin][np.isneginf(joint[fin])] == 0)


FULL_SIZE = [
    # name, N, T, U, V, lx range, ly range, sigma
    ("typical_asr_batch", 32, 250, 60, 1024, (150, 250), (30, 60), 1.0),
    ("large_vocab_long_lattice", 8, 500, 120, 4096, (400, 500), (80, 120), 2.0),
]


@pytest.mark.parametrize("cfg", FULL_SIZE, ids=[c[0] for c in FULL_SIZE])
def test_full_size(cfg):
    """Full-size batches of the benchmark configurations: costs and unit
    gradients against the C oracle in float64; the 2 GB / 7.9 GB dense gradient
    is checked on the GPU through size-independent properties (support,
    per-frame mass -1, gathered values)."""
    import warp_ctct
    name, N, T, U, V, lx_rng, ly_rng, sigma = cfg
    g = torch.Generator(device="cuda").manual_seed(1234)
    logits = torch.randn(N, T, U + 1, V, device="cuda", generator=g).mul_(sigma)
    joint = logits.log_softmax(-1)
    del logits
    rng = np.random.default_rng(1234)
    lx = rng.integers(lx_rng[0], lx_rng[1] + 1, N).astype(np.int32)
    ly = rng.integers(ly_rng[0], ly_rng[1] + 1, N).astype(np.int32)
    lx[3], ly[5] = lx_rng[1], ly_rng[1]
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    ys[:, 7] = ys[:, 6]
    d_ys, d_lx, d_ly = dev(ys), dev(lx), dev(ly)
    t_idx = torch.arange(T, device="cuda")[None, :, None, None]
    u_idx = torch.arange(U + 1, device="cuda")[None, None, :, None]
    pad = (t_idx >= d_lx[:, None, None, None]) | (u_idx > d_ly[:, None, None, None])
    joint.masked_fill_(pad, 0.0)
    joint.requires_grad_(True)
    w = torch.tensor(rng.standard_normal(N), dtype=torch.float32, device="cuda")
    costs = warp_ctct.ctct_loss(joint, d_ys, d_lx, d_ly, reduction="none")
    (costs * w).sum().backward()
    dense = joint.grad
    # reference from the gathered units (exactly what the reference's gather yields)
    index = torch.zeros(N, U + 1, 3, dtype=torch.long, device="cuda")
    index[:, 1:, 1] = d_ys
    index[:, :U, 2] = d_ys
    index = index[:, None].expand(-1, T, -1, -1)
    lp3 = joint.detach().gather(-1, index).cpu().numpy()
    costs_ref, ug_ref = C.ctct_loss_fwd(lp3, ys, lx, ly, dtype=np.float64)
    np.testing.assert_allclose(costs.detach().cpu().numpy(), costs_ref, rtol=LOSS_RTOL)
    ug_ref_w = ug_ref * w.cpu().numpy().astype(np.float64)[:, None, None, None]
    # values on the gathered columns (context 7 has coincident columns k=1,k=2)
    got = dense.gather(-1, index).cpu().numpy().astype(np.float64)
    exp = ug_ref_w.copy()
    assert (ys[:, 6] == ys[:, 7]).all()
    for n in range(N):
        for u in range(1, U):
            if ys[n, u - 1] == ys[n, u]:
                both = ug_ref_w[n, :, u, 1] + ug_ref_w[n, :, u, 2]
                exp[n, :, u, 1] = both
                exp[n, :, u, 2] = both
    exp[:, :, 0, 1] = exp[:, :, 0, 0]          # u=0,k=1 and u=U,k=2 gather column 0
    exp[:, :, U, 2] = exp[:, :, U, 0]
    scale = max(1.0, float(w.abs().max()))
    np.testing.assert_allclose(got, exp, atol=GRAD_ATOL * scale, rtol=0)
    # support: every non-zero sits on a gathered column
    mask = torch.zeros_like(dense, dtype=torch.bool)
    mask.scatter_(-1, index, True)
    assert int((dense != 0).sum()) == int(((dense != 0) & mask).sum())
    assert int((dense[pad.expand_as(dense)] != 0).sum()) == 0
    # per-frame mass: sum over (u, v) = -w[n] for t < lx[n], 0 beyond
    mass = dense.sum((2, 3), dtype=torch.float64).cpu().numpy()
    wn = w.cpu().numpy().astype(np.float64)
    for n in range(N):
        np.testing.assert_allclose(mass[n, :lx[n]], -wn[n], rtol=1e-4, atol=1e-5)
        assert np.all(mass[n, lx[n]:] == 0)


@pytest.mark.parametrize("dtype,logits", [(torch.float16, True), (torch.bfloat16, False)],
                         ids=["float16_logits", "bfloat16_joint"])
def test_full_size_typical_batch_in_half_precision(dtype, logits):
    """The typical batch (N=32, T<=250, U<=60, V=1024) with 2-byte elements,
    through the fused logits entry and through the joint, against the float64
    oracle on the rounded inputs: loss within 1e-5 relative, every gradient
    entry within 1e-4 of the sample weight (1/N) plus one unit in the last
    place of the type."""
    import warp_ctct
    N, T, U, V = 32, 250, 60, 1024
    rng = np.random.default_rng(5)
    lx = rng.integers(150, T + 1, N).astype(np.int32)
    ly = rng.integers(30, U + 1, N).astype(np.int32)
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    gen = torch.Generator(device="cuda").manual_seed(5)
    x = torch.randn(N, T, U + 1, V, device="cuda", generator=gen) * 2
    if not logits:
        x = x.log_softmax(-1)
    x = x.to(dtype).requires_grad_(True)
    fn = warp_ctct.ctct_loss_with_logits if logits else warp_ctct.ctct_loss
    loss = fn(x, dev(ys), dev(lx), dev(ly), reduction="mean")
    loss.backward()
    rounded = x.detach().double().cpu().numpy()
    if logits:
        ref_loss, ref_grad, _ = O.ctct_loss_with_logits(rounded, ys, lx, ly, "mean", False)
    else:
        ref_loss, ref_grad, _ = O.ctct_loss(rounded, ys, lx, ly, reduction="mean")
    del rounded
    np.testing.assert_allclose(loss.item(), ref_loss, rtol=LOSS_RTOL)
    got = x.grad.double().cpu().numpy()
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    assert np.all(np.abs(got - ref_grad) <= GRAD_ATOL / N + ulp * np.abs(ref_grad))
    assert np.all(got[ref_grad == 0] == 0)


@pytest.mark.parametrize("shape", [(800, 96, 40), (300, 96, 100)], ids=["lone_wavefronts", "chains_of_two"])
def test_many_lattices_at_once_repeat_bit_for_bit(shape):
    """1600 or 1200 wavefronts of sweeps in one launch, several per SIMD, in both
    launches that sweep (with the clear of the gradient riding along, and
    without): the rows of the lattices are stored 16 bytes per lane, and a store
    like that whose data registers the next instruction overwrites came out
    wrong now and then on a full chip.  Two calls must agree bit for bit, and with
    the oracle on a few samples."""
    import warp_ctct
    (N, T, U), V = shape, 4
    rng = np.random.default_rng(3)
    lx = rng.integers(T - 30, T + 1, size=N)
    ly = rng.integers(U // 2, U + 1, size=N)
    joint, ys, lx, ly = make_joint_case(31, N, T, U, V, lx=lx, ly=ly)
    w = rng.standard_normal(N)
    some = [0, 1, N // 2, N - 1]
    _, ref_dense, ref_costs = O.ctct_loss(joint[some], ys[some], lx[some], ly[some], reduction="none",
                                          grad_output=w[some])
    before = warp_ctct.CLEAR_GRADIENT_IN_FORWARD
    try:
        for clear_in_forward in (True, False):
            warp_ctct.CLEAR_GRADIENT_IN_FORWARD = clear_in_forward
            runs = []
            for _ in range(2):
                x = dev(joint).requires_grad_(True)
                costs = warp_ctct.ctct_loss(x, dev(ys), dev(lx), dev(ly), reduction="none")
                (costs * dev(w, torch.float32)).sum().backward()
                runs.append((costs.detach().cpu().numpy(), x.grad.cpu().numpy()))
            assert np.array_equal(runs[0][0], runs[1][0])
            assert np.array_equal(runs[0][1], runs[1][1])
            np.testing.assert_allclose(runs[0][0][some], ref_costs, rtol=LOSS_RTOL)
            np.testing.assert_allclose(runs[0][1][some], ref_dense, atol=GRAD_ATOL * np.abs(w).max(), rtol=0)
    finally:
        warp_ctct.CLEAR_GRADIENT_IN_FORWARD = before
