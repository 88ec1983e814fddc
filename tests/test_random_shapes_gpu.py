"""Seeded random cases around the sizes at which the library changes kernels
(chains of workgroups per lattice, hand-over chunks, 16-byte vector rows, the
shapes of the log-matmul kernels), against the float64 oracle through the
public API.  Every case prints its parameters before it runs, so a failure or
a fault names its case.

WARPCTCT_RANDOM_CASES_SCALE=k in the environment runs k times as many cases per
test (the same seeds, longer streams) for an occasional long run;
WARPCTCT_RANDOM_SEED_OFFSET=m adds m to every seed, for other cases than the
committed ones."""
import os

import numpy as np
import pytest
import torch

import hip_lib
from ctct_cases import make_joint_case, make_simple_case
from oracle import c_oracle as C
from oracle import ctct_oracle as O

pytestmark = pytest.mark.gpu

SCALE = max(1, int(os.environ.get("WARPCTCT_RANDOM_CASES_SCALE", "1")))
SEED_OFFSET = int(os.environ.get("WARPCTCT_RANDOM_SEED_OFFSET", "0"))
LOSS_RTOL = 1e-5     # loss: relative
GRAD_ATOL = 1e-4     # gradients: absolute


def dev(a, dtype=None):
    return torch.as_tensor(np.ascontiguousarray(a), device="cuda", dtype=dtype)


def same_costs(got, ref, atol=1e-5):
    got, ref = np.asarray(got, dtype=np.float64), np.asarray(ref, dtype=np.float64)
    fin = np.isfinite(ref)
    assert np.array_equal(np.isfinite(got), fin)
    np.testing.assert_allclose(got[fin], ref[fin], rtol=LOSS_RTOL, atol=atol)
    return bool(np.all(fin))


@pytest.mark.parametrize("seed", [11, 12])
def test_random_joint_and_logits_cases(seed):
    """ctct_loss and ctct_loss_with_logits: all three element types, views,
    reductions, average_frames, weights per sample."""
    import warp_ctct
    rng = np.random.default_rng(seed + SEED_OFFSET)
    Ts = [1, 2, 7, 8, 9, 11, 12, 13, 23, 24, 25, 36, 37, 70, 140]
    Us = [0, 1, 2, 5, 62, 63, 64, 65, 127, 128, 129, 200]
    Vs = [2, 3, 4, 5, 8, 31, 32, 33, 64, 100]
    dts = [torch.float32, torch.float32, torch.bfloat16, torch.float16]
    done = 0
    while done < 600 * SCALE:
        N, T = int(rng.integers(1, 5)), int(rng.choice(Ts))
        U, V = int(rng.choice(Us)), int(rng.choice(Vs))
        if N * T * (U + 1) * V > 3e6:
            continue
        dt = dts[int(rng.integers(0, 4))]
        reduction = ["none", "mean", "sum"][int(rng.integers(0, 3))]
        avg, logits = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        view = int(rng.integers(0, 3)) == 0 and not logits
        case_seed = int(rng.integers(0, 1 << 30))
        print("case N=%d T=%d U=%d V=%d %s %s avg=%s logits=%s view=%s seed=%d"
              % (N, T, U, V, dt, reduction, avg, logits, view, case_seed), flush=True)
        joint, ys, lx, ly = make_joint_case(case_seed, N, T, U, V)
        if logits:
            joint = (np.random.default_rng(case_seed).standard_normal(joint.shape) * 2).astype(np.float32)
        if view:
            wide = torch.zeros(N, T, U + 1, V + 3, device="cuda", dtype=dt)
            wide[..., 1:V + 1] = dev(joint).to(dt)
            x = wide[..., 1:V + 1].detach().requires_grad_(True)
        else:
            x = dev(joint).to(dt).requires_grad_(True)
        rounded = x.detach().double().cpu().numpy()
        w = rng.standard_normal(N) if reduction == "none" else None
        w_costs = None if w is None else (w / lx if avg else w)     # d(loss)/d(costs)
        with np.errstate(all="ignore"):
            if logits:
                ref_loss, ref_grad, _ = O.ctct_loss_with_logits(rounded, ys, lx, ly, reduction, avg,
                                                                grad_output=w_costs)
            else:
                ref_loss, ref_grad, _ = O.ctct_loss(rounded, ys, lx, ly, reduction=reduction,
                                                    average_frames=avg, grad_output=w_costs)
        fn = warp_ctct.ctct_loss_with_logits if logits else warp_ctct.ctct_loss
        loss = fn(x, dev(ys), dev(lx), dev(ly), reduction=reduction, average_frames=avg)
        if reduction == "none":
            loss.backward(dev(w, torch.float32))
        else:
            loss.backward()
        if same_costs(loss.detach().cpu().numpy(), ref_loss):
            got = x.grad.double().cpu().numpy()
            ulp = {torch.float32: 0.0, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dt]
            scale = max(1.0, float(np.abs(w).max())) if w is not None else 1.0
            assert np.all(np.abs(got - ref_grad) <= GRAD_ATOL * scale + ulp * np.abs(ref_grad))
        done += 1


@pytest.mark.parametrize("seed", [21, 22])
def test_random_joiner_cases(seed):
    """ctct_simple_loss, normalized and not: sizes around 128 frames, 16..96
    contexts and vocabularies of 512..2048 in chunks of 32, where the
    log-matmul kernels change, and some long inputs with up to 261 contexts;
    -inf vocabulary entries and a frame far below the others in a quarter of
    the cases; the lattices swept in the linear domain in half of them."""
    import warp_ctct
    rng = np.random.default_rng(seed + SEED_OFFSET)
    # (the long ones for the sweeps in the linear domain: whole turns of their
    # chunks, and chains of up to five workgroups that run into one another)
    Ts = [1, 17, 96, 127, 128, 129, 143, 144, 160, 333, 700]
    Us = [0, 1, 15, 16, 31, 32, 47, 48, 61, 62, 63, 64, 79, 80, 95, 96, 97, 123, 124, 130, 260]
    Vs = [3, 33, 256, 480, 511, 512, 544, 800, 1000, 1024, 1056, 2016, 2047, 2048, 2049, 2080, 2304]
    done = 0
    while done < 150 * SCALE:
        N, T = int(rng.integers(1, 4)), int(rng.choice(Ts))
        U, V = int(rng.choice(Us)), int(rng.choice(Vs))
        if T * (U + 1) * V * N > 40e6:
            continue
        normalized, mask = bool(rng.integers(0, 2)), int(rng.integers(0, 4)) == 0
        # the lattices swept in the linear domain (with their check and the log
        # domain as fall-back) in half of the cases, whatever the number of frames
        linear = int(rng.integers(0, 2))
        case_seed = int(rng.integers(0, 1 << 30))
        print("case N=%d T=%d U=%d V=%d normalized=%s mask=%s linear=%d seed=%d"
              % (N, T, U, V, normalized, mask, linear, case_seed), flush=True)
        hip_lib.lib().warpctct_joiner_linear_lattice(linear)
        warp_ctct.status(reset=True)
        f, g, ys, lx, ly = make_simple_case(case_seed, N, T, U, V, normalized=normalized)
        if mask:
            cols = rng.integers(1, V, size=max(2, V // 7))
            f[:, :, cols[: len(cols) // 2]] = -np.inf
            g[:, :, cols[len(cols) // 2:]] = -np.inf
            f[0, T // 2] -= 300.0
        # the reduction over the batch and the division by the frame counts are
        # part of the kernels: drawn at random too, with an upstream gradient
        # per sample (no reduction) or one for the reduced scalar
        reduction = ["none", "sum", "mean"][int(rng.integers(0, 3))]
        average_frames = bool(rng.integers(0, 2))
        w = rng.standard_normal(N) if reduction == "none" else rng.standard_normal(1)
        per_sample = np.broadcast_to(w, (N,)).astype(np.float64)
        if average_frames:
            per_sample = per_sample / lx
        if reduction == "mean":
            per_sample = per_sample / N
        with np.errstate(all="ignore"):
            loss, gf, gg, costs = O.ctct_simple_loss(f, g, ys, lx, ly, reduction=reduction,
                                                     average_frames=average_frames,
                                                     normalized=normalized, grad_output=per_sample)
        tf, tg = dev(f).requires_grad_(True), dev(g).requires_grad_(True)
        out = warp_ctct.ctct_simple_loss(tf, tg, dev(ys), dev(lx), dev(ly), reduction=reduction,
                                         average_frames=average_frames, normalized=normalized)
        (out * dev(w, torch.float32)).sum().backward()
        # (a frame 300 below the others cancels against its own normaliser: a cost
        # near 0 then carries the rounding of float32 numbers of size 300, 3e-5 each)
        if same_costs(np.atleast_1d(out.detach().cpu().numpy()), np.atleast_1d(loss),
                      atol=1e-4 if (mask and normalized) else 1e-5):
            scale = max(1.0, float(np.abs(w).max()))
            # dense gradients sum up to T (resp. U+1) unit gradients per entry.  With the
            # normalisation, the denominators are float32 here as in the reference (the
            # oracle's are float64): their rounding, ~5e-7 per frame, moves the weight of
            # an alignment against one that dwells elsewhere by ~1e-5 over some hundred
            # frames (333 frames in 17 contexts: 7-13e-6 on the entries that sum a
            # context's ~100 posteriors, in either domain of the sweeps)
            rtol = 2e-5 if normalized else 1e-5
            np.testing.assert_allclose(tf.grad.cpu().numpy(), gf, atol=GRAD_ATOL * scale, rtol=rtol)
            # (with masked columns a row may be left with one admissible entry, whose
            # probability is 1: its gradient wrt g is the sum over the frames of
            # posterior - probability = 1 - 1, formed in float32 from factors that
            # are each good to ~4e-6, and 700 such frames leave 3e-3 (allowed: 1e-5 per frame) where the oracle
            # has 1e-12)
            atol_g = GRAD_ATOL * scale * (max(1.0, T / 10.0) if (mask and normalized) else 1.0)
            np.testing.assert_allclose(tg.grad.cpu().numpy(), gg, atol=atol_g, rtol=rtol)
        # (ordinary input: the linear sweeps hold on their own; a sample that has no
        # alignment at all -- too few frames for its labels and their repeats, or,
        # with masked columns, a label without any mass -- sends them back to the
        # log domain, and so does the frame that the mask pushes down by 300)
        fell_back = warp_ctct.status(reset=True) & warp_ctct.STATUS_LINEAR_FELL_BACK
        assert mask or not fell_back or not np.all(np.isfinite(costs))
        done += 1
    hip_lib.lib().warpctct_joiner_linear_lattice(-1)


@pytest.mark.parametrize("seed", [31, 32])
def test_random_log_matmul_cases(seed):
    """_C.log_matmul and log_matmul_backward: either operand the long one, the
    right operand contiguous, a transposed view, or shared by the batch, or both
    operands views into wider tensors; rows
    and columns of -inf and maxima 300 apart in a quarter of the cases."""
    from warp_ctct import _C
    rng = np.random.default_rng(seed + SEED_OFFSET)
    Ms = [1, 3, 15, 16, 17, 31, 33, 64, 95, 96, 97, 127, 128, 129, 144, 200, 260]
    Ks = [1, 2, 31, 32, 33, 64, 255, 256, 257, 300, 511, 512, 544, 800, 1024, 2047, 2048, 2049, 2304]
    Ns = [1, 2, 15, 16, 17, 32, 33, 48, 64, 80, 96, 97, 130, 200]
    done = 0
    while done < 400 * SCALE:
        B, M = int(rng.integers(1, 4)), int(rng.choice(Ms))
        K, Nn = int(rng.choice(Ks)), int(rng.choice(Ns))
        if rng.integers(0, 2):
            M, Nn = Nn, M
        if B * M * K * Nn > 20e6:
            continue
        layout = ["contiguous", "transposed", "shared", "offset"][int(rng.integers(0, 4))]
        special = int(rng.integers(0, 4)) == 0
        case_seed = int(rng.integers(0, 1 << 30))
        print("case B=%d M=%d K=%d Nn=%d %s special=%s seed=%d"
              % (B, M, K, Nn, layout, special, case_seed), flush=True)
        r = np.random.default_rng(case_seed)
        lhs = (r.standard_normal((B, M, K)) * 3).astype(np.float32)
        Br = 1 if layout == "shared" else B
        rhs = (r.standard_normal((Br, K, Nn)) * 3).astype(np.float32)
        if special:
            lhs[0, r.integers(0, M), :] = -np.inf
            rhs[0, :, r.integers(0, Nn)] = -np.inf
            lhs[B - 1, r.integers(0, M), r.integers(0, K)] = 300.0
            rhs[Br - 1, r.integers(0, K), r.integers(0, Nn)] = 300.0
            lhs[0, :, r.integers(0, K)] = -np.inf
        rhs_full = np.ascontiguousarray(np.broadcast_to(rhs, (B, K, Nn)))
        with np.errstate(all="ignore"):
            ref = C.log_matmul(lhs, rhs_full)
        d_lhs = dev(lhs)
        if layout == "transposed":
            d_rhs = dev(np.ascontiguousarray(rhs.transpose(0, 2, 1))).transpose(1, 2)
        elif layout == "offset":    # both operands inside wider tensors, rows not on 16-byte boundaries
            wide_l = torch.zeros(B, M, K + 3, device="cuda")
            wide_l[..., 1:K + 1] = d_lhs
            d_lhs = wide_l[..., 1:K + 1]
            wide_r = torch.zeros(B, K, Nn + 2, device="cuda")
            wide_r[..., 1:Nn + 1] = dev(rhs)
            d_rhs = wide_r[..., 1:Nn + 1]
        else:
            d_rhs = dev(rhs)
        out = _C.log_matmul(d_lhs, d_rhs)
        got = out.cpu().numpy()
        fin = np.isfinite(ref)
        assert np.array_equal(np.isneginf(got), np.isneginf(ref))
        np.testing.assert_allclose(got[fin], ref[fin], rtol=1e-5, atol=1e-4)
        # the gradient from the float32 result the operator is given, as the
        # reference computes it
        go = r.standard_normal((B, M, Nn)).astype(np.float32)
        with np.errstate(all="ignore"):
            gl, gr = O.log_matmul_backward(go, lhs, rhs_full, got.astype(np.float64))
        if layout == "shared":
            gr = gr.sum(0, keepdims=True)
        out_l, out_r = _C.log_matmul_backward(dev(go), d_lhs, d_rhs, out, [True, True])
        assert out_l.shape == d_lhs.shape and tuple(out_r.shape) == tuple(d_rhs.shape)
        # entries of 300 leave float32 sums with an absolute error of their own size's rounding
        # (one ulp of 300 is 3e-5, and a term of the gradient is e^(lhs + rhs - out): runs over
        # other seeds have shown up to 4.1e-4)
        atol = 6e-4 if special else 3e-5
        np.testing.assert_allclose(out_l.cpu().numpy(), gl, atol=atol, rtol=1e-4)
        np.testing.assert_allclose(out_r.cpu().numpy(), gr, atol=atol * Br if layout != "shared" else atol * B,
                                   rtol=1e-4)
        done += 1


@pytest.mark.parametrize("seed", [41, 42])
def test_random_cases_of_the_operators_on_gathered_inputs(seed):
    """_C.ctct_loss_fwd and _C.ctct_loss_simple_fwd (the reference's own operator
    surface): up to 601 contexts (chains of ten workgroups; beyond 512 the
    joiner's reductions take their own kernels), with and without gradients."""
    from warp_ctct import _C
    rng = np.random.default_rng(seed + SEED_OFFSET)
    Ts = [1, 2, 7, 8, 9, 12, 13, 24, 25, 37, 70, 140, 300]
    Us = [0, 1, 2, 5, 62, 63, 64, 65, 127, 128, 129, 200, 511, 512, 513, 600]
    done = 0
    while done < 300 * SCALE:
        N, T = int(rng.integers(1, 5)), int(rng.choice(Ts))
        U, V = int(rng.choice(Us)), int(rng.choice([3, 5, 9, 33]))
        if N * T * (U + 1) > 1.0e6:
            continue
        case_seed, want = int(rng.integers(0, 1 << 30)), bool(rng.integers(0, 4) > 0)
        which = int(rng.integers(0, 3))
        print("case op=%d N=%d T=%d U=%d V=%d requires_grad=%s seed=%d"
              % (which, N, T, U, V, want, case_seed), flush=True)
        if which == 0:
            joint, ys, lx, ly = make_joint_case(case_seed, N, T, U, V)
            lp3 = O.gather_units(joint, ys).astype(np.float32)
            with np.errstate(all="ignore"):
                costs_ref, grads_ref = O.ctct_loss_fwd(lp3, ys, lx, ly)
            costs, grads = _C.ctct_loss_fwd(dev(lp3), dev(ys), dev(lx), dev(ly), want)
            finite = same_costs(costs.cpu().numpy(), costs_ref)
            if want and finite:
                np.testing.assert_allclose(grads.cpu().numpy(), grads_ref, atol=GRAD_ATOL, rtol=0)
            if not want:       # the reference returns the costs twice
                np.testing.assert_array_equal(grads.cpu().numpy(), costs.cpu().numpy())
        else:
            normalized = which == 1
            f, g, ys, lx, ly = make_simple_case(case_seed, N, T, U, V, normalized=normalized)
            f_g, g_g = O.gather_separate(f, g, ys)
            den = O.log_matmul(f, np.swapaxes(g, 1, 2)).astype(np.float32) if normalized else None
            with np.errstate(all="ignore"):
                costs_ref, gf, gg, gd = O.ctct_loss_simple_fwd(f_g, g_g, ys, den, lx, ly)
            d_den = dev(den) if normalized else torch.empty(1)
            out = _C.ctct_loss_simple_fwd(dev(f_g), dev(g_g), dev(ys), d_den, dev(lx), dev(ly), want)
            finite = same_costs(out[0].cpu().numpy(), costs_ref)
            if want and finite:
                np.testing.assert_allclose(out[1].cpu().numpy(), gf, atol=GRAD_ATOL, rtol=0)
                np.testing.assert_allclose(out[2].cpu().numpy(), gg, atol=GRAD_ATOL, rtol=1e-5)
                if normalized:
                    np.testing.assert_allclose(out[3].cpu().numpy(), gd, atol=GRAD_ATOL, rtol=0)
            if not want:
                assert out[1] is None and out[2] is None and out[3] is None
        done += 1
