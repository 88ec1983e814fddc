"""warpctct_loss_forward_static: the forward without a workspace argument,
whose work buffers live in a device array of the library (for callers that
cannot allocate).  Called through the C ABI and compared with
warpctct_loss_forward on the same inputs: same kernels on the same values, so
costs and unit gradients must agree bit for bit, and both must meet the
oracle (loss rel-err <= 1e-5, gradient abs-err <= 1e-4).  Two calls in a row,
the second on a smaller problem, share the array: the second must not see what
the first left behind."""
import ctypes

import numpy as np
import pytest
import torch

import hip_lib
from ctct_cases import make_joint_case
from oracle import ctct_oracle as O

pytestmark = pytest.mark.gpu

STATIC_BYTES = 32 << 20
ETOOLARGE = 5


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a)).cuda()


def forward_both(joint, ys, lx, ly):
    lib = hip_lib.lib()
    N, T, U1, V = joint.shape
    U = U1 - 1
    p, s = hip_lib.ptr, hip_lib.stream_ptr()
    d_joint, d_ys, d_lx, d_ly = dev(joint), dev(ys), dev(lx), dev(ly)
    need = lib.warpctct_workspace_bytes(N, T, U)
    assert need <= STATIC_BYTES
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    out = []
    for static in (False, True):
        costs = torch.full((N,), float("nan"), device="cuda")
        ug = torch.full((N, T, U1, 3), float("nan"), device="cuda")
        if static:
            rc = lib.warpctct_loss_forward_static(p(d_joint), 0, p(d_ys), p(d_lx), p(d_ly), N, T, U,
                                                  V, p(costs), p(ug), s)
        else:
            rc = lib.warpctct_loss_forward(p(d_joint), 0, p(d_ys), p(d_lx), p(d_ly), N, T, U, V,
                                           p(ws), ctypes.c_size_t(need), p(costs), p(ug), s)
        hip_lib.check(rc)
        torch.cuda.synchronize()
        out.append((costs.cpu().numpy(), ug.cpu().numpy()))
    return out


def test_static_scratch_forward_matches_the_workspace_forward():
    lib = hip_lib.lib()
    big = make_joint_case(101, 6, 120, 40, 50, lx=range(70, 121), ly=range(15, 41))
    # lattices of two and three workgroups each: their hand-over slots lie in the array too
    chains = make_joint_case(103, 3, 150, 140, 7, lx=range(145, 151), ly=range(70, 141))
    small = make_joint_case(102, 3, 31, 9, 17, lx=range(12, 32), ly=range(2, 10))
    for joint, ys, lx, ly in (big, chains, small):        # the last call is the smallest problem
        (c_ws, g_ws), (c_st, g_st) = forward_both(joint, ys, lx, ly)
        np.testing.assert_array_equal(c_st, c_ws)
        np.testing.assert_array_equal(g_st, g_ws)
        lp3 = O.gather_units(joint, ys)
        costs, grads = O.ctct_loss_fwd(lp3, ys, lx, ly)
        np.testing.assert_allclose(c_st, costs, rtol=1e-5)
        np.testing.assert_allclose(g_st, grads, atol=1e-4, rtol=0)
        assert np.all(g_st[grads == 0] == 0)
    # a problem whose work buffers exceed the array is refused before any launch
    N, T, U = 64, 600, 60
    assert lib.warpctct_workspace_bytes(N, T, U) > STATIC_BYTES
    x = torch.zeros(8, device="cuda")
    p = hip_lib.ptr
    rc = lib.warpctct_loss_forward_static(p(x), 0, p(x), p(x), p(x), N, T, U, 16, p(x), p(x),
                                          hip_lib.stream_ptr())
    assert rc == ETOOLARGE
    assert b"static scratch" in lib.warpctct_error_string(rc)
    # no-grad mode (unit_grads NULL) through the same array
    joint, ys, lx, ly = small
    N, T, U1, V = joint.shape
    costs = torch.full((N,), float("nan"), device="cuda")
    d_joint, d_ys, d_lx, d_ly = dev(joint), dev(ys), dev(lx), dev(ly)
    hip_lib.check(lib.warpctct_loss_forward_static(p(d_joint), 0, p(d_ys), p(d_lx), p(d_ly), N, T,
                                                   U1 - 1, V, p(costs), p(None),
                                                   hip_lib.stream_ptr()))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(costs.cpu().numpy(), c_st)
