"""ctypes loader for the C oracle (oracle/ctct_oracle.c).  TEST INFRASTRUCTURE
ONLY — see ctct_oracle.py.  Build with `make -C oracle`."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
# (CTCT_ORACLE_LIB: another build of the same sources, e.g. with sanitizers)
_SO = os.environ.get("CTCT_ORACLE_LIB") or os.path.join(_HERE, "libctct_oracle.so")
_lib = None


def build(force=False):
    """Compile the C oracle in place (gcc + OpenMP)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.check_call(["make", "-C", _HERE, "libctct_oracle.so"], stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
    return _lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _real(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32"
    if dtype == np.float64:
        return "f64"
    raise TypeError(dtype)


def num_threads():
    return int(lib().oracle_num_threads())


def set_num_threads(n):
    lib().oracle_set_num_threads(int(n))


def ctct_loss_fwd(lp3, ys, lx, ly, requires_grad=True, dtype=np.float64):
    """costs (N,), grads (N,T,U+1,3) or None; arithmetic in `dtype`."""
    suf = _real(dtype)
    lp3 = np.ascontiguousarray(lp3, dtype=dtype)
    ys = np.ascontiguousarray(ys, dtype=np.int32)
    lx = np.ascontiguousarray(lx, dtype=np.int32)
    ly = np.ascontiguousarray(ly, dtype=np.int32)
    N, T, U1, three = lp3.shape
    assert three == 3 and ys.shape == (N, U1 - 1)
    costs = np.zeros(N, dtype=dtype)
    grads = np.empty_like(lp3) if requires_grad else None
    rc = getattr(lib(), "oracle_ctct_loss_fwd_" + suf)(
        _p(lp3), _p(ys), _p(lx), _p(ly), N, T, U1 - 1, _p(costs),
        _p(grads) if requires_grad else None)
    if rc:
        raise RuntimeError("oracle_ctct_loss_fwd failed: %d" % rc)
    return costs, grads


def ctct_loss_dense(joint, ys, lx, ly, grad_out=None, want_grad=True, dtype=np.float32):
    """costs (N,), dense (N,T,U+1,V) or None for the whole ctct_loss path."""
    suf = _real(dtype)
    joint = np.ascontiguousarray(joint, dtype=dtype)
    ys = np.ascontiguousarray(ys, dtype=np.int32)
    lx = np.ascontiguousarray(lx, dtype=np.int32)
    ly = np.ascontiguousarray(ly, dtype=np.int32)
    N, T, U1, V = joint.shape
    costs = np.zeros(N, dtype=dtype)
    dense = np.empty_like(joint) if want_grad else None
    go = None if grad_out is None else np.ascontiguousarray(grad_out, dtype=dtype)
    rc = getattr(lib(), "oracle_ctct_loss_dense_" + suf)(
        _p(joint), _p(ys), _p(lx), _p(ly), N, T, U1 - 1, V,
        _p(go) if go is not None else None, _p(costs), _p(dense) if want_grad else None)
    if rc:
        raise RuntimeError("oracle_ctct_loss_dense failed: %d" % rc)
    return costs, dense


def log_matmul(lhs, rhs, dtype=np.float64):
    suf = _real(dtype)
    lhs = np.ascontiguousarray(lhs, dtype=dtype)
    rhs = np.ascontiguousarray(rhs, dtype=dtype)
    B, M, K = lhs.shape
    Nn = rhs.shape[2]
    assert rhs.shape[:2] == (B, K)
    res = np.empty((B, M, Nn), dtype=dtype)
    getattr(lib(), "oracle_log_matmul_" + suf)(_p(lhs), _p(rhs), B, M, K, Nn, _p(res))
    return res
