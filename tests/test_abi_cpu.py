"""CPU-side checks of the C-ABI library: it loads without a GPU, exports every
symbol the header declares, and rejects bad arguments without touching a
device."""
import ctypes

import hip_lib


def test_library_exports_every_declared_symbol():
    lib = hip_lib.lib()
    names = hip_lib.declared_symbols()
    assert "warpctct_loss_forward_f32" in names and "warpctct_dense_grad_f32" in names
    for name in names:
        assert hasattr(lib, name), name


def test_library_exports_nothing_but_the_declared_symbols():
    """The shared object is linked with hidden visibility and a version script:
    its dynamic symbol table holds the C ABI of include/warp_ctct_hip.h and no
    C++ internals, helper functions or compiler-generated data."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", hip_lib.LIB_PATH], capture_output=True,
                         text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if line.strip())
    assert exported == hip_lib.declared_symbols()


def test_version_and_error_strings():
    lib = hip_lib.lib()
    assert lib.warpctct_version().decode().count(".") == 2
    assert lib.warpctct_error_string(0) == b"ok"
    for code in range(1, 6):
        assert len(lib.warpctct_error_string(code)) > 3
    assert lib.warpctct_error_string(99) == b"unknown error"


def test_workspace_size_is_monotone_and_covers_buffers():
    lib = hip_lib.lib()
    N, T, U = 32, 250, 60
    need = lib.warpctct_workspace_bytes(N, T, U)
    P = lib.warpctct_padded_contexts(U)
    assert P == 64 and lib.warpctct_padded_contexts(64) == 128 and lib.warpctct_padded_contexts(0) == 64
    floor = 8 * N * T * P * 3 + 2 * 8 * N * (T + 1) * P * 2
    assert need >= floor and need < floor + 3 * 256
    # wider than one wavefront: the relay slots are part of the workspace
    lib.warpctct_lattice_relay_bytes.restype = ctypes.c_size_t
    wide = lib.warpctct_workspace_bytes(N, T, 100)
    floor = 8 * N * T * 128 * 3 + 2 * 8 * N * (T + 1) * 128 * 2 + lib.warpctct_lattice_relay_bytes(N, T, 100)
    assert wide >= floor and wide < floor + 4 * 256
    assert lib.warpctct_workspace_bytes(N, T + 1, U) > need
    assert lib.warpctct_workspace_bytes(-1, T, U) == 0


def test_invalid_arguments_are_rejected_on_the_host():
    lib = hip_lib.lib()
    null = ctypes.c_void_p(0)
    EINVAL, EWORKSPACE = 1, 3
    # negative size / null pointers: refused before any launch
    assert lib.warpctct_gather_units_f32(null, null, null, null, null, -1, 4, 2, 8, null) == EINVAL
    assert lib.warpctct_gather_units_f32(null, null, null, null, null, 2, 4, 2, 8, null) == EINVAL
    assert lib.warpctct_dense_grad_f32(null, null, null, null, null, null, 2, 4, 2, 8, null) == EINVAL
    buf = (ctypes.c_float * 16)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    lib.warpctct_lattice_relay_bytes.restype = ctypes.c_size_t
    # a lattice of more than 64 contexts needs relay scratch: missing or too small is refused
    assert lib.warpctct_lattice_relay_bytes(3, 10, 63) == 0
    need = lib.warpctct_lattice_relay_bytes(3, 10, 64)
    assert need >= 3 * 2 * 1 * 10 * 8 and lib.warpctct_lattice_relay_bytes(3, 10, 300) == 4 * need
    assert lib.warpctct_lattice_f32(p, p, p, p, p, p, p, 3, 10, 64, 0, null, ctypes.c_size_t(0),
                                    null) == EINVAL
    assert lib.warpctct_lattice_f32(p, p, p, p, p, p, p, 3, 10, 64, 0, p, ctypes.c_size_t(need - 8),
                                    null) == EWORKSPACE
    # sizes whose cell count does not fit 31 bits
    assert lib.warpctct_lattice_f32(p, p, p, p, p, p, p, 1, 1 << 26, 63, 0, null,
                                    ctypes.c_size_t(0), null) == EINVAL
    assert lib.warpctct_loss_forward_f32(p, p, p, p, 1, 1, 1, 8, p, ctypes.c_size_t(16), p, p,
                                         null) == EWORKSPACE
    # empty batch is a no-op
    assert lib.warpctct_loss_forward_f32(null, null, null, null, 0, 4, 2, 8, null,
                                         ctypes.c_size_t(0), null, null, null) == 0
    # the forward on the library's own scratch array: same argument checks, and a
    # problem larger than the array is refused before any device is touched
    ETOOLARGE = 5
    assert lib.warpctct_loss_forward_static(null, 0, null, null, null, 2, 4, 2, 8, null, null,
                                            null) == EINVAL
    assert lib.warpctct_loss_forward_static(p, 4, p, p, p, 2, 4, 2, 8, p, p, null) == EINVAL
    assert lib.warpctct_workspace_bytes(64, 600, 60) > (32 << 20)
    assert lib.warpctct_loss_forward_static(p, 0, p, p, p, 64, 600, 60, 8, p, p, null) == ETOOLARGE
    assert lib.warpctct_loss_forward_static(null, 0, null, null, null, 0, 4, 2, 8, null, null,
                                            null) == 0


def test_generic_dtype_and_logits_entry_points_check_their_arguments():
    lib = hip_lib.lib()
    lib.warpctct_logits_workspace_bytes.restype = ctypes.c_size_t
    lib.warpctct_logmm_workspace_bytes.restype = ctypes.c_size_t
    lib.warpctct_simple_backward_workspace_bytes.restype = ctypes.c_size_t
    null = ctypes.c_void_p(0)
    EINVAL, EWORKSPACE = 1, 3
    buf = (ctypes.c_float * 16)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    small = ctypes.c_size_t(16)
    f = ctypes.c_float
    # unknown element type, unknown reduction, reduction without a place for the result
    assert lib.warpctct_loss_lattice(p, 7, p, p, p, 1, 1, 1, 8, p, small, p, 1, 0, 0, null, null) == EINVAL
    assert lib.warpctct_loss_lattice(p, 0, p, p, p, 1, 1, 1, 8, p, small, p, 1, 3, 0, p, null) == EINVAL
    assert lib.warpctct_loss_lattice(p, 2, p, p, p, 1, 1, 1, 8, p, small, p, 1, 2, 0, null, null) == EINVAL
    # valid arguments, workspace too small (checked before any launch)
    assert lib.warpctct_loss_lattice(p, 2, p, p, p, 1, 1, 1, 8, p, small, p, 1, 2, 0, p, null) == EWORKSPACE
    assert lib.warpctct_logits_loss_lattice(p, 1, p, p, p, 1, 1, 1, 8, p, small, p, 1, 0, 0, null,
                                            null) == EWORKSPACE
    # the clearing form refuses the same things, before it forks its stream
    strides = (ctypes.c_long * 4)(16, 16, 8, 1)
    assert lib.warpctct_loss_lattice_clearing(p, 7, strides, p, p, p, 1, 1, 1, 8, p, small, p, 1, 0,
                                              0, null, p, small, null) == EINVAL
    assert lib.warpctct_loss_lattice_clearing(p, 0, null, p, p, p, 1, 1, 1, 8, p, small, p, 1, 0,
                                              0, null, p, small, null) == EINVAL
    assert lib.warpctct_loss_lattice_clearing(p, 2, strides, p, p, p, 1, 1, 1, 8, p, small, p, 1, 2,
                                              0, p, p, small, null) == EWORKSPACE
    assert lib.warpctct_logits_grad_lattice(p, small, p, 0, p, p, p, p, 1, f(1.0), 0, p, 1, 1, 1, 8,
                                            null) == EWORKSPACE
    assert lib.warpctct_logits_grad_lattice(p, small, p, 5, p, p, p, p, 1, f(1.0), 0, p, 1, 1, 1, 8,
                                            null) == EINVAL
    assert lib.warpctct_dense_grad_lattice(p, small, p, p, p, p, 1, f(1.0), 0, null, 0, 1, 1, 1, 8,
                                           null) == EINVAL
    assert lib.warpctct_loss_forward(p, 9, p, p, p, 1, 1, 1, 8, p, small, p, p, null) == EINVAL
    assert lib.warpctct_zero_fill(null, ctypes.c_size_t(64), null) == EINVAL
    assert lib.warpctct_zero_fill(null, ctypes.c_size_t(0), null) == 0
    # the wait limit of the chained lattice: a process-wide setting, returned on change
    default = lib.warpctct_lattice_wait_limit(5)
    assert default > 1000 and lib.warpctct_lattice_wait_limit(-1) == 5
    assert lib.warpctct_lattice_wait_limit(-1) == default
    # from how many frames on the joiner sweeps in the linear domain: the same
    # kind of setting (negative: the defaults), also through the Python package
    assert lib.warpctct_joiner_linear_lattice(0) < 0
    assert lib.warpctct_joiner_linear_lattice(700) == 0
    assert lib.warpctct_joiner_linear_lattice(-5) == 700
    import warp_ctct
    assert warp_ctct.joiner_linear_lattice(1) < 0 and warp_ctct.joiner_linear_lattice(-1) == 1
    assert lib.warpctct_joiner_linear_lattice(-1) < 0
    # workspace sizes: logits = lattice + one float per row; log-matmul grows with K
    N, T, U = 4, 50, 20
    lat = lib.warpctct_workspace_bytes(N, T, U)
    lg = lib.warpctct_logits_workspace_bytes(N, T, U)
    assert lat + 4 * N * T * (U + 1) <= lg < lat + 4 * N * T * (U + 1) + 256
    assert lib.warpctct_logmm_padded_reduction(1) == 32 and lib.warpctct_logmm_padded_reduction(2048) == 2048
    assert lib.warpctct_logmm_padded_reduction(2049) == 2080
    w1 = lib.warpctct_logmm_workspace_bytes(2, 10, 64, 5)
    w2 = lib.warpctct_logmm_workspace_bytes(2, 10, 65, 5)
    assert w2 - w1 == 4 * 32 * 2 * (10 + 5)
    assert lib.warpctct_simple_backward_workspace_bytes(N, T, U) >= 4 * N * T * (U + 1) + 4 * N * T
    # the pair factors once more as three bfloat16 planes over frames padded to 32,
    # and a float per padded frame, where the gradient wrt g uses them (U+1 <= 96, T >= 128)
    small = lib.warpctct_simple_backward_workspace_bytes(2, 120, 80)
    assert small < 2 * 120 * 96 * 4 + 2 * 120 * 4 + 1024
    big = lib.warpctct_simple_backward_workspace_bytes(2, 400, 80)
    assert big >= 2 * 400 * 96 * 4 + 2 * 400 * 4 + 3 * 2 * 96 * 416 * 2 + 2 * 416 * 4
    # whether the joiner path stores exp(f - fmax): not for its production shapes
    lib.warpctct_simple_needs_fexp.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_int]
    aligned, odd = ctypes.c_void_p(4096), ctypes.c_void_p(4100)
    assert lib.warpctct_simple_needs_fexp(aligned, 400, 80, 2048) == 0
    assert lib.warpctct_simple_needs_fexp(aligned, 128, 0, 512) == 0
    assert lib.warpctct_simple_needs_fexp(odd, 400, 80, 2048) == 1       # rows not 16-byte aligned
    assert lib.warpctct_simple_needs_fexp(aligned, 400, 80, 2040) == 1   # not whole chunks of 32
    assert lib.warpctct_simple_needs_fexp(aligned, 400, 80, 4096) == 1   # beyond the slab kernels
    assert lib.warpctct_simple_needs_fexp(aligned, 100, 80, 2048) == 1   # too few frames
    assert lib.warpctct_simple_needs_fexp(aligned, 400, 100, 2048) == 1  # too many contexts


def test_status_word_entry_point_without_a_device():
    """warpctct_status refuses a null pointer, and reports that there is no
    usable device where there is none (it is the one entry point that talks to
    the device on its own; the CPU suite runs where no GPU is visible)."""
    lib = hip_lib.lib()
    EINVAL, ENODEVICE = 1, 4
    assert lib.warpctct_status(ctypes.c_void_p(0), 0) == EINVAL
    bits = ctypes.c_uint(0xdead)
    rc = lib.warpctct_status(ctypes.byref(bits), 1)
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        assert rc == 0 and bits.value < 8
    else:
        assert rc == ENODEVICE and bits.value == 0xdead
