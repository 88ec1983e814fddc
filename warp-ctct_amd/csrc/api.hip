// extern "C" surface of libwarpctct_hip.so (declared in include/warp_ctct_hip.h).
// Host code only: argument validation, workspace carving, kernel launches.
// No allocation, no host synchronisation, no process exit.
#include "warp_ctct_hip.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <mutex>

#include "launch.h"

// Work buffers of warpctct_loss_forward_static: part of the code object, one
// copy per GPU at its own address.  In host code this name is only a handle
// for hipGetSymbolAddress, never a device address.  (No `used` attribute: it
// would keep the device symbol local, and the runtime finds it by name.)
static __device__ __align__(256) unsigned char scratch[WARPCTCT_STATIC_SCRATCH_BYTES];

namespace {

using namespace wctct;

constexpr int kMaxGrid = 65535;

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline int done(hipError_t e) {
    if (e == hipSuccess) return WARPCTCT_OK;
    return e == hipErrorInvalidValue ? WARPCTCT_EINVAL : WARPCTCT_ELAUNCH;
}

// N is a grid dimension; cells of one sample are counted in 32 bits.  (The
// reference has no limit of its own: its grid is (sT/32, 2U+1, N),
// csrc/gather.cu:293-297, i.e. 2U+1 <= 65535 and N <= 65535 in practice.)
inline bool dims_ok(int N, int T, int U) {
    return N >= 0 && T >= 0 && U >= 0 && N <= kMaxGrid && U < (1 << 24) &&
           (long)T * padded_contexts(U) < (1L << 31);
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct Workspace {
    double *units;    // (N,T,P,3),   P = padded_contexts(U)
    double *alphas;   // (N,T+1,P,2)
    double *betas;    // (N,T+1,P,2)
    void *relay;      // lattice_relay_slots(N,T,U) 64-bit words (none for U+1 <= 64)
    unsigned *counter;   // arrivals of the batch reduction (see CostReduce)
    size_t bytes;
};

Workspace carve(void *base, int N, int T, int U) {
    const size_t P = (size_t)padded_contexts(U);
    const size_t units_b = align256((size_t)N * T * P * 3 * sizeof(double));
    const size_t lat_b = align256((size_t)N * (T + 1) * P * 2 * sizeof(double));
    const uintptr_t p = reinterpret_cast<uintptr_t>(base);
    Workspace w;
    w.units = reinterpret_cast<double *>(p);
    w.alphas = reinterpret_cast<double *>(p + units_b);
    w.betas = reinterpret_cast<double *>(p + units_b + lat_b);
    const size_t relay_b = align256(lattice_relay_slots(N, T, U) * sizeof(unsigned long long));
    w.relay = relay_b ? reinterpret_cast<void *>(p + units_b + 2 * lat_b) : nullptr;
    w.counter = reinterpret_cast<unsigned *>(p + units_b + 2 * lat_b + relay_b);
    w.bytes = units_b + 2 * lat_b + relay_b + 256;
    return w;
}

int forward_from_units(const Workspace &w, const int *ys, const int *lx, const int *ly, int N,
                       int T, int U, float *costs, float *unit_grads, hipStream_t stream) {
    LatticeArgs a = {};
    a.units = w.units;
    a.ys = ys;
    a.lx = lx;
    a.ly = ly;
    a.alphas = w.alphas;
    a.betas = w.betas;
    a.relay = w.relay;
    a.costs = costs;
    a.N = N;
    a.T = T;
    a.U = U;
    a.beta_only = (unit_grads == nullptr);
    int rc = done(launch_lattice(a, stream));
    if (rc != WARPCTCT_OK || !unit_grads) return rc;
    return done(launch_unit_grads(w.units, ys, lx, ly, w.alphas, w.betas, unit_grads, N, T, U,
                                  stream));
}

// from how many frames on the fused joiner forward sweeps its lattices in the
// linear domain first (warpctct_joiner_linear_lattice; 0: never; negative: the
// defaults below).  The linear sweeps save 35-50 ns per frame and cost ~10 us
// per call (three launches that return at once, a slower gather; the gather
// more so where it also finishes the denominators): measured, with the
// normalisation they gain from 384 frames on (+0.6 to +2.9 % per step at 400
// frames for 4 to 32 lattices of 81 contexts, V = 2048), and without it the GPU
// gains from about 450 frames on.  Without the normalisation, though, a step of
// that length has so little other work that it may be bound by the host, which
// the three additional launches cost ~9 us (-4 to -10 % at 400 frames): the
// limit there lies where the step is bound by the GPU on a slow host too.
constexpr int kLinearFromFrames = 768, kLinearFromFramesNormalized = 384;
std::atomic<int> g_linear_from{-1};

// With the default limits, only for batches whose sweeps are bound by the
// latency of their instructions rather than by the memory system, where the
// linear form has nothing to gain (it moves 24 + 8 bytes per column, direction
// and frame, the log form 12 + 16): up to 256 wavefronts of sweeps (one per
// compute unit) where a lattice needs one per direction, up to 768 for chains,
// which the log domain sweeps more slowly.  Measured at 800 and 1500 frames: per
// step +2 to +6 % for 64-128 lattices of one wavefront per direction, -1.6 %
// for 192; chains of three +10 to +18 % for 32-64 lattices, +0.4 to +1 % for
// 128-256; chains of five +7 to +10 % for 32-64, -0.4 % for 128.
bool linear_batch_fits(int N, int U) {
    const long W = lin_waves(U), wavefronts = 2L * N * W;
    return wavefronts <= (W == 1 ? 256 : 768);
}

struct SimpleWorkspace {
    Workspace lattice;
    float *unit_grads;   // (N,T,U+1,3)
    float *partial;      // logmm_fwd_partial_floats: partial sums of a split log-matmul reduction
    // For the lattices in the linear domain (launch_lattice_lin): units and
    // lattices in that form's layout, in the memory of the log-domain ones (which
    // are written only if the linear ones are given up, and from scratch then);
    // scales, the flag that sends the batch through the log-domain kernels, and
    // an arrival counter of its own for the batch reduction (the log-domain one
    // lies in memory that the linear buffers may cover).
    double *lin_units, *lin_alphas, *lin_betas;
    int *lin_scales;
    unsigned *lin_flag, *lin_counter;
    size_t bytes;
};

SimpleWorkspace carve_simple(void *base, int N, int T, int U) {
    SimpleWorkspace w;
    w.lattice = carve(base, N, T, U);
    const bool lin = simple_grads_lin_applies(T, U);
    const size_t Pl = (size_t)lin_padded(U);
    const size_t lin_units_b = lin ? align256((size_t)N * T * Pl * kLinUnit * sizeof(double)) : 0;
    const size_t lin_lat_b = lin ? align256((size_t)N * (T + 1) * Pl * 2 * sizeof(unsigned)) : 0;
    const uintptr_t b = reinterpret_cast<uintptr_t>(base);
    w.lin_units = reinterpret_cast<double *>(b);
    w.lin_alphas = reinterpret_cast<double *>(b + lin_units_b);
    w.lin_betas = reinterpret_cast<double *>(b + lin_units_b + lin_lat_b);
    const size_t lattice_b = std::max(w.lattice.bytes, lin_units_b + 2 * lin_lat_b);
    const uintptr_t p = b + lattice_b;
    const size_t ug_b = align256((size_t)N * T * (U + 1) * 3 * sizeof(float));
    w.unit_grads = reinterpret_cast<float *>(p);
    w.partial = reinterpret_cast<float *>(p + ug_b);
    const size_t partial_b = align256(logmm_fwd_partial_floats(N, T, U + 1) * sizeof(float));
    const size_t scales_b = lin ? align256(lattice_lin_scales(N, T, U) * sizeof(int)) : 0;
    w.lin_scales = reinterpret_cast<int *>(p + ug_b + partial_b);
    w.lin_flag = reinterpret_cast<unsigned *>(p + ug_b + partial_b + scales_b);
    w.lin_counter = w.lin_flag + 32;
    w.bytes = lattice_b + ug_b + partial_b + scales_b + 256;
    return w;
}

// Work buffers of the log-matmul backward: pair factors (B,M,logmm_pair_row(Nn)) and row flags (B,M).
struct PairWorkspace {
    float *factors;
    int *flags;
    LogmmPairPlanes planes;   // null where they have no use
    size_t bytes;
};

PairWorkspace carve_pairs(void *base, int B, int M, int Nn) {
    PairWorkspace w;
    const size_t fb = align256((size_t)B * M * logmm_pair_row(Nn) * sizeof(float));
    w.factors = reinterpret_cast<float *>(base);
    w.flags = reinterpret_cast<int *>(reinterpret_cast<uintptr_t>(base) + fb);
    w.bytes = fb + align256((size_t)B * M * sizeof(int));
    const size_t pb = logmm_pair_planes_bytes(B, M, Nn), sb = logmm_pair_shifts_bytes(B, M, Nn);
    w.planes = {nullptr, nullptr};
    if (pb && sb) {
        w.planes.planes = reinterpret_cast<unsigned short *>(reinterpret_cast<uintptr_t>(base) + w.bytes);
        w.planes.shifts = reinterpret_cast<float *>(reinterpret_cast<uintptr_t>(base) + w.bytes + pb);
        w.bytes += pb + sb;
    }
    return w;
}

// Work buffers of the standalone log-matmul: maxima, shifted exponentials, pairs.
struct LogmmWorkspace {
    LogmmShifted sh;
    PairWorkspace pw;
    float *partial;   // forward only: partial sums of a split reduction
    size_t bytes;
};

LogmmWorkspace carve_logmm(void *base, int B, int M, int K, int Nn) {
    LogmmWorkspace w;
    const size_t Kp = (size_t)logmm_padded_reduction(K);
    uintptr_t p = reinterpret_cast<uintptr_t>(base);
    const uintptr_t p0 = p;
    w.sh.lmax = reinterpret_cast<float *>(p);
    p += align256((size_t)B * M * sizeof(float));
    w.sh.rmax = reinterpret_cast<float *>(p);
    p += align256((size_t)B * Nn * sizeof(float));
    w.sh.El = reinterpret_cast<float *>(p);
    p += align256((size_t)B * M * Kp * sizeof(float));
    w.sh.Er = reinterpret_cast<float *>(p);
    p += align256((size_t)B * Nn * Kp * sizeof(float));
    w.pw = carve_pairs(reinterpret_cast<void *>(p), B, M, Nn);
    p += w.pw.bytes;
    w.partial = reinterpret_cast<float *>(p);
    p += align256(logmm_fwd_partial_floats(B, M, Nn) * sizeof(float));
    w.bytes = p - p0;
    return w;
}

// Address of `scratch` on the current device, looked up once per device with
// that device current and kept for the life of the process.
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void **out) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices)
        return WARPCTCT_ENODEVICE;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[device]) {
        void *p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p)
            return WARPCTCT_ENODEVICE;
        g_scratch_ptr[device] = p;
    }
    *out = g_scratch_ptr[device];
    return WARPCTCT_OK;
}

// lattice + unit gradients + reductions, shared by the two simple forwards
int simple_from_units(const SimpleWorkspace &w, const int *ys, const int *lx, const int *ly, int N,
                      int T, int U, float *costs, float *grad_f, float *grad_g, float *grad_den,
                      bool want_grad, bool relay_is_clear, const CostReduce &reduce,
                      hipStream_t stream, const unsigned *only_if = nullptr) {
    // alpha is needed only for the gradients; those are reduced straight from the
    // lattices (the unit-gradient region of the workspace holds the partial sums)
    LatticeArgs a = {};
    a.units = w.lattice.units;
    a.ys = ys;
    a.lx = lx;
    a.ly = ly;
    a.alphas = w.lattice.alphas;
    a.betas = w.lattice.betas;
    a.relay = w.lattice.relay;
    a.relay_is_clear = relay_is_clear;
    a.costs = costs;
    a.N = N;
    a.T = T;
    a.U = U;
    a.beta_only = !want_grad;
    a.reduce = reduce;
    // only_if: the run behind the lattices in the linear domain (see the caller)
    int rc = done(launch_lattice(a, stream, only_if));
    if (rc != WARPCTCT_OK || !want_grad) return rc;
    return done(launch_simple_grads(w.lattice.units, ys, lx, ly, w.lattice.alphas, w.lattice.betas,
                                    w.unit_grads, grad_f, grad_g, grad_den, N, T, U, stream, only_if));
}

}  // namespace

extern "C" {

const char *warpctct_error_string(int code) {
    switch (code) {
        case WARPCTCT_OK: return "ok";
        case WARPCTCT_EINVAL:
            return "invalid argument (null pointer, negative size, or size limit: N <= 65535, "
                   "T * (U+1 rounded up to 64) < 2^31)";
        case WARPCTCT_ELAUNCH: return "kernel launch failed";
        case WARPCTCT_EWORKSPACE: return "workspace too small";
        case WARPCTCT_ENODEVICE: return "no usable HIP device";
        case WARPCTCT_ETOOLARGE:
            return "the work buffers of this problem exceed the static scratch array "
                   "(WARPCTCT_STATIC_SCRATCH_BYTES); use the entry point with a workspace argument";
        default: return "unknown error";
    }
}

const char *warpctct_version(void) { return "0.2.0"; }

int warpctct_padded_contexts(int U) { return U < 0 ? 0 : padded_contexts(U); }

size_t warpctct_workspace_bytes(int N, int T, int U) {
    if (N < 0 || T < 0 || U < 0) return 0;
    return carve(nullptr, N, T, U).bytes;
}

int warpctct_gather_units_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              double *units_out, int N, int T, int U, int V, void *stream) {
    if (!dims_ok(N, T, U) || V < 1) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!joint || !lx || !ly || !units_out || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    return done(launch_gather_units(joint, dense_joint_strides(T, U, V), kIoF32, ys, lx, ly,
                                    units_out, N, T, U, V, false, nullptr, RelaySlots{},
                                    as_stream(stream)));
}

int warpctct_scale_units_f32(const float *units_nat, const int *lx, const int *ly,
                             double *units_out, int N, int T, int U, void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!units_nat || !lx || !ly || !units_out) return WARPCTCT_EINVAL;
    return done(launch_scale_units(units_nat, lx, ly, units_out, N, T, U, as_stream(stream)));
}

int warpctct_simple_units_f32(const float *f_g, const float *g_g, const float *den,
                              const int *lx, const int *ly, double *units_out, int N, int T, int U,
                              void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!f_g || !g_g || !lx || !ly || !units_out) return WARPCTCT_EINVAL;
    return done(launch_simple_units(f_g, g_g, den, lx, ly, units_out, N, T, U, as_stream(stream)));
}

int warpctct_lattice_wait_limit(int spins) { return lattice_wait_limit(spins); }

int warpctct_joiner_linear_lattice(int from_frames) {
    return g_linear_from.exchange(from_frames < 0 ? -1 : from_frames, std::memory_order_relaxed);
}

size_t warpctct_lattice_relay_bytes(int N, int T, int U) {
    if (N < 0 || T < 0 || U < 0) return 0;
    return lattice_relay_slots(N, T, U) * sizeof(unsigned long long);
}

int warpctct_lattice_f32(const double *units, const int *ys, const int *lx, const int *ly,
                         double *alphas, double *betas, float *costs, int N, int T, int U,
                         int beta_only, void *relay, size_t relay_bytes, void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !betas || !costs || (T > 0 && !units) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    if (!beta_only && !alphas) return WARPCTCT_EINVAL;
    const size_t relay_need = warpctct_lattice_relay_bytes(N, T, U);
    if (relay_need > 0 && !relay) return WARPCTCT_EINVAL;
    if (relay_bytes < relay_need) return WARPCTCT_EWORKSPACE;
    if (relay_need > 0 && (reinterpret_cast<uintptr_t>(relay) & 7u)) return WARPCTCT_EINVAL;
    LatticeArgs a = {};
    a.units = units;
    a.ys = ys;
    a.lx = lx;
    a.ly = ly;
    a.alphas = alphas;
    a.betas = betas;
    a.relay = relay_need > 0 ? relay : nullptr;
    a.costs = costs;
    a.N = N;
    a.T = T;
    a.U = U;
    a.beta_only = beta_only != 0;
    return done(launch_lattice(a, as_stream(stream)));
}

int warpctct_unit_grads_f32(const double *units, const int *ys, const int *lx, const int *ly,
                            const double *alphas, const double *betas, float *unit_grads, int N,
                            int T, int U, void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!units || !lx || !ly || !alphas || !betas || !unit_grads || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    return done(launch_unit_grads(units, ys, lx, ly, alphas, betas, unit_grads, N, T, U,
                                  as_stream(stream)));
}

int warpctct_dense_grad_f32(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                            const float *grad_out, float *dense, int N, int T, int U, int V,
                            void *stream) {
    if (!dims_ok(N, T, U) || V < 1) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!unit_grads || !lx || !ly || !dense || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    return done(launch_dense_grad(unit_grads, ys, lx, ly, grad_out, dense, N, T, U, V,
                                  as_stream(stream)));
}

int warpctct_dense_patch_f32(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                             const float *grad_out, float *dense, int N, int T, int U, int V,
                             void *stream) {
    if (!dims_ok(N, T, U) || V < 1) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!unit_grads || !lx || !ly || !dense || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    return done(launch_dense_patch(unit_grads, ys, lx, ly, grad_out, dense, N, T, U, V,
                                   as_stream(stream)));
}

int warpctct_loss_lattice(const void *joint, int dtype, const int *ys, const int *lx,
                          const int *ly, int N, int T, int U, int V, void *workspace,
                          size_t workspace_bytes, float *costs, int want_alpha, int reduction,
                          int average_frames, float *reduced, void *stream) {
    const JointStrides js = dense_joint_strides(T, U, V);
    const long strides[4] = {js.n, js.t, js.u, js.v};
    return warpctct_loss_lattice_strided(joint, dtype, strides, ys, lx, ly, N, T, U, V, workspace,
                                         workspace_bytes, costs, want_alpha, reduction,
                                         average_frames, reduced, stream);
}

namespace {

// What warpctct_loss_lattice_strided refuses, before anything is launched.
int check_loss_lattice(const void *joint, int dtype, const long *strides, const int *ys,
                       const int *lx, const int *ly, int N, int T, int U, int V,
                       const void *workspace, size_t workspace_bytes, const float *costs,
                       int reduction, const float *reduced) {
    if (!dims_ok(N, T, U) || V < 1 || !io_valid(dtype) || reduction < 0 || reduction > 2 ||
        !strides)
        return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !costs || !workspace || (T > 0 && !joint) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    if (reduction != 0 && !reduced) return WARPCTCT_EINVAL;
    if (workspace_bytes < carve(nullptr, N, T, U).bytes) return WARPCTCT_EWORKSPACE;
    return WARPCTCT_OK;
}

// gather + lattices, with `fill` cleared inside the lattice kernel's launch
int loss_lattice_run(const void *joint, int dtype, const long *strides, const int *ys,
                     const int *lx, const int *ly, int N, int T, int U, int V, void *workspace,
                     float *costs, int want_alpha, int reduction, int average_frames,
                     float *reduced, const FillTail &fill, hipStream_t st) {
    const JointStrides js = {strides[0], strides[1], strides[2], strides[3]};
    const Workspace w = carve(workspace, N, T, U);
    unsigned *counter = reduction != 0 ? w.counter : nullptr;
    if (T > 0) {
        int rc = done(launch_gather_units(joint, js, dtype, ys, lx, ly, w.units, N, T, U, V, true,
                                          counter, relay_slots_of(w.relay, N, T, U), st));
        if (rc != WARPCTCT_OK) return rc;
    } else if (counter) {
        int rc = done(launch_clear_counter(counter, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    LatticeArgs a = {};
    a.units = w.units;
    a.ys = ys;
    a.lx = lx;
    a.ly = ly;
    a.alphas = w.alphas;
    a.betas = w.betas;
    a.relay = w.relay;
    a.relay_is_clear = T > 0;             // by the gather kernel
    a.costs = costs;
    a.N = N;
    a.T = T;
    a.U = U;
    a.beta_only = (want_alpha == 0);
    a.reduce.reduced = reduction != 0 ? reduced : nullptr;
    a.reduce.counter = counter;
    a.reduce.mode = reduction;
    a.reduce.average_frames = average_frames != 0;
    a.fill = fill;
    return done(launch_lattice(a, st));
}

}  // namespace

int warpctct_loss_lattice_clearing(const void *joint, int dtype, const long *strides,
                                   const int *ys, const int *lx, const int *ly, int N, int T,
                                   int U, int V, void *workspace, size_t workspace_bytes,
                                   float *costs, int want_alpha, int reduction, int average_frames,
                                   float *reduced, void *dense, size_t dense_bytes, void *stream) {
    int rc = check_loss_lattice(joint, dtype, strides, ys, lx, ly, N, T, U, V, workspace,
                                workspace_bytes, costs, reduction, reduced);
    if (rc != WARPCTCT_OK) return rc;
    hipStream_t st = as_stream(stream);
    if (!dense) dense_bytes = 0;
    if (N == 0) return done(launch_zero_fill_bytes(dense, dense_bytes, st));
    // the 16-byte vectors of the buffer ride in the lattice kernel's launch;
    // the few bytes before and after them (if any) are cleared on their own
    unsigned char *p = static_cast<unsigned char *>(dense);
    size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15u)) & 15u;
    if (head > dense_bytes) head = dense_bytes;
    FillTail fill;
    fill.p = p + head;
    fill.n4 = (dense_bytes - head) / 16;
    const size_t tail = dense_bytes - head - fill.n4 * 16;
    if ((rc = done(launch_zero_fill_bytes(p, head, st))) != WARPCTCT_OK) return rc;
    if ((rc = done(launch_zero_fill_bytes(p + head + fill.n4 * 16, tail, st))) != WARPCTCT_OK)
        return rc;
    return loss_lattice_run(joint, dtype, strides, ys, lx, ly, N, T, U, V, workspace, costs,
                            want_alpha, reduction, average_frames, reduced, fill, st);
}

int warpctct_loss_lattice_strided(const void *joint, int dtype, const long *strides,
                                  const int *ys, const int *lx, const int *ly, int N, int T, int U,
                                  int V, void *workspace, size_t workspace_bytes, float *costs,
                                  int want_alpha, int reduction, int average_frames,
                                  float *reduced, void *stream) {
    const int ok = check_loss_lattice(joint, dtype, strides, ys, lx, ly, N, T, U, V, workspace,
                                      workspace_bytes, costs, reduction, reduced);
    if (ok != WARPCTCT_OK || N == 0) return ok;
    return loss_lattice_run(joint, dtype, strides, ys, lx, ly, N, T, U, V, workspace, costs,
                            want_alpha, reduction, average_frames, reduced, FillTail(),
                            as_stream(stream));
}

int warpctct_loss_lattice_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              int N, int T, int U, int V, void *workspace, size_t workspace_bytes,
                              float *costs, int want_alpha, void *stream) {
    return warpctct_loss_lattice(joint, WARPCTCT_F32, ys, lx, ly, N, T, U, V, workspace,
                                 workspace_bytes, costs, want_alpha, 0, 0, nullptr, stream);
}

int warpctct_dense_patch_lattice(const void *workspace, size_t workspace_bytes, const int *ys,
                                 const int *lx, const int *ly, const float *grad_out,
                                 int grad_out_stride, float scale, int average_frames, void *dense,
                                 int dtype, int N, int T, int U, int V, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || grad_out_stride < 0 || !io_valid(dtype))
        return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!workspace || !lx || !ly || !dense || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    const Workspace w = carve(const_cast<void *>(workspace), N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    return done(launch_dense_patch_lattice(w.units, w.alphas, w.betas, ys, lx, ly, grad_out,
                                           grad_out_stride, scale, average_frames, dense, dtype, N,
                                           T, U, V, as_stream(stream)));
}

int warpctct_dense_grad_lattice(const void *workspace, size_t workspace_bytes, const int *ys,
                                const int *lx, const int *ly, const float *grad_out,
                                int grad_out_stride, float scale, int average_frames, void *dense,
                                int dtype, int N, int T, int U, int V, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || grad_out_stride < 0 || !io_valid(dtype))
        return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!workspace || !lx || !ly || !dense || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    if (workspace_bytes < carve(nullptr, N, T, U).bytes) return WARPCTCT_EWORKSPACE;
    int rc = done(launch_zero_fill_bytes(dense, (size_t)N * T * (U + 1) * V * io_size(dtype),
                                         as_stream(stream)));
    if (rc != WARPCTCT_OK) return rc;
    return warpctct_dense_patch_lattice(workspace, workspace_bytes, ys, lx, ly, grad_out,
                                        grad_out_stride, scale, average_frames, dense, dtype, N, T,
                                        U, V, stream);
}

int warpctct_dense_patch_lattice_f32(const void *workspace, size_t workspace_bytes, const int *ys,
                                     const int *lx, const int *ly, const float *grad_out,
                                     int grad_out_stride, float scale, int average_frames,
                                     float *dense, int N, int T, int U, int V, void *stream) {
    return warpctct_dense_patch_lattice(workspace, workspace_bytes, ys, lx, ly, grad_out,
                                        grad_out_stride, scale, average_frames, dense,
                                        WARPCTCT_F32, N, T, U, V, stream);
}

int warpctct_dense_grad_lattice_f32(const void *workspace, size_t workspace_bytes, const int *ys,
                                    const int *lx, const int *ly, const float *grad_out,
                                    int grad_out_stride, float scale, int average_frames,
                                    float *dense, int N, int T, int U, int V, void *stream) {
    return warpctct_dense_grad_lattice(workspace, workspace_bytes, ys, lx, ly, grad_out,
                                       grad_out_stride, scale, average_frames, dense, WARPCTCT_F32,
                                       N, T, U, V, stream);
}

namespace {

// Lattice workspace followed by the row-wise logsumexp (N,T,U+1) of the logits.
struct LogitsWorkspace {
    Workspace lattice;
    float *lse;
    size_t bytes;
};

LogitsWorkspace carve_logits(void *base, int N, int T, int U) {
    LogitsWorkspace w;
    w.lattice = carve(base, N, T, U);
    w.lse = reinterpret_cast<float *>(reinterpret_cast<uintptr_t>(base) + w.lattice.bytes);
    w.bytes = w.lattice.bytes + align256((size_t)N * T * (U + 1) * sizeof(float));
    return w;
}

}  // namespace

size_t warpctct_logits_workspace_bytes(int N, int T, int U) {
    if (N < 0 || T < 0 || U < 0) return 0;
    return carve_logits(nullptr, N, T, U).bytes;
}

int warpctct_logits_loss_lattice(const void *logits, int dtype, const int *ys, const int *lx,
                                 const int *ly, int N, int T, int U, int V, void *workspace,
                                 size_t workspace_bytes, float *costs, int want_alpha,
                                 int reduction, int average_frames, float *reduced, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || !io_valid(dtype) || reduction < 0 || reduction > 2)
        return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !costs || !workspace || (T > 0 && !logits) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    if (reduction != 0 && !reduced) return WARPCTCT_EINVAL;
    const LogitsWorkspace w = carve_logits(workspace, N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    unsigned *counter = reduction != 0 ? w.lattice.counter : nullptr;
    if (T > 0) {
        int rc = done(launch_logits_units(logits, dtype, ys, lx, ly, w.lattice.units, w.lse, N, T,
                                          U, V, counter, st));
        if (rc != WARPCTCT_OK) return rc;
    } else if (counter) {
        int rc = done(launch_clear_counter(counter, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    LatticeArgs a = {};
    a.units = w.lattice.units;
    a.ys = ys;
    a.lx = lx;
    a.ly = ly;
    a.alphas = w.lattice.alphas;
    a.betas = w.lattice.betas;
    a.relay = w.lattice.relay;
    a.costs = costs;
    a.N = N;
    a.T = T;
    a.U = U;
    a.beta_only = (want_alpha == 0);
    a.reduce.reduced = reduction != 0 ? reduced : nullptr;
    a.reduce.counter = counter;
    a.reduce.mode = reduction;
    a.reduce.average_frames = average_frames != 0;
    return done(launch_lattice(a, st));
}

int warpctct_logits_grad_lattice(const void *workspace, size_t workspace_bytes,
                                 const void *logits, int dtype, const int *ys, const int *lx,
                                 const int *ly, const float *grad_out, int grad_out_stride,
                                 float scale, int average_frames, void *grad_logits, int N, int T,
                                 int U, int V, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || grad_out_stride < 0 || !io_valid(dtype))
        return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!workspace || !logits || !lx || !ly || !grad_logits || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    const LogitsWorkspace w = carve_logits(const_cast<void *>(workspace), N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    return done(launch_logits_grad(logits, dtype, w.lse, w.lattice.units, w.lattice.alphas,
                                   w.lattice.betas, ys, lx, ly, grad_out, grad_out_stride, scale,
                                   average_frames, grad_logits, N, T, U, V, as_stream(stream)));
}

int warpctct_zero_fill(void *p, size_t bytes, void *stream) {
    if (bytes == 0) return WARPCTCT_OK;
    if (!p) return WARPCTCT_EINVAL;
    return done(launch_zero_fill_bytes(p, bytes, as_stream(stream)));
}

int warpctct_loss_forward(const void *joint, int dtype, const int *ys, const int *lx,
                          const int *ly, int N, int T, int U, int V, void *workspace,
                          size_t workspace_bytes, float *costs, float *unit_grads, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || !io_valid(dtype)) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !costs || !workspace || (T > 0 && !joint) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    const Workspace w = carve(workspace, N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    if (T > 0) {
        int rc = done(launch_gather_units(joint, dense_joint_strides(T, U, V), dtype, ys, lx, ly,
                                          w.units, N, T, U, V, true, nullptr, RelaySlots{},
                                          as_stream(stream)));
        if (rc != WARPCTCT_OK) return rc;
    }
    return forward_from_units(w, ys, lx, ly, N, T, U, costs, T > 0 ? unit_grads : nullptr,
                              as_stream(stream));
}

int warpctct_loss_forward_static(const void *joint, int dtype, const int *ys, const int *lx,
                                 const int *ly, int N, int T, int U, int V, float *costs,
                                 float *unit_grads, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || !io_valid(dtype)) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !costs || (T > 0 && !joint) || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    if (carve(nullptr, N, T, U).bytes > (size_t)WARPCTCT_STATIC_SCRATCH_BYTES)
        return WARPCTCT_ETOOLARGE;
    void *base = nullptr;
    const int rc = static_scratch(&base);
    if (rc != WARPCTCT_OK) return rc;
    // Every cell of the array that a kernel reads has been written earlier in
    // the same call (units by the gather, alpha / beta by the lattice sweep),
    // so what an earlier call left behind is never seen and nothing needs
    // clearing; the arrival counter of the batch reduction is not used here.
    return warpctct_loss_forward(joint, dtype, ys, lx, ly, N, T, U, V, base,
                                 (size_t)WARPCTCT_STATIC_SCRATCH_BYTES, costs, unit_grads, stream);
}

int warpctct_loss_forward_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              int N, int T, int U, int V, void *workspace, size_t workspace_bytes,
                              float *costs, float *unit_grads, void *stream) {
    return warpctct_loss_forward(joint, WARPCTCT_F32, ys, lx, ly, N, T, U, V, workspace,
                                 workspace_bytes, costs, unit_grads, stream);
}

int warpctct_loss_forward_units_f32(const float *units_nat, const int *ys, const int *lx,
                                    const int *ly, int N, int T, int U, void *workspace,
                                    size_t workspace_bytes, float *costs, float *unit_grads,
                                    void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !costs || !workspace || (T > 0 && !units_nat) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    const Workspace w = carve(workspace, N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    if (T > 0) {
        int rc = done(launch_scale_units(units_nat, lx, ly, w.units, N, T, U, as_stream(stream)));
        if (rc != WARPCTCT_OK) return rc;
    }
    return forward_from_units(w, ys, lx, ly, N, T, U, costs, T > 0 ? unit_grads : nullptr,
                              as_stream(stream));
}

int warpctct_simple_gather_units_f32(const float *f, const float *g, const float *den,
                                     const int *ys, const int *lx, const int *ly,
                                     double *units_out, int N, int T, int U, int V, void *stream) {
    if (!dims_ok(N, T, U) || V < 1) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!f || !g || !lx || !ly || !units_out || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    return done(launch_simple_gather_units(f, g, const_cast<float *>(den), ys, lx, ly, units_out, N,
                                           T, U, V, RelaySlots{}, LogmmDeferred{}, nullptr, nullptr,
                                           as_stream(stream)));
}

int warpctct_simple_reduce_f32(const float *unit_grads, float *grad_f, float *grad_g,
                               float *grad_den, int N, int T, int U, void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!grad_g || (T > 0 && (!unit_grads || !grad_f))) return WARPCTCT_EINVAL;
    return done(launch_simple_reduce(unit_grads, grad_f, grad_g, grad_den, N, T, U,
                                     as_stream(stream)));
}

int warpctct_simple_scatter_f32(const float *grad_f, const float *grad_g, const int *ys,
                                const int *lx, const int *ly, const float *grad_out,
                                float *dense_f, float *dense_g, int N, int T, int U, int V,
                                void *stream) {
    if (!dims_ok(N, T, U) || V < 1) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || (U > 0 && !ys) || (dense_f && !grad_f) || (dense_g && !grad_g))
        return WARPCTCT_EINVAL;
    return done(launch_simple_scatter(grad_f, grad_g, ys, lx, ly, grad_out, T > 0 ? dense_f : nullptr,
                                      dense_g, N, T, U, V, as_stream(stream)));
}

int warpctct_zero_fill_f32(float *p, size_t n, void *stream) {
    if (n == 0) return WARPCTCT_OK;
    if (!p) return WARPCTCT_EINVAL;
    return done(launch_zero_fill(p, n, as_stream(stream)));
}

size_t warpctct_simple_workspace_bytes(int N, int T, int U) {
    if (N < 0 || T < 0 || U < 0) return 0;
    return carve_simple(nullptr, N, T, U).bytes;
}

int warpctct_simple_needs_fexp(const float *f, int T, int U, int V) {
    if (T < 0 || U < 0 || V < 1) return 1;
    const LogmmOperand lhs = {f, (long)T * V, (long)V, 1L};
    return logmm_reads_lhs_itself(lhs, T, V, U + 1) ? 0 : 1;
}

int warpctct_simple_forward_f32(const float *f, const float *g, const int *ys, const int *lx,
                                const int *ly, int N, int T, int U, int V, int normalized,
                                void *workspace, size_t workspace_bytes, float *den, float *fmax,
                                float *gmax, float *fexp, float *gexp, float *costs,
                                float *grad_f, float *grad_g, float *grad_den, void *stream) {
    return warpctct_simple_forward_reduced_f32(f, g, ys, lx, ly, N, T, U, V, normalized, workspace,
                                               workspace_bytes, den, fmax, gmax, fexp, gexp, costs,
                                               grad_f, grad_g, grad_den, 0, 0, nullptr, stream);
}

int warpctct_simple_forward_reduced_f32(const float *f, const float *g, const int *ys,
                                        const int *lx, const int *ly, int N, int T, int U, int V,
                                        int normalized, void *workspace, size_t workspace_bytes,
                                        float *den, float *fmax, float *gmax, float *fexp,
                                        float *gexp, float *costs, float *grad_f, float *grad_g,
                                        float *grad_den, int reduction, int average_frames,
                                        float *reduced, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || reduction < 0 || reduction > 2) return WARPCTCT_EINVAL;
    if (reduction != 0 && !reduced) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    const bool want_grad = grad_f || grad_g || grad_den;
    if (!g || !lx || !ly || !costs || !workspace || (T > 0 && !f) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    // (without frames the gradients of f and den have no elements, and no address)
    if (want_grad && (!grad_g || (T > 0 && (!grad_f || (normalized && !grad_den)))))
        return WARPCTCT_EINVAL;
    // where the log-matmul kernels read f itself, exp(f - fmax) is not stored
    const bool keeps_fexp = warpctct_simple_needs_fexp(f, T, U, V) != 0;
    if (normalized && T > 0 && (!den || !fmax || !gmax || !gexp || (keeps_fexp && !fexp)))
        return WARPCTCT_EINVAL;
    const SimpleWorkspace w = carve_simple(workspace, N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    // the batch reduction rides in the lattice kernel; its arrival counter is
    // cleared by the gather (or, without frames, by a launch of its own)
    CostReduce reduce = {};
    reduce.reduced = reduction != 0 ? reduced : nullptr;
    reduce.counter = reduction != 0 ? w.lattice.counter : nullptr;
    reduce.mode = reduction;
    reduce.average_frames = average_frames != 0;
    if (T == 0 && reduce.counter) {
        int rc = done(launch_clear_counter(reduce.counter, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    if (T > 0) {
        LogmmDeferred deferred = {};
        if (normalized) {
            // den[n,t,u] = logsumexp_v(f[n,t,v] + g[n,u,v]):  lhs = f, rhs[b,k,j] = g[b,j,k]
            const LogmmOperand lhs = {f, (long)T * V, (long)V, 1L};
            const LogmmOperand rhs = {g, (long)(U + 1) * V, 1L, (long)V};
            const LogmmShifted sh = {fmax, gmax, keeps_fexp ? fexp : nullptr, gexp};
            int rc = done(launch_logmm_shift_exp(lhs, rhs, sh, N, T, V, U + 1, lx, ly, st));
            if (rc != WARPCTCT_OK) return rc;
            // (its last pass, where it is a pass of its own, is left to the gather)
            rc = done(launch_logmm_fwd(lhs, rhs, sh, den, w.partial, N, T, V, U + 1, lx, ly,
                                       &deferred, st));
            if (rc != WARPCTCT_OK) return rc;
        }
        int linear_from = g_linear_from.load(std::memory_order_relaxed);
        bool batch_fits = true;   // a limit that the caller has set holds for every batch
        if (linear_from < 0) {
            linear_from = normalized ? kLinearFromFramesNormalized : kLinearFromFrames;
            batch_fits = linear_batch_fits(N, U);
        }
        if (want_grad && linear_from > 0 && T >= linear_from && batch_fits && simple_grads_lin_applies(T, U)) {
            // The lattices in the linear domain (less than half the time per frame),
            // checked by the kernel that forms the gradients from them; the
            // log-domain kernels follow and return at once unless that check, or
            // anything else on the way, has raised the flag.
            CostReduce lin_reduce = reduce;
            if (lin_reduce.counter) lin_reduce.counter = w.lin_counter;
            int rc = done(launch_simple_gather_units_lin(f, g, normalized ? den : nullptr, ys, lx, ly,
                                                         w.lin_units, N, T, U, V, deferred, fmax,
                                                         lin_reduce.counter, w.lin_flag, st));
            if (rc != WARPCTCT_OK) return rc;
            LatticeArgs a = {};
            a.units = w.lin_units;
            a.ys = ys, a.lx = lx, a.ly = ly;
            a.alphas = w.lin_alphas, a.betas = w.lin_betas;
            a.costs = costs;
            a.N = N, a.T = T, a.U = U;
            a.reduce = lin_reduce;
            rc = done(launch_lattice_lin(a, w.lin_scales, w.lin_flag, st));
            if (rc != WARPCTCT_OK) return rc;
            rc = done(launch_simple_grads_lin(w.lin_units, ys, lx, ly, w.lin_alphas, w.lin_betas,
                                              w.lin_scales, w.unit_grads, grad_f,
                                              normalized ? grad_den : nullptr, N, T, U, w.lin_flag, st));
            if (rc != WARPCTCT_OK) return rc;
            const unsigned *guard = w.lin_flag;
            rc = done(launch_simple_gather_units(f, g, normalized ? den : nullptr, ys, lx, ly,
                                                 w.lattice.units, N, T, U, V,
                                                 relay_slots_of(w.lattice.relay, N, T, U), deferred,
                                                 fmax, reduce.counter, st, guard));
            if (rc != WARPCTCT_OK) return rc;
            return simple_from_units(w, ys, lx, ly, N, T, U, costs, grad_f, grad_g,
                                     normalized ? grad_den : nullptr, true, true, reduce, st,
                                     guard);
        }
        int rc = done(launch_simple_gather_units(f, g, normalized ? den : nullptr, ys, lx, ly,
                                                 w.lattice.units, N, T, U, V,
                                                 relay_slots_of(w.lattice.relay, N, T, U), deferred,
                                                 fmax, reduce.counter, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    if (want_grad && T == 0) {   // no frames: the only gradient with elements is all zeros
        int rc = done(launch_zero_fill(grad_g, (size_t)N * (U + 1) * 3, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    return simple_from_units(w, ys, lx, ly, N, T, U, costs, grad_f, grad_g,
                             normalized ? grad_den : nullptr, want_grad && T > 0, T > 0, reduce,
                             st);
}

int warpctct_simple_forward_units_f32(const float *f_g, const float *g_g, const float *den,
                                      const int *ys, const int *lx, const int *ly, int N, int T,
                                      int U, void *workspace, size_t workspace_bytes, float *costs,
                                      float *grad_f, float *grad_g, float *grad_den, void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    const bool want_grad = grad_f || grad_g || grad_den;
    if (!g_g || !lx || !ly || !costs || !workspace || (T > 0 && !f_g) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    if (want_grad && (!grad_g || (T > 0 && (!grad_f || (den && !grad_den)))))
        return WARPCTCT_EINVAL;
    const SimpleWorkspace w = carve_simple(workspace, N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    if (T > 0) {
        int rc = done(launch_simple_units(f_g, g_g, den, lx, ly, w.lattice.units, N, T, U, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    if (want_grad && T == 0) {
        int rc = done(launch_zero_fill(grad_g, (size_t)N * (U + 1) * 3, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    return simple_from_units(w, ys, lx, ly, N, T, U, costs, grad_f, grad_g,
                             den ? grad_den : nullptr, want_grad && T > 0, false, CostReduce{}, st);
}

size_t warpctct_simple_backward_workspace_bytes(int N, int T, int U) {
    if (N < 0 || T < 0 || U < 0) return 0;
    return carve_pairs(nullptr, N, T, U + 1).bytes;
}

int warpctct_simple_backward_f32(const float *f, const float *g, const float *den,
                                 const float *fmax, const float *gmax, const float *fexp,
                                 const float *gexp, const float *grad_f,
                                 const float *grad_g, const float *grad_den,
                                 const int *ys, const int *lx, const int *ly,
                                 const float *grad_out, int N, int T, int U, int V,
                                 void *workspace, size_t workspace_bytes, float *dense_f,
                                 float *dense_g, void *stream) {
    return warpctct_simple_backward_weighted_f32(f, g, den, fmax, gmax, fexp, gexp, grad_f, grad_g,
                                                 grad_den, ys, lx, ly, grad_out, 1, 1.0f, 0,
                                                 nullptr, N, T, U, V, workspace, workspace_bytes,
                                                 dense_f, dense_g, stream);
}

int warpctct_simple_backward_weighted_f32(const float *f, const float *g, const float *den,
                                          const float *fmax, const float *gmax, const float *fexp,
                                          const float *gexp, const float *grad_f,
                                          const float *grad_g, const float *grad_den,
                                          const int *ys, const int *lx, const int *ly,
                                          const float *grad_out, int grad_out_stride, float scale,
                                          int average_frames, float *weights, int N, int T, int U,
                                          int V, void *workspace, size_t workspace_bytes,
                                          float *dense_f, float *dense_g, void *stream) {
    if (!dims_ok(N, T, U) || V < 1 || (grad_out_stride != 0 && grad_out_stride != 1))
        return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || (U > 0 && !ys) || (dense_f && !grad_f) || (dense_g && !grad_g))
        return WARPCTCT_EINVAL;
    const Weight weight = {grad_out, grad_out_stride, scale, average_frames != 0};
    // grad_out as it is serves as the array of per-sample weights
    const bool plain = scale == 1.0f && !average_frames && (!grad_out || grad_out_stride == 1);
    const bool keeps_fexp = warpctct_simple_needs_fexp(f, T, U, V) != 0;
    if (den && (!f || !g || !grad_den || !fmax || !gmax || !gexp || !workspace ||
                (keeps_fexp && !fexp)))
        return WARPCTCT_EINVAL;
    if (den && workspace_bytes < warpctct_simple_backward_workspace_bytes(N, T, U))
        return WARPCTCT_EWORKSPACE;
    hipStream_t st = as_stream(stream);
    const int U1 = U + 1;
    if (T == 0) dense_f = nullptr;
    if (!den && simple_dense_rows_fit(V))
        // whole rows of both gradients built and written once, instead of
        // zero-fill + atomic adds
        return done(launch_simple_dense_rows(grad_f, grad_g, ys, lx, ly, weight, dense_f, dense_g,
                                             N, T, U, V, st));
    // the other kernels read an array of N weights: the first kernel of the
    // normalised path leaves it behind, otherwise a launch of its own does
    if (!plain && !weights) return WARPCTCT_EINVAL;
    if (!plain && !(den && T > 0)) {
        int rc = done(launch_sample_weights(weight, lx, weights, N, st));
        if (rc != WARPCTCT_OK) return rc;
        grad_out = weights;
    }
    if (den) {
        const LogmmOperand lhs = {f, (long)T * V, (long)V, 1L};
        const LogmmOperand rhs = {g, (long)U1 * V, 1L, (long)V};
        const PairWorkspace pw = carve_pairs(workspace, N, T, U1);
        const LogmmShifted sh = {const_cast<float *>(fmax), const_cast<float *>(gmax),
                                 keeps_fexp ? const_cast<float *>(fexp) : nullptr,
                                 const_cast<float *>(gexp)};
        if (T > 0) {
            int rc = done(launch_logmm_pair_factor(grad_den, den, fmax, gmax, weight,
                                                   plain ? nullptr : weights, lx, ly, pw.factors,
                                                   pw.flags, pw.planes, N, T, U1, st));
            if (rc != WARPCTCT_OK) return rc;
        }
        if (!plain) grad_out = weights;
        // (the gradient wrt g first: it only reads f, which the gradient wrt f then
        // finds in the memory-side cache, and whose own 4*N*T*V bytes of output are
        // still there for the scatter that follows)
        if (dense_g) {
            // gradient of rhs[b,k,j] = g[b,j,k] stored straight into the (N,U+1,V) layout
            const LogmmGrad gr = {dense_g, (long)U1 * V, 1L, (long)V};
            int rc = done(launch_logmm_bwd_rhs(lhs, rhs, sh, grad_den, den, pw.factors, pw.flags,
                                               pw.planes,
                                               gr, N, T, V, U1, lx, ly, grad_out, st));
            if (rc != WARPCTCT_OK) return rc;
        }
        if (dense_f) {
            const LogmmGrad gl = {dense_f, (long)T * V, (long)V, 1L};
            int rc = done(launch_logmm_bwd_lhs(lhs, rhs, sh, grad_den, den, pw.factors, pw.flags,
                                               gl, N, T, V, U1, lx, ly, grad_out, st));
            if (rc != WARPCTCT_OK) return rc;
        }
    } else {
        if (dense_f) {
            int rc = done(launch_zero_fill(dense_f, (size_t)N * T * V, st));
            if (rc != WARPCTCT_OK) return rc;
        }
        if (dense_g) {
            int rc = done(launch_zero_fill(dense_g, (size_t)N * U1 * V, st));
            if (rc != WARPCTCT_OK) return rc;
        }
    }
    return done(launch_simple_scatter(grad_f, grad_g, ys, lx, ly, grad_out, dense_f, dense_g, N, T,
                                      U, V, st));
}

int warpctct_logmm_padded_reduction(int K) { return K < 0 ? 0 : logmm_padded_reduction(K); }

size_t warpctct_logmm_workspace_bytes(int B, int M, int K, int Nn) {
    if (B < 0 || M < 0 || K < 0 || Nn < 0) return 0;
    return carve_logmm(nullptr, B, M, K, Nn).bytes;
}

int warpctct_logmm_fwd_f32(const float *lhs, long lsb, long lsm, long lsk, const float *rhs,
                           long rsb, long rsk, long rsn, int B, int M, int K, int Nn,
                           void *workspace, size_t workspace_bytes, float *res, void *stream) {
    if (B < 0 || M < 0 || K < 0 || Nn < 0 || B > kMaxGrid || Nn > kMaxGrid * 32)
        return WARPCTCT_EINVAL;
    if (B == 0 || M == 0 || Nn == 0) return WARPCTCT_OK;
    if (!res || !workspace || (K > 0 && (!lhs || !rhs))) return WARPCTCT_EINVAL;
    const LogmmWorkspace w = carve_logmm(workspace, B, M, K, Nn);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    const LogmmOperand l = {lhs, lsb, lsm, lsk};
    const LogmmOperand r = {rhs, rsb, rsk, rsn};
    int rc = done(launch_logmm_shift_exp(l, r, w.sh, B, M, K, Nn, nullptr, nullptr,
                                         as_stream(stream)));
    if (rc != WARPCTCT_OK) return rc;
    return done(launch_logmm_fwd(l, r, w.sh, res, w.partial, B, M, K, Nn, nullptr, nullptr,
                                 nullptr, as_stream(stream)));
}

int warpctct_logmm_bwd_f32(const float *grad_out, const float *lhs, long lsb, long lsm, long lsk,
                           const float *rhs, long rsb, long rsk, long rsn, const float *res, int B,
                           int M, int K, int Nn, void *workspace, size_t workspace_bytes,
                           float *grad_lhs, long glsb, long glsm, long glsk, float *grad_rhs,
                           long grsb, long grsk, long grsn, void *stream) {
    if (B < 0 || M < 0 || K < 0 || Nn < 0 || B > kMaxGrid || K > kMaxGrid * 64)
        return WARPCTCT_EINVAL;
    if (B == 0 || K == 0) return WARPCTCT_OK;
    if (!workspace || (M > 0 && !lhs) || (Nn > 0 && !rhs) ||
        ((M > 0 && Nn > 0) && (!grad_out || !res)))
        return WARPCTCT_EINVAL;
    const LogmmWorkspace w = carve_logmm(workspace, B, M, K, Nn);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    const LogmmOperand l = {lhs, lsb, lsm, lsk};
    const LogmmOperand r = {rhs, rsb, rsk, rsn};
    hipStream_t st = as_stream(stream);
    {
        int rc = done(launch_logmm_shift_exp(l, r, w.sh, B, M, K, Nn, nullptr, nullptr, st));
        if (rc != WARPCTCT_OK) return rc;
        rc = done(launch_logmm_pair_factor(grad_out, res, w.sh.lmax, w.sh.rmax,
                                           Weight{nullptr, 1, 1.0f, 0}, nullptr, nullptr,
                                           nullptr, w.pw.factors, w.pw.flags, w.pw.planes, B, M, Nn, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    if (grad_lhs) {
        const LogmmGrad g = {grad_lhs, glsb, glsm, glsk};
        int rc = done(launch_logmm_bwd_lhs(l, r, w.sh, grad_out, res, w.pw.factors, w.pw.flags, g,
                                           B, M, K, Nn, nullptr, nullptr, nullptr, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    if (grad_rhs) {
        const LogmmGrad g = {grad_rhs, grsb, grsk, grsn};
        int rc = done(launch_logmm_bwd_rhs(l, r, w.sh, grad_out, res, w.pw.factors, w.pw.flags,
                                           w.pw.planes, g,
                                           B, M, K, Nn, nullptr, nullptr, nullptr, st));
        if (rc != WARPCTCT_OK) return rc;
    }
    return WARPCTCT_OK;
}

}  // extern "C"
