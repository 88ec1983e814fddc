// extern "C" surface of libwarpctct_hip.so (declared in include/warp_ctct_hip.h).
// Host code only: argument validation, workspace carving, kernel launches.
// No allocation, no host synchronisation, no process exit.
#include "warp_ctct_hip.h"

#include <hip/hip_runtime.h>

#include "launch.h"

namespace {

using namespace wctct;

constexpr int kMaxGrid = 65535;

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline int done(hipError_t e) { return e == hipSuccess ? WARPCTCT_OK : WARPCTCT_ELAUNCH; }

inline bool dims_ok(int N, int T, int U) {
    return N >= 0 && T >= 0 && U >= 0 && N <= kMaxGrid && T <= kMaxGrid &&
           (U + 1) <= lattice_max_contexts() && (long)T * (U + 1) < (1L << 31);
}

inline size_t align256(size_t x) { return (x + 255) & ~(size_t)255; }

struct Workspace {
    double *units;    // (N,T,U+1,3)
    double *alphas;   // (N,T+1,U+1,2)
    double *betas;    // (N,T+1,U+1,2)
    size_t bytes;
};

Workspace carve(void *base, int N, int T, int U) {
    const size_t units_b = align256((size_t)N * T * (U + 1) * 3 * sizeof(double));
    const size_t lat_b = align256((size_t)N * (T + 1) * (U + 1) * 2 * sizeof(double));
    const uintptr_t p = reinterpret_cast<uintptr_t>(base);
    Workspace w;
    w.units = reinterpret_cast<double *>(p);
    w.alphas = reinterpret_cast<double *>(p + units_b);
    w.betas = reinterpret_cast<double *>(p + units_b + lat_b);
    w.bytes = units_b + 2 * lat_b;
    return w;
}

int forward_from_units(const Workspace &w, const int *ys, const int *lx, const int *ly, int N,
                       int T, int U, float *costs, float *unit_grads, hipStream_t stream) {
    LatticeArgs a;
    a.units = w.units;
    a.ys = ys;
    a.lx = lx;
    a.ly = ly;
    a.alphas = w.alphas;
    a.betas = w.betas;
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

}  // namespace

extern "C" {

const char *warpctct_error_string(int code) {
    switch (code) {
        case WARPCTCT_OK: return "ok";
        case WARPCTCT_EINVAL:
            return "invalid argument (null pointer, negative size, or size limit: N,T <= 65535, "
                   "U+1 <= 512)";
        case WARPCTCT_ELAUNCH: return "kernel launch failed";
        case WARPCTCT_EWORKSPACE: return "workspace too small";
        case WARPCTCT_ENODEVICE: return "no usable HIP device";
        default: return "unknown error";
    }
}

const char *warpctct_version(void) { return "0.1.0"; }

size_t warpctct_workspace_bytes(int N, int T, int U) {
    if (N < 0 || T < 0 || U < 0) return 0;
    return carve(nullptr, N, T, U).bytes;
}

int warpctct_gather_units_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              double *units_out, int N, int T, int U, int V, void *stream) {
    if (!dims_ok(N, T, U) || V < 1) return WARPCTCT_EINVAL;
    if (N == 0 || T == 0) return WARPCTCT_OK;
    if (!joint || !lx || !ly || !units_out || (U > 0 && !ys)) return WARPCTCT_EINVAL;
    return done(launch_gather_units(joint, ys, lx, ly, units_out, N, T, U, V, as_stream(stream)));
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

int warpctct_lattice_f32(const double *units, const int *ys, const int *lx, const int *ly,
                         double *alphas, double *betas, float *costs, int N, int T, int U,
                         int beta_only, void *stream) {
    if (!dims_ok(N, T, U)) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !betas || !costs || (T > 0 && !units) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    if (!beta_only && !alphas) return WARPCTCT_EINVAL;
    LatticeArgs a;
    a.units = units;
    a.ys = ys;
    a.lx = lx;
    a.ly = ly;
    a.alphas = alphas;
    a.betas = betas;
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

int warpctct_loss_forward_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              int N, int T, int U, int V, void *workspace, size_t workspace_bytes,
                              float *costs, float *unit_grads, void *stream) {
    if (!dims_ok(N, T, U) || V < 1) return WARPCTCT_EINVAL;
    if (N == 0) return WARPCTCT_OK;
    if (!lx || !ly || !costs || !workspace || (T > 0 && !joint) || (U > 0 && !ys))
        return WARPCTCT_EINVAL;
    const Workspace w = carve(workspace, N, T, U);
    if (workspace_bytes < w.bytes) return WARPCTCT_EWORKSPACE;
    if (T > 0) {
        int rc = done(launch_gather_units(joint, ys, lx, ly, w.units, N, T, U, V,
                                          as_stream(stream)));
        if (rc != WARPCTCT_OK) return rc;
    }
    return forward_from_units(w, ys, lx, ly, N, T, U, costs, T > 0 ? unit_grads : nullptr,
                              as_stream(stream));
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

}  // extern "C"
