// Per-cell "units" of the CTC-Transducer lattice and their gradients.
//
// A unit is one of the three log-probabilities a cell (t,u) contributes:
//   k=0 blank, k=1 label y[u-1] ("current"), k=2 label y[u] ("next")
// (csrc/gather.cu:16-21 of the reference).  The kernels here
//   * pull the units out of the (N,T,U+1,V) joint tensor (replaces the index
//     build + torch.gather of warp_ctct/__init__.py:124-131),
//   * or form them from the log-add joiner operands f, g, den (replaces the
//     LOGPROBY/LOGPROBB macros of csrc/simple.cu:20-26, simple_unnorm.cu:20-25),
//   * and turn alpha/beta into d(cost)/d(unit) (replaces k_fill_grad,
//     csrc/gather.cu:311-374).
// Units are stored as doubles scaled to log2, the lattice's working format
// (v_exp_f32 / v_log_f32 are base 2, and the lattice sums in double), in a
// buffer of P = padded_contexts(U) contexts per frame.  One thread per cell;
// cells of padding (t >= lx[n] or u > ly[n]) are never read from the inputs.
// For t < lx[n] the padding contexts u > ly[n] get the neutral units
// {0, 0, -inf}, and "next" is -inf at u = ly[n]: no mass can flow there.
#include "device_utils.h"
#include "launch.h"
#include "unit_grad.h"

namespace wctct {

namespace {

constexpr int kCellBlock = 256;

struct Cell {
    int n, t, u, Tn, Un;
    bool in_range, live;
};

// Cell of a (T x W) grid of sample blockIdx.y, W = U+1 (tensors of the
// interface) or W = P (work buffers).
__device__ __forceinline__ Cell locate_cell(const int *lx, const int *ly, int T, int U, int W) {
    Cell c;
    c.n = blockIdx.y;
    const int cell = blockIdx.x * kCellBlock + threadIdx.x;
    c.in_range = cell < T * W;
    c.t = cell / W;
    c.u = cell - c.t * W;
    c.Tn = min(max(lx[c.n], 0), T);
    c.Un = min(max(ly[c.n], 0), U);
    c.live = c.in_range && c.t < c.Tn && c.u <= c.Un;
    return c;
}

// The gather's scattered reads of the joint, non-temporal: every one of them
// pulls in a line of which 4 bytes are used and nothing is used again; left out
// of the caches the kernel takes 27 us instead of 43 us (typical batch).
__device__ __forceinline__ float nt_load(const float *p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ float nt_load(const __half *p) {
    return (float)__builtin_nontemporal_load(reinterpret_cast<const _Float16 *>(p));
}
__device__ __forceinline__ float nt_load(const __hip_bfloat16 *p) {
    const unsigned short b = __builtin_nontemporal_load(reinterpret_cast<const unsigned short *>(p));
    return __uint_as_float((unsigned)b << 16);
}

// b, cur, nxt in natural-log units; nxt is only meaningful for u < Un.
__device__ __forceinline__ void store_units(double *units, const Cell &c, int T, int P, double b,
                                            double cur, double nxt) {
    double *o = units + (((size_t)c.n * T + c.t) * P + c.u) * 3;
    o[0] = b * kLog2e;
    o[1] = cur * kLog2e;
    o[2] = (c.u < c.Un) ? nxt * kLog2e : neg_inf();
}

// Padding context of a live frame: neutral units.  Returns true if handled.
__device__ __forceinline__ bool store_padding(double *units, const Cell &c, int T, int P) {
    if (c.live) return false;
    if (c.in_range && c.t < c.Tn) {
        double *o = units + (((size_t)c.n * T + c.t) * P + c.u) * 3;
        o[0] = 0.0;
        o[1] = 0.0;
        o[2] = neg_inf();
    }
    return true;
}

// BAND_ONLY: cells that no complete alignment can pass through (see
// outside_band in unit_grad.h) get neutral units instead of a gather.  Costs
// and gradients do not change: such a cell is entered with alpha = -inf or
// left towards beta = -inf whatever its units are; only the alpha / beta values
// of dead cells themselves differ from a full gather's.
// counter (may be null) is cleared for the cost reduction of the lattice
// kernel that follows on the same stream.
template <bool BAND_ONLY, typename IO>
__global__ __launch_bounds__(kCellBlock) void gather_units_kernel(
    const IO *__restrict__ joint, const JointStrides js, const int *__restrict__ ys,
    const int *__restrict__ lx, const int *__restrict__ ly, double *__restrict__ units, int T,
    int U, int V, int P, unsigned *__restrict__ counter, const RelaySlots relay,
    unsigned *__restrict__ status) {
    if (counter && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *counter = 0u;
    relay_clear_share(relay);
    Cell c = locate_cell(lx, ly, T, U, P);
    if (BAND_ONLY && c.live && outside_band(c.t, c.u, c.Tn, c.Un)) c.live = false;
    if (store_padding(units, c, T, P)) return;
    const IO *row = joint + (long)c.n * js.n + (long)c.t * js.t + (long)c.u * js.u;
    const int *y = ys + (size_t)c.n * U;
    const float b = nt_load(row);
    float cur = b, nxt = b;   // the reference gathers index 0 where no label exists
    // labels are clamped into [0,V) so that a corrupt label cannot fault
    if (c.u >= 1) cur = nt_load(row + (long)label_column(y[c.u - 1], V, status) * js.v);
    if (c.u < c.Un) nxt = nt_load(row + (long)label_column(y[c.u], V, status) * js.v);
    store_units(units, c, T, P, unit_or_log_zero(b, status), unit_or_log_zero(cur, status),
                unit_or_log_zero(nxt, status));
}

__global__ __launch_bounds__(kCellBlock) void scale_units_kernel(
    const float *__restrict__ units_nat, const int *__restrict__ lx, const int *__restrict__ ly,
    double *__restrict__ units, int T, int U, int P) {
    const Cell c = locate_cell(lx, ly, T, U, P);
    if (store_padding(units, c, T, P)) return;
    const float *i = units_nat + (((size_t)c.n * T + c.t) * (U + 1) + c.u) * 3;
    store_units(units, c, T, P, i[0], i[1], i[2]);
}

// LP(t,u,0) = f_g[t,0]   + g_g[u,0] - den[t,u]
// LP(t,u,k) = f_g[t,u+k-1] + g_g[u,k] - den[t,u],  k = 1 (u >= 1), 2 (u < U)
__global__ __launch_bounds__(kCellBlock) void simple_units_kernel(
    const float *__restrict__ f_g, const float *__restrict__ g_g, const float *__restrict__ den,
    const int *__restrict__ lx, const int *__restrict__ ly, double *__restrict__ units, int T,
    int U, int P) {
    const Cell c = locate_cell(lx, ly, T, U, P);
    if (store_padding(units, c, T, P)) return;
    const int U1 = U + 1;
    const float *fr = f_g + ((size_t)c.n * T + c.t) * U1;
    const float *gr = g_g + ((size_t)c.n * U1 + c.u) * 3;
    const double d = den ? (double)den[((size_t)c.n * T + c.t) * U1 + c.u] : 0.0;
    const double b = (double)fr[0] + (double)gr[0] - d;
    const double cur = (c.u >= 1) ? (double)fr[c.u] + (double)gr[1] - d : b;
    const double nxt = (c.u < c.Un) ? (double)fr[c.u + 1] + (double)gr[2] - d : b;
    store_units(units, c, T, P, b, cur, nxt);
}

// One thread per cell of the (N,T,U+1,3) unit-gradient tensor; zeros in padding.
__global__ __launch_bounds__(kCellBlock) void unit_grads_kernel(
    const double *__restrict__ units, const int *__restrict__ ys, const int *__restrict__ lx,
    const int *__restrict__ ly, const double *__restrict__ alphas,
    const double *__restrict__ betas, float *__restrict__ unit_grads, int T, int U, int P) {
    const Cell c = locate_cell(lx, ly, T, U, U + 1);
    if (!c.in_range) return;
    float *go = unit_grads + (((size_t)c.n * T + c.t) * (U + 1) + c.u) * 3;
    UnitGrad g = {0.0f, 0.0f, 0.0f};
    // outside the band of complete alignments the gradient is exactly zero
    if (c.live && !outside_band(c.t, c.u, c.Tn, c.Un)) {
        const size_t lat = (size_t)(T + 1) * P * 2;
        g = unit_grad_cell(units + (size_t)c.n * T * P * 3, alphas + (size_t)c.n * lat,
                           betas + (size_t)c.n * lat, ys + (size_t)c.n * U, c.t, c.u, c.Un, P);
    }
    go[0] = g.g0;
    go[1] = g.g1;
    go[2] = g.g2;
}

inline dim3 cell_grid(int N, int T, int W) {
    const long cells = (long)T * W;
    return dim3((unsigned)((cells + kCellBlock - 1) / kCellBlock), (unsigned)N);
}

}  // namespace

namespace {

__global__ void clear_counter_kernel(unsigned *counter) { *counter = 0u; }

template <typename IO>
void launch_gather_typed(const void *joint, const JointStrides &js, const int *ys, const int *lx,
                         const int *ly, double *units, int N, int T, int U, int V, bool band_only,
                         unsigned *counter, const RelaySlots &relay, hipStream_t stream) {
    const int P = padded_contexts(U);
    const IO *j = static_cast<const IO *>(joint);
    unsigned *status = device_status_word();
    if (band_only) {
        TIMED_LAUNCH((gather_units_kernel<true, IO>), cell_grid(N, T, P), dim3(kCellBlock),
                           0, stream, j, js, ys, lx, ly, units, T, U, V, P, counter, relay, status);
    } else {
        TIMED_LAUNCH((gather_units_kernel<false, IO>), cell_grid(N, T, P), dim3(kCellBlock),
                           0, stream, j, js, ys, lx, ly, units, T, U, V, P, counter, relay, status);
    }
}

}  // namespace

hipError_t launch_gather_units(const void *joint, const JointStrides &js, int io_type,
                               const int *ys, const int *lx, const int *ly, double *units, int N,
                               int T, int U, int V, bool band_only, unsigned *counter,
                               const RelaySlots &relay, hipStream_t stream) {
    switch (io_type) {
        case kIoF32:
            launch_gather_typed<float>(joint, js, ys, lx, ly, units, N, T, U, V, band_only, counter, relay, stream);
            break;
        case kIoF16:
            launch_gather_typed<__half>(joint, js, ys, lx, ly, units, N, T, U, V, band_only, counter, relay, stream);
            break;
        case kIoBF16:
            launch_gather_typed<__hip_bfloat16>(joint, js, ys, lx, ly, units, N, T, U, V,
                                                band_only, counter, relay, stream);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_clear_counter(unsigned *counter, hipStream_t stream) {
    TIMED_LAUNCH(clear_counter_kernel, dim3(1), dim3(1), 0, stream, counter);
    return hipGetLastError();
}

hipError_t launch_scale_units(const float *units_nat, const int *lx, const int *ly, double *units,
                              int N, int T, int U, hipStream_t stream) {
    const int P = padded_contexts(U);
    TIMED_LAUNCH(scale_units_kernel, cell_grid(N, T, P), dim3(kCellBlock), 0, stream,
                       units_nat, lx, ly, units, T, U, P);
    return hipGetLastError();
}

hipError_t launch_simple_units(const float *f_g, const float *g_g, const float *den,
                               const int *lx, const int *ly, double *units, int N, int T, int U,
                               hipStream_t stream) {
    const int P = padded_contexts(U);
    TIMED_LAUNCH(simple_units_kernel, cell_grid(N, T, P), dim3(kCellBlock), 0, stream, f_g,
                       g_g, den, lx, ly, units, T, U, P);
    return hipGetLastError();
}

hipError_t launch_unit_grads(const double *units, const int *ys, const int *lx, const int *ly,
                             const double *alphas, const double *betas, float *unit_grads, int N,
                             int T, int U, hipStream_t stream) {
    TIMED_LAUNCH(unit_grads_kernel, cell_grid(N, T, U + 1), dim3(kCellBlock), 0, stream,
                       units, ys, lx, ly, alphas, betas, unit_grads, T, U, padded_contexts(U));
    return hipGetLastError();
}

}  // namespace wctct
