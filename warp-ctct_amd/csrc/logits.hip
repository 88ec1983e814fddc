// ctct_loss on un-normalised joiner outputs ("logits"): log_softmax over the
// vocabulary is taken inside the gather, and its backward inside the kernel
// that writes the dense gradient, so the (N,T,U+1,V) log-probability tensor
// that a caller of the reference has to materialise before
// warp_ctct.ctct_loss (and whose gradient autograd has to push back through
// log_softmax) never exists:
//   forward   lse[n,t,u] = logsumexp_v logits[n,t,u,v]          (live rows only)
//             units      = logits[n,t,u,{0, y[u-1], y[u]}] - lse
//   backward  d/dlogits[v] = w_n * (G[v] - softmax[v] * (g0 + g1 + g2))
// where G is the gather backward of the unit gradients g (non-zero in at most
// three columns, csrc/gather.cu:311-374 of the reference) and w_n the upstream
// weight of sample n.  Rows of padding and rows outside the band of complete
// alignments are not read at all; their gradient is zero.
// One wavefront per row; a row is read once in each direction.
#include "device_utils.h"
#include "launch.h"
#include "unit_grad.h"

namespace wctct {

namespace {

constexpr int kRowsPerBlock = 4;       // wavefronts per workgroup, forward
constexpr int kGradWaves = 1;          // ... and backward: 4 KiB per workgroup, like the plain zero-fill
constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kLn2F = 0.6931471805599453f;

// one 16-byte vector of floats
__device__ __forceinline__ void load4(const float *p, float (&x)[4]) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    const v4f v = *reinterpret_cast<const v4f *>(p);
    x[0] = v.x;
    x[1] = v.y;
    x[2] = v.z;
    x[3] = v.w;
}
__device__ __forceinline__ void store4(float *p, const float (&x)[4]) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    *reinterpret_cast<v4f *>(p) = v4f{x[0], x[1], x[2], x[3]};
}

// 16-byte vectors of 2-byte elements
__device__ __forceinline__ void load8(const __half *p, float (&x)[8]) {
    typedef _Float16 v8h __attribute__((ext_vector_type(8)));
    const v8h v = *reinterpret_cast<const v8h *>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = (float)v[i];
}
__device__ __forceinline__ void load8(const __hip_bfloat16 *p, float (&x)[8]) {
    typedef unsigned short v8u __attribute__((ext_vector_type(8)));
    const v8u v = *reinterpret_cast<const v8u *>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = __uint_as_float((unsigned)v[i] << 16);
}
// two floats rounded to nearest even into one 32-bit word of 2-byte elements
__device__ __forceinline__ unsigned pack2(const __half *, float a, float b) {
    const __half2 h = __floats2half2_rn(a, b);
    return *reinterpret_cast<const unsigned *>(&h);
}
__device__ __forceinline__ unsigned pack2(const __hip_bfloat16 *, float a, float b) {
    const __hip_bfloat162 h = __float22bfloat162_rn(make_float2(a, b));
    return *reinterpret_cast<const unsigned *>(&h);
}
template <typename IO>
__device__ __forceinline__ void store8(IO *p, const float (&x)[8]) {
    uint4 v;
    v.x = pack2(p, x[0], x[1]);
    v.y = pack2(p, x[2], x[3]);
    v.z = pack2(p, x[4], x[5]);
    v.w = pack2(p, x[6], x[7]);
    *reinterpret_cast<uint4 *>(p) = v;
}
// EV elements = one 16-byte vector of the element type
__device__ __forceinline__ void load_vec(const float *p, float (&x)[4]) { load4(p, x); }
__device__ __forceinline__ void load_vec(const __half *p, float (&x)[8]) { load8(p, x); }
__device__ __forceinline__ void load_vec(const __hip_bfloat16 *p, float (&x)[8]) { load8(p, x); }
__device__ __forceinline__ void store_vec(float *p, const float (&x)[4]) { store4(p, x); }
__device__ __forceinline__ void store_vec(__half *p, const float (&x)[8]) { store8(p, x); }
__device__ __forceinline__ void store_vec(__hip_bfloat16 *p, const float (&x)[8]) { store8(p, x); }

// Maximum / sum over a group of LANES consecutive lanes (64 or 32).
template <int LANES>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int off = LANES / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int off = LANES / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Rows are addressable by 16-byte vectors when every row starts on a 16-byte
// boundary and holds a whole number of them.
template <typename IO>
__device__ __forceinline__ bool rows_vectorised(const IO *base, int V) {
    return (V % (16 / (int)sizeof(IO))) == 0 && (reinterpret_cast<uintptr_t>(base) & 15u) == 0;
}

// ROWS rows per wavefront (64 / ROWS lanes each): one for 4-byte elements, two
// for 2-byte ones, so that a wavefront has 4 KiB of loads in flight either way.
// Each group of lanes owns one cell (t,u) of the work buffer (P contexts per
// frame) of sample blockIdx.y.  Live cells inside the band: logsumexp of the
// row in one pass (running maximum and rescaled sum per lane, combined over
// the group), then the three units.  Other cells of live frames: neutral
// units, as gather_units_kernel.
template <typename IO, int ROWS>
__global__ __launch_bounds__(64 * kRowsPerBlock) void logits_units_kernel(
    const IO *__restrict__ logits, const int *__restrict__ ys, const int *__restrict__ lx,
    const int *__restrict__ ly, double *__restrict__ units, float *__restrict__ lse, int T, int U,
    int V, int P, unsigned *__restrict__ counter) {
    constexpr int LANES = 64 / ROWS;            // lanes per row
    constexpr int EV = 16 / (int)sizeof(IO);    // elements per 16-byte vector
    constexpr int NV = 1024 / (LANES * EV);     // vectors per lane and round of 1024 elements
    if (counter && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *counter = 0u;
    const int n = blockIdx.y;
    const int lane = threadIdx.x & 63, hl = lane % LANES;
    const int cell = (blockIdx.x * kRowsPerBlock + (threadIdx.x >> 6)) * ROWS + lane / LANES;
    const int t = cell / P, u = cell - t * P;
    const int Tn = min(max(lx[n], 0), T), Un = min(max(ly[n], 0), U);
    if (cell >= T * P || t >= Tn) return;
    double *o = units + (((size_t)n * T + t) * P + u) * 3;
    // The groups of a wavefront part ways here; what follows (loads, the
    // reductions over LANES lanes) involves the lanes of one group only.
    if (u > Un || outside_band(t, u, Tn, Un)) {
        if (hl == 0) {
            o[0] = 0.0;
            o[1] = 0.0;
            o[2] = neg_inf();
        }
        return;
    }
    const size_t r = ((size_t)n * T + t) * (U + 1) + u;
    const IO *row = logits + r * (size_t)V;
    // the three logits that become units are requested now (every lane of the
    // group the same address), so that their latency runs in parallel with the
    // row's instead of after the reduction
    const int *y = ys + (size_t)n * U;
    const int c1 = (u >= 1) ? min(max(y[u - 1], 0), V - 1) : 0;
    const int c2 = (u < Un) ? min(max(y[u], 0), V - 1) : 0;
    const float xb = load_as_float(row), x1 = load_as_float(row + c1), x2 = load_as_float(row + c2);
    // running maximum m and sum s of 2^(x*log2e - m) over this lane's elements
    float m = -__builtin_huge_valf(), s = 0.0f;
    if (rows_vectorised(logits, V)) {
        // 1024 elements per round: NV 16-byte vectors per lane, all loads issued
        // before anything is computed (addresses past the row are clamped into
        // it and the values dropped)
        for (int k0 = 0; k0 < V; k0 += 1024) {
            float x[NV][EV];
#pragma unroll
            for (int j = 0; j < NV; ++j)
                load_vec(row + min(k0 + (j * LANES + hl) * EV, V - EV), x[j]);
            float mn = m;
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const bool in = (k0 + (j * LANES + hl) * EV) < V;
#pragma unroll
                for (int i = 0; i < EV; ++i) {
                    x[j][i] = in ? x[j][i] * kLog2eF : -__builtin_huge_valf();
                    mn = fmaxf(mn, x[j][i]);
                }
            }
            // mn = -inf only while everything seen is -inf: keep s = 0
            const float mf = fmaxf(mn, -3.0e38f);
            float acc = s * exp2_hw(m - mf);
#pragma unroll
            for (int j = 0; j < NV; ++j)
#pragma unroll
                for (int i = 0; i < EV; ++i) acc += exp2_hw(x[j][i] - mf);
            s = acc;
            m = mn;
        }
    } else {
        for (int k = hl; k < V; k += LANES) {
            const float x = load_as_float(row + k) * kLog2eF;
            const float mn = fmaxf(m, x);
            const float mf = fmaxf(mn, -3.0e38f);
            s = s * exp2_hw(m - mf) + exp2_hw(x - mf);
            m = mn;
        }
    }
    const float M = group_max<LANES>(m);
    const float Mf = fmaxf(M, -3.0e38f);
    const float S = group_sum<LANES>(s * exp2_hw(m - Mf));
    if (hl != 0) return;
    const float l = (M + log2_hw(S)) * kLn2F;   // natural-log logsumexp of the row
    lse[r] = l;
    const double b = (double)xb - (double)l;
    double cur = b, nxt = neg_inf();
    if (u >= 1) cur = (double)x1 - (double)l;
    if (u < Un) nxt = ((double)x2 - (double)l) * kLog2e;
    o[0] = b * kLog2e;
    o[1] = cur * kLog2e;
    o[2] = nxt;
}

// ROWS rows (n,t,u) of the gradient per wavefront, 64 / ROWS lanes each (see
// logits_units_kernel); blockIdx.y = n.
template <typename IO, int ROWS>
__global__ __launch_bounds__(64 * kGradWaves) void logits_grad_kernel(
    const IO *__restrict__ logits, const float *__restrict__ lse, const double *__restrict__ units,
    const double *__restrict__ alphas, const double *__restrict__ betas,
    const int *__restrict__ ys, const int *__restrict__ lx, const int *__restrict__ ly,
    Weight weight, IO *__restrict__ grad, int T, int U, int V, int P) {
    constexpr int LANES = 64 / ROWS;
    constexpr int EV = 16 / (int)sizeof(IO);    // elements per 16-byte vector
    constexpr int ROUND = 1024;                 // elements of a row per round
    constexpr int NV = ROUND / (LANES * EV);    // vectors per lane and round
    const int U1 = U + 1;
    const int n = blockIdx.y;
    const int lane = threadIdx.x & 63, hl = lane % LANES;
    const int cell = (blockIdx.x * kGradWaves + (threadIdx.x >> 6)) * ROWS + lane / LANES;
    if (cell >= T * U1) return;
    const int t = cell / U1, u = cell - t * U1;
    const int lxn = lx[n];
    const int Tn = min(max(lxn, 0), T), Un = min(max(ly[n], 0), U);
    const size_t r = ((size_t)n * T + t) * U1 + u;
    IO *out = grad + r * (size_t)V;
    const bool vec = rows_vectorised(logits, V) && rows_vectorised(grad, V);
    if (t >= Tn || u > Un || outside_band(t, u, Tn, Un)) {
        if (vec) {
            // zeros in 16-byte pieces whatever the element type
            constexpr int E16 = 16 / (int)sizeof(IO);
            const uint4 zero = {0u, 0u, 0u, 0u};
            for (int k = hl * E16; k < V; k += LANES * E16) *reinterpret_cast<uint4 *>(out + k) = zero;
        } else {
            for (int k = hl; k < V; k += LANES) store_from_float(out + k, 0.0f);
        }
        return;
    }
    // the first round of the row is requested before the (dependent) loads of
    // the unit gradients, not after them
    const IO *row = logits + r * (size_t)V;
    float x[NV][EV];
    if (vec) {
#pragma unroll
        for (int j = 0; j < NV; ++j) load_vec(row + min((j * LANES + hl) * EV, V - EV), x[j]);
    }
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * P * 2;
    const UnitGrad g = unit_grad_cell(units + (size_t)n * T * P * 3, alphas + (size_t)n * lat,
                                      betas + (size_t)n * lat, y, t, u, Un, P);
    const float w = sample_weight(weight, n, lxn);
    const float g0 = g.g0 * w, g1 = g.g1 * w, g2 = g.g2 * w;   // g1 = 0 at u = 0, g2 = 0 at u = Un
    const float total = g0 + g1 + g2;
    const int c1 = (u >= 1) ? min(max(y[u - 1], 0), V - 1) : -1;
    const int c2 = (u < Un) ? min(max(y[u], 0), V - 1) : -1;
    const float shift = lse[r] * kLog2eF;
    if (vec) {
        for (int k0 = 0; k0 < V; k0 += ROUND) {
            if (k0 > 0) {
#pragma unroll
                for (int j = 0; j < NV; ++j)
                    load_vec(row + min(k0 + (j * LANES + hl) * EV, V - EV), x[j]);
            }
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int k = k0 + (j * LANES + hl) * EV;
                if (k >= V) continue;
#pragma unroll
                for (int i = 0; i < EV; ++i) {
                    float v = -total * exp2_hw(x[j][i] * kLog2eF - shift);
                    const int col = k + i;
                    if (col == 0) v += g0;
                    if (col == c1) v += g1;
                    if (col == c2) v += g2;
                    x[j][i] = v;
                }
                store_vec(out + k, x[j]);
            }
        }
    } else {
        for (int k = hl; k < V; k += LANES) {
            float v = -total * exp2_hw(load_as_float(row + k) * kLog2eF - shift);
            if (k == 0) v += g0;
            if (k == c1) v += g1;
            if (k == c2) v += g2;
            store_from_float(out + k, v);
        }
    }
}

// Rows per wavefront by element size: 4 KiB of a row per 64 lanes either way.
template <typename IO> struct RowsPerWave { static constexpr int value = sizeof(IO) == 4 ? 1 : 2; };

template <typename IO>
void launch_units_typed(const void *logits, const int *ys, const int *lx, const int *ly,
                        double *units, float *lse, int N, int T, int U, int V, unsigned *counter,
                        hipStream_t stream) {
    const int P = padded_contexts(U);
    const long cells = (long)T * P;
    constexpr int ROWS = RowsPerWave<IO>::value, PER_BLOCK = kRowsPerBlock * ROWS;
    dim3 grid((unsigned)((cells + PER_BLOCK - 1) / PER_BLOCK), (unsigned)N);
    TIMED_LAUNCH((logits_units_kernel<IO, ROWS>), grid, dim3(64 * kRowsPerBlock), 0, stream,
                       static_cast<const IO *>(logits), ys, lx, ly, units, lse, T, U, V, P,
                       counter);
}

template <typename IO>
void launch_grad_typed(const void *logits, const float *lse, const double *units,
                       const double *alphas, const double *betas, const int *ys, const int *lx,
                       const int *ly, const Weight &w, void *grad, int N, int T, int U, int V,
                       hipStream_t stream) {
    const long cells = (long)T * (U + 1);
    constexpr int ROWS = RowsPerWave<IO>::value, PER_BLOCK = kGradWaves * ROWS;
    dim3 grid((unsigned)((cells + PER_BLOCK - 1) / PER_BLOCK), (unsigned)N);
    TIMED_LAUNCH((logits_grad_kernel<IO, ROWS>), grid, dim3(64 * kGradWaves), 0, stream,
                       static_cast<const IO *>(logits), lse, units, alphas, betas, ys, lx, ly, w,
                       static_cast<IO *>(grad), T, U, V, padded_contexts(U));
}

}  // namespace

hipError_t launch_logits_units(const void *logits, int io_type, const int *ys, const int *lx,
                               const int *ly, double *units, float *lse, int N, int T, int U,
                               int V, unsigned *counter, hipStream_t stream) {
    if (N == 0 || T == 0) return hipSuccess;
    switch (io_type) {
        case kIoF32:
            launch_units_typed<float>(logits, ys, lx, ly, units, lse, N, T, U, V, counter, stream);
            break;
        case kIoF16:
            launch_units_typed<__half>(logits, ys, lx, ly, units, lse, N, T, U, V, counter,
                                       stream);
            break;
        case kIoBF16:
            launch_units_typed<__hip_bfloat16>(logits, ys, lx, ly, units, lse, N, T, U, V, counter,
                                               stream);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_logits_grad(const void *logits, int io_type, const float *lse,
                              const double *units, const double *alphas, const double *betas,
                              const int *ys, const int *lx, const int *ly, const float *grad_out,
                              int grad_out_stride, float scale, int average_frames, void *grad,
                              int N, int T, int U, int V, hipStream_t stream) {
    if (N == 0 || T == 0) return hipSuccess;
    const Weight w = {grad_out, grad_out_stride, scale, average_frames};
    switch (io_type) {
        case kIoF32:
            launch_grad_typed<float>(logits, lse, units, alphas, betas, ys, lx, ly, w, grad, N, T,
                                     U, V, stream);
            break;
        case kIoF16:
            launch_grad_typed<__half>(logits, lse, units, alphas, betas, ys, lx, ly, w, grad, N, T,
                                      U, V, stream);
            break;
        case kIoBF16:
            launch_grad_typed<__hip_bfloat16>(logits, lse, units, alphas, betas, ys, lx, ly, w,
                                              grad, N, T, U, V, stream);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace wctct
