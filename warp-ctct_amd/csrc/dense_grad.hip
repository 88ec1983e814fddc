// Dense gradient of ctct_loss wrt the (N,T,U+1,V) joint tensor.
//
// The reference obtains it in two steps: CTCTLoss.backward scales the saved
// unit gradients by grad_output (warp_ctct/__init__.py:30-33) and autograd's
// gather backward zero-fills an (N,T,U+1,V) tensor and scatter-adds into it.
// The result is all zeros except, in row (n,t,u), columns 0, y[u-1], y[u],
// which hold grad_out[n] * g0 / g1 / g2 (coincident columns add).
//
// The zero-fill is pure HBM write traffic (4*N*T*(U+1)*V bytes) and decides
// the throughput of the whole loss, so it is kept free of everything else.
// Measurements on MI355X (N=32, T=250, U=60, V=1024; 2.0 GB) behind this:
//  * zero_fill_vec_kernel — a 256-thread workgroup issues ONE 16-byte store
//    per thread (4 KiB contiguous per workgroup) and retires — reaches
//    ~6.7 TB/s (295 us); workgroups that loop over 16-64 KiB, persistent
//    grid-stride loops and non-temporal stores all lose 10-35 %;
//  * a fused kernel whose workgroups also fetch their row's labels and unit
//    gradients (before the store, or after it with the non-zero lanes storing
//    a second time) takes 370-480 us: a wave that waits for a load keeps its
//    slot, and the fill lives off instant wave turnover;
//  * the separate sparse pass (patch_kernel) costs 25-35 us whether it reads
//    ready-made unit gradients or computes them on the fly from alpha / beta.
//    What it stores matters beyond its own duration: 4-byte stores into lines
//    that have left the caches leave partial lines behind whose write-back
//    (a read-modify-write on the memory side) slows whatever runs next: the
//    following step's zero-fill took 305 us instead of 292 us, 335 us when it
//    came right after the patch.  Whole aligned 128-byte segments, written by
//    8 lanes x 16 bytes each, cost the fill nothing and the patch itself
//    27 us instead of 35 us (one thread writing its row's segments alone:
//    44 us; 64-byte segments: 28 us but the fill still suffers);
//  * running the fill on a second stream next to the gather / lattice kernels
//    is no faster than running everything back to back (the fill takes 330 us
//    instead of 290 us, and forking and joining the streams costs ~30 us, which
//    a small batch feels most);
//  * the fill does not need every wave slot: at 4 (or 2) wavefronts per SIMD
//    it takes 280 us, at all 8 it takes 289 us, at 1 it takes 460 us; 64-thread
//    workgroups take 415 us, 512 threads 289 us, 1024 threads 313 us;
//  * workgroups of the fill appended to the LATTICE kernel's launch (see
//    lattice_fill_kernel) run beside the sweeps at the fill's own speed
//    (282 us for both): the sweeps wait on chains of dependent arithmetic and
//    hardly touch memory.  The same trick with the gather kernel gains nothing
//    (its workgroups in front: they run first, then the fill) or loses (spread
//    between the fill's: scattered reads between the writes slow the fill by
//    half).
// Hence: the forward clears the buffer inside the lattice kernel's launch when
// the caller hands it over (warpctct_loss_lattice_clearing) and the backward
// only patches; or, on a buffer of the backward's own, fill then patch.
#include "device_utils.h"
#include "launch.h"
#include "unit_grad.h"

namespace wctct {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;

// p[i] = 0 for i < n bytes, for the few bytes before and after the 16-byte
// aligned body of a buffer.
__global__ __launch_bounds__(kBlock) void zero_fill_byte_kernel(unsigned char *__restrict__ p,
                                                                size_t n) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    if (i < n) p[i] = 0;
}

// p4[i] = 0 for i < n4: one store per thread, no loop; at most 4 wavefronts per
// SIMD (with all 8 the memory side queues up and the fill takes 3 % longer;
// 2 are as good as 4, 1 is far too few).
__global__ __launch_bounds__(kBlock) __attribute__((amdgpu_waves_per_eu(4, 4))) void
zero_fill_vec_kernel(v4f *__restrict__ p4, size_t n4) {
    const size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x;
    const v4f z = {0.0f, 0.0f, 0.0f, 0.0f};
    if (i < n4) p4[i] = z;
}

// The non-zero entries of one row of the dense gradient, coincident columns
// merged: v0 at column 0, v1 at column c1 (if c1 > 0), v2 at column c2 (if
// c2 > 0); c1 != c2.
struct RowPatch {
    float v0, v1, v2;
    int c1, c2;
};

// Row (n,t,u): columns 0, y[u-1], y[u] hold v0, v1, v2; columns that coincide
// are summed so that every element is written by exactly one store.
__device__ __forceinline__ RowPatch merge_columns(const int *y, int u, int Un, int V, float v0,
                                                  float v1, float v2) {
    const bool has1 = (u >= 1), has2 = (u < Un);
    RowPatch r;
    r.c1 = has1 ? min(max(y[u - 1], 0), V - 1) : -1;
    r.c2 = has2 ? min(max(y[u], 0), V - 1) : -1;
    if (!has1) v1 = 0.0f;
    if (!has2) v2 = 0.0f;
    if (r.c2 == r.c1) {   // y[u-1] == y[u]: both label units land in one column
        v1 += v2;
        r.c2 = -1;
    }
    if (r.c1 == 0) {      // a label equal to the blank index
        v0 += v1;
        r.c1 = -1;
    }
    if (r.c2 == 0) {
        v0 += v2;
        r.c2 = -1;
    }
    r.v0 = v0, r.v1 = v1, r.v2 = v2;
    return r;
}

// Aligned piece of a row that the patch writes whole (zeros around the value).
// A partial write of a 128-byte line costs the memory side a read-modify-write
// whose drain slows the kernels that follow (the next zero-fill by ~15 us on
// the 2 GB gradient of a typical batch); a whole line does not.
constexpr int kSegment = 128;

// The 16 bytes number `part` of segment `seg` of a row.
template <typename IO>
__device__ __forceinline__ void store_segment_part(IO *row, int seg, int part, const RowPatch &r) {
    constexpr int W = kSegment / (int)sizeof(IO);   // elements per segment
    constexpr int E = 16 / (int)sizeof(IO);         // elements per 16-byte store
    const int first = seg * W + part * E;
    alignas(16) IO vals[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
        const int col = first + i;
        float v = 0.0f;
        if (col == 0) v = r.v0;
        if (col == r.c1) v = r.v1;
        if (col == r.c2) v = r.v2;
        store_from_float(&vals[i], v);
    }
    *reinterpret_cast<uint4 *>(row + first) = *reinterpret_cast<const uint4 *>(vals);
}

// One thread per cell (t,u) of sample blockIdx.y computes the row's entries;
// FROM_LATTICE computes the unit gradients on the fly from units / alpha /
// beta (work-buffer layout, P contexts per frame), otherwise they are read
// from the (N,T,U+1,3) tensor.  The entries are then written by the whole
// wavefront: 8 lanes per row, each 16 bytes of a 128-byte segment, so that a
// store instruction covers 8 whole lines (rows whose size or address does not
// allow that are written element by element by their own thread).
template <bool FROM_LATTICE, typename IO>
__global__ __launch_bounds__(kBlock) void patch_kernel(
    const float *__restrict__ unit_grads, const double *__restrict__ units,
    const double *__restrict__ alphas, const double *__restrict__ betas,
    const int *__restrict__ ys, const int *__restrict__ lx, const int *__restrict__ ly,
    Weight weight, IO *__restrict__ dense, int T, int U, int V, int P) {
    const int U1 = U + 1;
    const int n = blockIdx.y;
    const int cell = blockIdx.x * kBlock + threadIdx.x;
    const int t = cell / U1, u = cell - t * U1;
    const int lxn = lx[n];
    const int Tn = min(max(lxn, 0), T);
    const int Un = min(max(ly[n], 0), U);
    // outside the band the gradient is exactly zero: the fill wrote it already
    const bool live = cell < T * U1 && t < Tn && u <= Un &&
                      !(FROM_LATTICE && outside_band(t, u, Tn, Un));
    const size_t row = ((size_t)n * T + t) * U1 + u;
    RowPatch r = {0.0f, 0.0f, 0.0f, -1, -1};
    if (live) {
        const int *y = ys + (size_t)n * U;
        UnitGrad g;
        if (FROM_LATTICE) {
            const size_t lat = (size_t)(T + 1) * P * 2;
            g = unit_grad_cell(units + (size_t)n * T * P * 3, alphas + (size_t)n * lat,
                               betas + (size_t)n * lat, y, t, u, Un, P);
        } else {
            const float *p = unit_grads + row * 3;
            g.g0 = p[0];
            g.g1 = p[1];
            g.g2 = p[2];
        }
        const float w = sample_weight(weight, n, lxn);
        r = merge_columns(y, u, Un, V, g.g0 * w, g.g1 * w, g.g2 * w);
    }
    // rows start on segment boundaries and hold whole segments
    const bool segments = ((size_t)V * sizeof(IO)) % kSegment == 0 &&
                          (reinterpret_cast<uintptr_t>(dense) & (kSegment - 1)) == 0;
    if (!segments) {
        if (live) {
            IO *out = dense + row * (size_t)V;
            store_from_float(out, r.v0);
            if (r.c1 > 0) store_from_float(out + r.c1, r.v1);
            if (r.c2 > 0) store_from_float(out + r.c2, r.v2);
        }
        return;
    }
    constexpr int W = kSegment / (int)sizeof(IO);
    const int lane = threadIdx.x & 63;
    const int part = lane & 7, group = lane >> 3;
    // consecutive lanes hold consecutive rows: row of lane 0 of this wavefront
    IO *wave_rows = dense + (row - lane) * (size_t)V;
    for (int j = 0; j < 8; ++j) {
        const int src = j * 8 + group;
        const int src_live = __shfl((int)live, src, 64);
        if (__ballot(src_live) == 0) continue;   // wavefront-uniform
        RowPatch q;
        q.v0 = __shfl(r.v0, src, 64);
        q.v1 = __shfl(r.v1, src, 64);
        q.v2 = __shfl(r.v2, src, 64);
        q.c1 = __shfl(r.c1, src, 64);
        q.c2 = __shfl(r.c2, src, 64);
        if (src_live) {
            IO *out = wave_rows + (size_t)src * V;
            const int s1 = q.c1 > 0 ? q.c1 / W : 0, s2 = q.c2 > 0 ? q.c2 / W : 0;
            store_segment_part(out, 0, part, q);
            if (s1 > 0) store_segment_part(out, s1, part, q);
            if (s2 > 0 && s2 != s1) store_segment_part(out, s2, part, q);
        }
    }
}

}  // namespace

hipError_t launch_zero_fill_bytes(void *ptr, size_t bytes, hipStream_t stream) {
    if (bytes == 0) return hipSuccess;
    // leading bytes up to the first 16-byte boundary, then vectors, then the tail
    unsigned char *p = static_cast<unsigned char *>(ptr);
    size_t head = (16 - (reinterpret_cast<uintptr_t>(p) & 15u)) & 15u;
    if (head > bytes) head = bytes;
    const size_t n4 = (bytes - head) / 16;
    const size_t tail = bytes - head - n4 * 16;
    if (head) {
        TIMED_LAUNCH(zero_fill_byte_kernel, dim3(1), dim3(kBlock), 0, stream, p, head);
    }
    if (n4) {
        const size_t blocks = (n4 + kBlock - 1) / kBlock;
        if (blocks > 0x7fffffffUL) return hipErrorInvalidValue;
        TIMED_LAUNCH(zero_fill_vec_kernel, dim3((unsigned)blocks), dim3(kBlock), 0, stream,
                           reinterpret_cast<v4f *>(p + head), n4);
    }
    if (tail) {
        TIMED_LAUNCH(zero_fill_byte_kernel, dim3(1), dim3(kBlock), 0, stream,
                           p + head + n4 * 16, tail);
    }
    return hipGetLastError();
}

hipError_t launch_zero_fill(float *p, size_t n, hipStream_t stream) {
    return launch_zero_fill_bytes(p, n * sizeof(float), stream);
}

hipError_t launch_dense_patch(const float *unit_grads, const int *ys, const int *lx,
                              const int *ly, const float *grad_out, float *dense, int N, int T,
                              int U, int V, hipStream_t stream) {
    const long cells = (long)T * (U + 1);
    if (cells == 0 || N == 0) return hipSuccess;
    dim3 grid((unsigned)((cells + kBlock - 1) / kBlock), (unsigned)N);
    const Weight w = {grad_out, 1, 1.0f, 0};
    TIMED_LAUNCH((patch_kernel<false, float>), grid, dim3(kBlock), 0, stream, unit_grads,
                       nullptr, nullptr, nullptr, ys, lx, ly, w, dense, T, U, V, 0);
    return hipGetLastError();
}

hipError_t launch_dense_patch_lattice(const double *units, const double *alphas,
                                      const double *betas, const int *ys, const int *lx,
                                      const int *ly, const float *grad_out, int grad_out_stride,
                                      float scale, int average_frames, void *dense, int io_type,
                                      int N, int T, int U, int V, hipStream_t stream) {
    const long cells = (long)T * (U + 1);
    if (cells == 0 || N == 0) return hipSuccess;
    dim3 grid((unsigned)((cells + kBlock - 1) / kBlock), (unsigned)N);
    const Weight w = {grad_out, grad_out_stride, scale, average_frames};
    const int P = padded_contexts(U);
    switch (io_type) {
        case kIoF32:
            TIMED_LAUNCH((patch_kernel<true, float>), grid, dim3(kBlock), 0, stream, nullptr,
                               units, alphas, betas, ys, lx, ly, w, static_cast<float *>(dense), T,
                               U, V, P);
            break;
        case kIoF16:
            TIMED_LAUNCH((patch_kernel<true, __half>), grid, dim3(kBlock), 0, stream,
                               nullptr, units, alphas, betas, ys, lx, ly, w,
                               static_cast<__half *>(dense), T, U, V, P);
            break;
        case kIoBF16:
            TIMED_LAUNCH((patch_kernel<true, __hip_bfloat16>), grid, dim3(kBlock), 0, stream,
                               nullptr, units, alphas, betas, ys, lx, ly, w,
                               static_cast<__hip_bfloat16 *>(dense), T, U, V, P);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_dense_grad(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                             const float *grad_out, float *dense, int N, int T, int U, int V,
                             hipStream_t stream) {
    hipError_t e = launch_zero_fill(dense, (size_t)N * T * (U + 1) * V, stream);
    if (e != hipSuccess) return e;
    return launch_dense_patch(unit_grads, ys, lx, ly, grad_out, dense, N, T, U, V, stream);
}

}  // namespace wctct
