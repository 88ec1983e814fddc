// Alpha / beta lattices of the CTC-Transducer loss on gfx950.
//
// One 64-lane wavefront owns one (sample, direction).  The sweep is
// time-synchronous: all states of frame t are updated from frame t-1 (alpha)
// or t+1 (beta); states of one frame do not depend on each other, so a step
// needs no barrier and no atomics — only one value from the neighbouring
// context, moved with single-lane DPP shifts.  Lane l owns K consecutive
// contexts u = l*K .. l*K+K-1 and, for each, the state pair
//     o = state 2u-1 (inside label y[u-1])      e = state 2u (blank after u labels)
// so the whole front lives in registers.  Values are log2 of the path mass,
// held in double; the exponentials and logarithms of the semiring sum run on
// the fp32 transcendental unit (see device_utils.h).  Units for the next
// frames are prefetched into registers one chunk of R frames ahead.
//
// Math restated from ref_ctct.py:6-74 of the reference (alpha :6-37, beta
// :40-74); this kernel replaces k_warp_alphas / k_warp_betas
// (csrc/gather.cu:36-291) and their spin-lock row pipeline.
#include "device_utils.h"
#include "launch.h"

namespace wctct {

template <int K>
struct Front {
    double e[K];
    double o[K];
};

template <int K>
__device__ __forceinline__ void front_store(double *dst, const Front<K> &f, int u0, int Un) {
    // dst points at [t][u0][0]; pairs {o, e}
#pragma unroll
    for (int j = 0; j < K; ++j) {
        if (u0 + j <= Un)
            *reinterpret_cast<double2 *>(dst + 2 * j) = make_double2(f.o[j], f.e[j]);
    }
}

template <int K, int R>
struct Chunk {
    double lp[R][K][3];
};

// Load the units of frames t_first + dir*r, r in [0,R), for this lane's
// contexts.  Frames outside [0,Tn) and contexts beyond Un are not touched in
// memory; their units read as 0, and the "next label" unit of context Un (and
// beyond) reads as -inf so that no mass flows past the last label.
template <int K, int R>
__device__ __forceinline__ void chunk_load(Chunk<K, R> &c, const double *units_n, int U1, int u0,
                                           int Un, int Tn, int t_first, int dir) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = t_first + dir * r;
        const bool t_ok = (t >= 0) && (t < Tn);
#pragma unroll
        for (int j = 0; j < K; ++j) {
            const int u = u0 + j;
            double b = 0.0, cur = 0.0, nxt = 0.0;
            if (t_ok && u <= Un) {
                const double *p = units_n + ((size_t)t * U1 + u) * 3;
                b = p[0];
                cur = p[1];
                nxt = p[2];
            }
            c.lp[r][j][0] = b;
            c.lp[r][j][1] = cur;
            c.lp[r][j][2] = (u < Un) ? nxt : neg_inf();
        }
    }
}

// ---- alpha ---------------------------------------------------------------
// alpha(t+1, 2u)   = [alpha(t,2u) (+) alpha(t,2u-1)] + LP(t,u,0)
// alpha(t+1, 2u-1) =  alpha(t,2u-1) + LP(t,u,1)
//                 (+) alpha(t,2u-2) + LP(t,u-1,2)
//                 (+) [y[u-1] != y[u-2]] alpha(t,2u-3) + LP(t,u-1,2)
template <int K>
__device__ __forceinline__ void alpha_step(Front<K> &f, const double (*lp)[3], const bool *skip) {
    double from_e[K], from_o[K];
#pragma unroll
    for (int j = 0; j < K; ++j) {
        from_e[j] = f.e[j] + lp[j][2];
        from_o[j] = f.o[j] + lp[j][2];
    }
    const double in_e = wave_shift_up(from_e[K - 1], neg_inf());
    const double in_o = wave_shift_up(from_o[K - 1], neg_inf());
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const double pe = (j == 0) ? in_e : from_e[j - 1];
        const double po = (j == 0) ? in_o : from_o[j - 1];
        const double ne = lse2(f.e[j], f.o[j]) + lp[j][0];
        const double no = lse3(f.o[j] + lp[j][1], pe, skip[j] ? po : neg_inf());
        f.e[j] = ne;
        f.o[j] = no;
    }
}

template <int K, int R>
__device__ void alpha_sweep(const double *units_n, const int *y, int Tn, int Un, int U1,
                            double *alpha_n) {
    const int lane = threadIdx.x;
    const int u0 = lane * K;
    bool skip[K];
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int u = u0 + j;
        skip[j] = (u >= 2) && (u <= Un) && (y[u - 1] != y[u - 2]);
    }
    Front<K> f;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        f.e[j] = neg_inf();
        f.o[j] = neg_inf();
    }
    if (lane == 0) f.e[0] = 0.0;
    const size_t row = (size_t)U1 * 2;
    double *out = alpha_n + (size_t)u0 * 2;
    front_store<K>(out, f, u0, Un);

    Chunk<K, R> a, b;
    chunk_load<K, R>(a, units_n, U1, u0, Un, Tn, 0, 1);
    for (int t0 = 0; t0 < Tn; t0 += 2 * R) {
        chunk_load<K, R>(b, units_n, U1, u0, Un, Tn, t0 + R, 1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int t = t0 + r;
            if (t < Tn) {
                alpha_step<K>(f, a.lp[r], skip);
                front_store<K>(out + (size_t)(t + 1) * row, f, u0, Un);
            }
        }
        chunk_load<K, R>(a, units_n, U1, u0, Un, Tn, t0 + 2 * R, 1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int t = t0 + R + r;
            if (t < Tn) {
                alpha_step<K>(f, b.lp[r], skip);
                front_store<K>(out + (size_t)(t + 1) * row, f, u0, Un);
            }
        }
    }
}

// ---- beta ----------------------------------------------------------------
// beta(t, 2u)   = beta(t+1,2u) + LP(t,u,0)  (+) [u<U] beta(t+1,2u+1) + LP(t,u,2)
// beta(t, 2u-1) = beta(t+1,2u-1) + LP(t,u,1) (+) beta(t+1,2u) + LP(t,u,0)
//              (+) [u<U, y[u-1] != y[u]] beta(t+1,2u+1) + LP(t,u,2)
template <int K>
__device__ __forceinline__ void beta_step(Front<K> &f, const double (*lp)[3], const bool *skip,
                                          const bool *has_o) {
    const double in_o = wave_shift_down(f.o[0], neg_inf());
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const double nb = (j == K - 1) ? in_o : f.o[j + 1];   // context j+1 is still at t+1
        const double nxt = nb + lp[j][2];
        const double stay_e = f.e[j] + lp[j][0];
        const double ne = lse2(stay_e, nxt);
        const double no = lse3(f.o[j] + lp[j][1], stay_e, skip[j] ? nxt : neg_inf());
        f.e[j] = ne;
        f.o[j] = has_o[j] ? no : neg_inf();
    }
}

template <int K, int R>
__device__ void beta_sweep(const double *units_n, const int *y, int Tn, int Un, int U1,
                           double *beta_n, float *cost_n) {
    const int lane = threadIdx.x;
    const int u0 = lane * K;
    bool skip[K], has_o[K];
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int u = u0 + j;
        has_o[j] = (u >= 1) && (u <= Un);
        skip[j] = (u >= 1) && (u < Un) && (y[u - 1] != y[u]);
    }
    Front<K> f;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int u = u0 + j;
        f.e[j] = (u == Un) ? 0.0 : neg_inf();
        f.o[j] = (u == Un && Un >= 1) ? 0.0 : neg_inf();
    }
    const size_t row = (size_t)U1 * 2;
    double *out = beta_n + (size_t)u0 * 2;
    front_store<K>(out + (size_t)Tn * row, f, u0, Un);

    Chunk<K, R> a, b;
    chunk_load<K, R>(a, units_n, U1, u0, Un, Tn, Tn - 1, -1);
    for (int s0 = 0; s0 < Tn; s0 += 2 * R) {
        chunk_load<K, R>(b, units_n, U1, u0, Un, Tn, Tn - 1 - (s0 + R), -1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int t = Tn - 1 - (s0 + r);
            if (t >= 0) {
                beta_step<K>(f, a.lp[r], skip, has_o);
                front_store<K>(out + (size_t)t * row, f, u0, Un);
            }
        }
        chunk_load<K, R>(a, units_n, U1, u0, Un, Tn, Tn - 1 - (s0 + 2 * R), -1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const int t = Tn - 1 - (s0 + R + r);
            if (t >= 0) {
                beta_step<K>(f, b.lp[r], skip, has_o);
                front_store<K>(out + (size_t)t * row, f, u0, Un);
            }
        }
    }
    // cost = -beta(0, state 0) in natural-log units (csrc/binding.cpp:86)
    if (lane == 0) *cost_n = (float)(-f.e[0] * kLn2);
}

// grid = (N, beta_only ? 1 : 2), block = 64.  blockIdx.y == 0 runs beta (it
// also produces the cost), blockIdx.y == 1 runs alpha.
template <int K, int R>
__global__ __launch_bounds__(64) void lattice_kernel(const double *__restrict__ units,
                                                     const int *__restrict__ ys,
                                                     const int *__restrict__ lx,
                                                     const int *__restrict__ ly,
                                                     double *__restrict__ alphas,
                                                     double *__restrict__ betas,
                                                     float *__restrict__ costs, int T, int U) {
    const int n = blockIdx.x;
    const int U1 = U + 1;
    // lengths outside the allocation are clamped: nothing is ever read or
    // written beyond (T, U), whatever the length tensors hold
    const int Tn = min(max(lx[n], 0), T);
    const int Un = min(max(ly[n], 0), U);
    const double *units_n = units + (size_t)n * T * U1 * 3;
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * U1 * 2;
    if (blockIdx.y == 0)
        beta_sweep<K, R>(units_n, y, Tn, Un, U1, betas + (size_t)n * lat, costs + n);
    else
        alpha_sweep<K, R>(units_n, y, Tn, Un, U1, alphas + (size_t)n * lat);
}

template <int K, int R>
static hipError_t launch_lattice_k(const LatticeArgs &a, hipStream_t stream) {
    dim3 grid(a.N, a.beta_only ? 1 : 2);
    hipLaunchKernelGGL((lattice_kernel<K, R>), grid, dim3(64), 0, stream, a.units, a.ys, a.lx,
                       a.ly, a.alphas, a.betas, a.costs, a.T, a.U);
    return hipGetLastError();
}

int lattice_max_contexts() { return 64 * 8; }

hipError_t launch_lattice(const LatticeArgs &a, hipStream_t stream) {
    const int K = (a.U + 1 + 63) / 64;
    switch (K) {
        case 1: return launch_lattice_k<1, 8>(a, stream);
        case 2: return launch_lattice_k<2, 4>(a, stream);
        case 3: return launch_lattice_k<3, 4>(a, stream);
        case 4: return launch_lattice_k<4, 2>(a, stream);
        case 5: return launch_lattice_k<5, 2>(a, stream);
        case 6: return launch_lattice_k<6, 2>(a, stream);
        case 7: return launch_lattice_k<7, 2>(a, stream);
        case 8: return launch_lattice_k<8, 2>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace wctct
