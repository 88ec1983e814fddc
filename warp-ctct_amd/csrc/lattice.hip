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

// Work buffers are padded to P = 64*K contexts per frame so that every lane
// loads and stores unconditionally: no exec-mask branches in the sweep, which
// lets the compiler count outstanding loads exactly and keep the prefetch of
// the next chunk in flight while the current one is consumed.
//   units  (N, T,   P, 3)  {blank, cur, next}; for u > Un: {0, 0, -inf},
//                          and next = -inf at u = Un (no label follows)
//   alpha, beta (N, T+1, P, 2) pairs {o, e}
template <int K>
__device__ __forceinline__ void front_store(double *dst, const Front<K> &f) {
#pragma unroll
    for (int j = 0; j < K; ++j)
        *reinterpret_cast<double2 *>(dst + 2 * j) = make_double2(f.o[j], f.e[j]);
}

template <int K, int R>
struct Chunk {
    double lp[R][K][3];
};

// Units of frames t_first + dir*r, r in [0,R); the frame index is clamped into
// [0, Tn-1] so that a prefetch past the end re-reads a valid row (its values
// are then not used).
template <int K, int R>
__device__ __forceinline__ void chunk_load(Chunk<K, R> &c, const double *units_lane, size_t row,
                                           int Tn, int t_first, int dir) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = min(max(t_first + dir * r, 0), Tn - 1);
        const double *p = units_lane + (size_t)t * row;
#pragma unroll
        for (int j = 0; j < K; ++j) {
            c.lp[r][j][0] = p[3 * j];
            c.lp[r][j][1] = p[3 * j + 1];
            c.lp[r][j][2] = p[3 * j + 2];
        }
    }
}

// ---- alpha ---------------------------------------------------------------
// alpha(t+1, 2u)   = [alpha(t,2u) (+) alpha(t,2u-1)] + LP(t,u,0)
// alpha(t+1, 2u-1) =  alpha(t,2u-1) + LP(t,u,1)
//                 (+) alpha(t,2u-2) + LP(t,u-1,2)
//                 (+) [y[u-1] != y[u-2]] alpha(t,2u-3) + LP(t,u-1,2)
// skip_mask[j] is 0 where the third arc exists and -inf where it does not.
template <int K>
__device__ __forceinline__ void alpha_step(Front<K> &f, const double (*lp)[3],
                                           const double *skip_mask) {
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
        const double no = lse3(f.o[j] + lp[j][1], pe, po + skip_mask[j]);
        f.e[j] = ne;
        f.o[j] = no;
    }
}

template <int K, int R>
__device__ void alpha_sweep(const double *units_n, const int *y, int Tn, int Un, int P,
                            double *alpha_n) {
    const int lane = threadIdx.x;
    const int u0 = lane * K;
    double skip_mask[K];
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int u = u0 + j;
        const bool skip = (u >= 2) && (u <= Un) && (y[u - 1] != y[u - 2]);
        skip_mask[j] = skip ? 0.0 : neg_inf();
    }
    Front<K> f;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        f.e[j] = neg_inf();
        f.o[j] = neg_inf();
    }
    if (lane == 0) f.e[0] = 0.0;
    const size_t srow = (size_t)P * 2;       // doubles per frame of alpha
    const size_t urow = (size_t)P * 3;       // doubles per frame of units
    double *out = alpha_n + (size_t)u0 * 2;
    const double *in = units_n + (size_t)u0 * 3;
    front_store<K>(out, f);
    if (Tn == 0) return;

    Chunk<K, R> a, b;
    int t0 = 0;
    chunk_load<K, R>(a, in, urow, Tn, 0, 1);
    while (t0 + 2 * R <= Tn) {
        chunk_load<K, R>(b, in, urow, Tn, t0 + R, 1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            alpha_step<K>(f, a.lp[r], skip_mask);
            front_store<K>(out + (size_t)(t0 + r + 1) * srow, f);
        }
        chunk_load<K, R>(a, in, urow, Tn, t0 + 2 * R, 1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            alpha_step<K>(f, b.lp[r], skip_mask);
            front_store<K>(out + (size_t)(t0 + R + r + 1) * srow, f);
        }
        t0 += 2 * R;
    }
    // fewer than 2R frames left
    chunk_load<K, R>(b, in, urow, Tn, t0 + R, 1);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (t0 + r < Tn) {
            alpha_step<K>(f, a.lp[r], skip_mask);
            front_store<K>(out + (size_t)(t0 + r + 1) * srow, f);
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (t0 + R + r < Tn) {
            alpha_step<K>(f, b.lp[r], skip_mask);
            front_store<K>(out + (size_t)(t0 + R + r + 1) * srow, f);
        }
    }
}

// ---- beta ----------------------------------------------------------------
// beta(t, 2u)   = beta(t+1,2u) + LP(t,u,0)  (+) [u<U] beta(t+1,2u+1) + LP(t,u,2)
// beta(t, 2u-1) = beta(t+1,2u-1) + LP(t,u,1) (+) beta(t+1,2u) + LP(t,u,0)
//              (+) [u<U, y[u-1] != y[u]] beta(t+1,2u+1) + LP(t,u,2)
// o_mask[j] is 0 for contexts that have a state 2u-1 (1 <= u <= Un), else -inf.
template <int K>
__device__ __forceinline__ void beta_step(Front<K> &f, const double (*lp)[3],
                                          const double *skip_mask, const double *o_mask) {
    const double in_o = wave_shift_down(f.o[0], neg_inf());
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const double nb = (j == K - 1) ? in_o : f.o[j + 1];   // context j+1 is still at t+1
        const double nxt = nb + lp[j][2];
        const double stay_e = f.e[j] + lp[j][0];
        const double ne = lse2(stay_e, nxt);
        const double no = lse3(f.o[j] + lp[j][1], stay_e, nxt + skip_mask[j]);
        f.e[j] = ne;
        f.o[j] = no + o_mask[j];
    }
}

template <int K, int R>
__device__ void beta_sweep(const double *units_n, const int *y, int Tn, int Un, int P,
                           double *beta_n, float *cost_n) {
    const int lane = threadIdx.x;
    const int u0 = lane * K;
    double skip_mask[K], o_mask[K];
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int u = u0 + j;
        const bool skip = (u >= 1) && (u < Un) && (y[u - 1] != y[u]);
        skip_mask[j] = skip ? 0.0 : neg_inf();
        o_mask[j] = ((u >= 1) && (u <= Un)) ? 0.0 : neg_inf();
    }
    Front<K> f;
#pragma unroll
    for (int j = 0; j < K; ++j) {
        const int u = u0 + j;
        f.e[j] = (u == Un) ? 0.0 : neg_inf();
        f.o[j] = (u == Un && Un >= 1) ? 0.0 : neg_inf();
    }
    const size_t srow = (size_t)P * 2;
    const size_t urow = (size_t)P * 3;
    double *out = beta_n + (size_t)u0 * 2;
    const double *in = units_n + (size_t)u0 * 3;
    front_store<K>(out + (size_t)Tn * srow, f);

    if (Tn > 0) {
        Chunk<K, R> a, b;
        int t1 = Tn - 1;                      // frame consumed by the next step
        chunk_load<K, R>(a, in, urow, Tn, t1, -1);
        while (t1 - 2 * R + 1 >= 0) {
            chunk_load<K, R>(b, in, urow, Tn, t1 - R, -1);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                beta_step<K>(f, a.lp[r], skip_mask, o_mask);
                front_store<K>(out + (size_t)(t1 - r) * srow, f);
            }
            chunk_load<K, R>(a, in, urow, Tn, t1 - 2 * R, -1);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                beta_step<K>(f, b.lp[r], skip_mask, o_mask);
                front_store<K>(out + (size_t)(t1 - R - r) * srow, f);
            }
            t1 -= 2 * R;
        }
        // fewer than 2R frames left: t1, t1-1, .., 0
        chunk_load<K, R>(b, in, urow, Tn, t1 - R, -1);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (t1 - r >= 0) {
                beta_step<K>(f, a.lp[r], skip_mask, o_mask);
                front_store<K>(out + (size_t)(t1 - r) * srow, f);
            }
        }
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (t1 - R - r >= 0) {
                beta_step<K>(f, b.lp[r], skip_mask, o_mask);
                front_store<K>(out + (size_t)(t1 - R - r) * srow, f);
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
    constexpr int P = 64 * K;
    // lengths outside the allocation are clamped: nothing is ever read or
    // written beyond (T, U), whatever the length tensors hold
    const int Tn = min(max(lx[n], 0), T);
    const int Un = min(max(ly[n], 0), U);
    const double *units_n = units + (size_t)n * T * P * 3;
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * P * 2;
    if (blockIdx.y == 0)
        beta_sweep<K, R>(units_n, y, Tn, Un, P, betas + (size_t)n * lat, costs + n);
    else
        alpha_sweep<K, R>(units_n, y, Tn, Un, P, alphas + (size_t)n * lat);
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
