// Kernels of the log-add joiner path (ctct_simple_loss): joint = f (+) g,
// optionally normalised by den = logsumexp_v(f + g).
//
//  * units straight from f (N,T,V), g (N,U+1,V), den (N,T,U+1): the two
//    torch.gather calls of warp_ctct/__init__.py:204-215 and the
//    LOGPROBY/LOGPROBB macros of csrc/simple.cu:20-26 in one pass;
//  * the reductions of the unit gradients that csrc/binding.cpp:198-219 does
//    with ATen ops: grad_den = -sum_k, grad_g = sum_t, grad_f[...,0] = sum_u g0,
//    grad_f[...,u>=1] = g1[u] + g2[u-1];
//  * the backward of the two gathers: scatter-add of those compact gradients
//    into the dense (N,T,V) and (N,U+1,V) tensors, scaled by grad_output[n]
//    (SimpleCTCTLoss.backward, warp_ctct/__init__.py:76-85).
#include "device_utils.h"
#include "launch.h"
#include "logmm_finish.h"
#include "unit_grad.h"

namespace wctct {

namespace {

constexpr int kBlock = 256;

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return min(max(v, lo), hi); }

// One thread per cell (t,u) of sample blockIdx.y; the 64 lanes of a wavefront
// are 64 consecutive contexts of one frame (P is a multiple of 64).  The value
// f[t, y[u]] serves two cells, as the next label of (t,u) and as the current
// label of (t,u+1): every lane reads it once and hands it to its neighbour
// (one scattered read of f per cell instead of two).
// DEFERRED: den is not there yet.  The log-matmul that produces it has left its
// last pass (the sum over the slabs of the reduction, LogmmDeferred) to this
// kernel: every cell u <= ly of a live frame computes its den[t,u], writes it
// (the backward reads all of them), and context 0 writes the frame's fmax.
// only_if (may be null): return at once while *only_if is 0 (the fall-back run
// behind the lattices in the linear domain).

// 2^(log2 unit): a unit as the linear sweeps take it; log 0 is 0.
__device__ __forceinline__ double unit_lin(double log2_unit) {
    if (log2_unit == neg_inf()) return 0.0;
    // 2^x = 2^floor(x) * 2^frac, the second factor on the fp32 transcendental unit
    // (relative error ~1e-7 per unit, without bias: a product of a thousand
    // units is off by a few 1e-6, the cost by as much in absolute terms)
    const double fl = __builtin_floor(log2_unit);
    const double clamped = __builtin_fmin(__builtin_fmax(fl, -2000.0), 2000.0);
    return __builtin_amdgcn_ldexp((double)exp2_hw((float)(log2_unit - fl)), (int)clamped);
}

template <bool DEFERRED>
__global__ __launch_bounds__(kBlock) void simple_gather_units_kernel(
    const float *__restrict__ f, const float *__restrict__ g, float *__restrict__ den,
    const int *__restrict__ ys, const int *__restrict__ lx, const int *__restrict__ ly,
    double *__restrict__ units, int T, int U, int V, int P, const RelaySlots relay,
    const LogmmDeferred deferred, float *__restrict__ fmax, unsigned *__restrict__ counter,
    unsigned *__restrict__ status, const unsigned *__restrict__ only_if) {
    if (only_if && *only_if == 0u) return;
    relay_clear_share(relay);
    // (the arrival counter of the lattice kernel's cost reduction, if there is one)
    if (counter && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *counter = 0u;
    const int U1 = U + 1;
    const int n = blockIdx.y;
    const int cell = blockIdx.x * kBlock + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int t = cell / P, u = cell - t * P;      // t is the same for the whole wavefront
    const int Tn = clampi(lx[n], 0, T), Un = clampi(ly[n], 0, U);
    if (t >= Tn) {                                 // (covers cell >= T * P)
        if (DEFERRED && t < T && u == 0) fmax[(size_t)n * T + t] = -__builtin_huge_valf();
        return;
    }
    const float *fr = f + ((size_t)n * T + t) * V;
    float den_tu = 0.0f;
    if (DEFERRED) {
        if (u <= Un) {
            float row_max;
            den_tu = logmm_finish_cell(deferred, n, t, u, fr, 1, g + ((size_t)n * U1 + u) * V, 1, V,
                                       row_max);
            den[((size_t)n * T + t) * U1 + u] = den_tu;
            if (u == 0) fmax[(size_t)n * T + t] = row_max;
        }
    } else if (den && u <= Un) {
        den_tu = den[((size_t)n * T + t) * U1 + u];
    }
    const bool live = u <= Un && !outside_band(t, u, Tn, Un);
    const int *y = ys + (size_t)n * U;
    // the next label's column: wanted by this cell or by the cell of context u+1
    const bool has2 = u < Un;
    const int c2 = has2 ? label_column(y[u], V, status) : 0;
    const bool wanted = has2 && (live || !outside_band(t, u + 1, Tn, Un));
    const float f2 = wanted ? fr[c2] : 0.0f;
    float f1 = __shfl_up(f2, 1, 64);
    const int c1 = (u >= 1 && u <= Un) ? clampi(y[u - 1], 0, V - 1) : 0;
    if (lane == 0 && live && u >= 1) f1 = fr[c1];  // the neighbour is in another wavefront
    double *o = units + (((size_t)n * T + t) * P + u) * 3;
    // padding context of a live frame, or a cell outside the band of complete
    // alignments (its units cannot influence costs or gradients): neutral units
    if (!live) {
        o[0] = 0.0;
        o[1] = 0.0;
        o[2] = neg_inf();
        return;
    }
    const float *gr = g + ((size_t)n * U1 + u) * V;
    const double d = (double)den_tu;
    const double b = (double)fr[0] + (double)gr[0] - d;
    double cur = b, nxt = neg_inf();
    if (u >= 1) cur = (double)f1 + (double)gr[c1] - d;
    if (has2) nxt = ((double)f2 + (double)gr[c2] - d) * kLog2e;
    // a NaN unit (NaN in f, g or den) enters the lattice as log 0 and is reported
    if (b != b || cur != cur || nxt != nxt) {
        if (status) atomicOr(status, kStatusNanInput);
        o[0] = (b != b) ? neg_inf() : b * kLog2e;
        o[1] = (cur != cur) ? neg_inf() : cur * kLog2e;
        o[2] = (nxt != nxt) ? neg_inf() : nxt;
        return;
    }
    o[0] = b * kLog2e;
    o[1] = cur * kLog2e;
    o[2] = nxt;
}

// The units for the sweeps in the linear domain (lattice_lin.hip): one thread per
// (frame, column); lanes 1..62 of a wavefront are the contexts 62 w .. 62 w + 61,
// lane 0 and lane 63 the columns through which the wavefronts below / above hand
// their boundary values over.  A context's cell holds {blank, label, next label}
// as linear factors.  Cells of the columns in between: lane 0 {1, 0, E}, lane 63
// {0, 1, E}, E = "nothing there yet" where a wavefront will write, 0 where none
// does; the 0 beside it takes the sender's scale.  den, fmax, counter, status: as
// in simple_gather_units_kernel; *flag is lowered.
template <bool DEFERRED>
__global__ __launch_bounds__(kBlock) void simple_gather_units_lin_kernel(
    const float *__restrict__ f, const float *__restrict__ g, float *__restrict__ den,
    const int *__restrict__ ys, const int *__restrict__ lx, const int *__restrict__ ly,
    double *__restrict__ units, int T, int U, int V, int Pl, const LogmmDeferred deferred,
    float *__restrict__ fmax, unsigned *__restrict__ counter, unsigned *__restrict__ status,
    unsigned *__restrict__ flag) {
    if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
        if (counter) *counter = 0u;
        *flag = 0u;
    }
    const int U1 = U + 1;
    const int n = blockIdx.y;
    const int cell = blockIdx.x * kBlock + threadIdx.x;
    const int lane = threadIdx.x & 63;
    const int t = cell / Pl, col = cell - t * Pl;   // t is the same for the whole wavefront
    const int w = col >> 6;
    const int u = w * kLinReal + lane - 1;
    const int Tn = clampi(lx[n], 0, T), Un = clampi(ly[n], 0, U);
    if (t >= Tn) {                                  // (covers cell >= T * Pl)
        if (DEFERRED && t < T && col == 0) fmax[(size_t)n * T + t] = -__builtin_huge_valf();
        return;
    }
    const float *fr = f + ((size_t)n * T + t) * V;
    const bool real = lane >= 1 && lane <= kLinReal;
    const bool in = real && u <= Un;
    float den_tu = 0.0f;
    if (DEFERRED) {
        if (in) {
            float row_max;
            den_tu = logmm_finish_cell(deferred, n, t, u, fr, 1, g + ((size_t)n * U1 + u) * V, 1, V,
                                       row_max);
            den[((size_t)n * T + t) * U1 + u] = den_tu;
            if (u == 0) fmax[(size_t)n * T + t] = row_max;
        }
    } else if (den && in) {
        den_tu = den[((size_t)n * T + t) * U1 + u];
    }
    const bool live = in && !outside_band(t, u, Tn, Un);
    const int *y = ys + (size_t)n * U;
    // the next label's column: wanted by this cell or by the cell of context u+1
    const bool has2 = real && u < Un;
    const int c2 = has2 ? label_column(y[u], V, status) : 0;
    const bool wanted = has2 && (live || !outside_band(t, u + 1, Tn, Un));
    const float f2 = wanted ? fr[c2] : 0.0f;
    float f1 = __shfl_up(f2, 1, 64);
    const int c1 = (in && u >= 1) ? clampi(y[u - 1], 0, V - 1) : 0;
    if (lane == 1 && live && u >= 1) f1 = fr[c1];   // the neighbour is in another wavefront
    // Padding, and cells outside the band of complete alignments (their units
    // cannot influence costs or gradients): all 0.  The mass of alignments that
    // cannot be completed is then gone where it leaves the band; with factors of
    // 1 it would stay there undiminished while the mass that counts shrinks with
    // every frame, and the scale of its wavefront would follow it.
    double v0 = 0.0, v1 = 0.0, v2 = 0.0;
    if (live) {
        const float *gr = g + ((size_t)n * U1 + u) * V;
        const double d = (double)den_tu;
        const double b = (double)fr[0] + (double)gr[0] - d;
        double cur = b, nxt = neg_inf();
        if (u >= 1) cur = (double)f1 + (double)gr[c1] - d;
        if (has2) nxt = ((double)f2 + (double)gr[c2] - d) * kLog2e;
        // a NaN unit (NaN in f, g or den) enters the lattice as log 0 and is reported
        if (b != b || cur != cur || nxt != nxt) {
            if (status) atomicOr(status, kStatusNanInput);
        }
        v0 = unit_lin((b != b) ? neg_inf() : b * kLog2e);
        v1 = unit_lin((cur != cur) ? neg_inf() : cur * kLog2e);
        v2 = unit_lin((nxt != nxt) ? neg_inf() : nxt);
    }
    const double empty = __longlong_as_double((long long)kRelayEmpty);
    if (lane == 0) {
        v0 = 1.0, v1 = 0.0;
        v2 = (w >= 1 && w * kLinReal <= Un) ? empty : 0.0;
    } else if (lane == 63) {
        v0 = 0.0, v1 = 1.0;
        v2 = ((w + 1) * kLinReal <= Un) ? empty : 0.0;
    }
    double *o = units + (((size_t)n * T + t) * Pl + col) * kLinUnit;
    o[0] = v0;
    o[1] = v1;
    o[2] = v2;
}

// Per frame: grad_den[t,u] = -(g0+g1+g2), grad_f[t,u>=1] = g1[t,u] + g2[t,u-1],
// grad_f[t,0] = sum_u g0[t,u].  One wavefront per (n,t); unit gradients are zero
// in padding already.
__global__ __launch_bounds__(kBlock) void simple_reduce_frames_kernel(
    const float *__restrict__ ug, float *__restrict__ grad_f, float *__restrict__ grad_den, int T,
    int U) {
    const int U1 = U + 1;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int t = blockIdx.x * 4 + wave;
    const int n = blockIdx.y;
    if (t >= T) return;
    const float *row = ug + ((size_t)n * T + t) * U1 * 3;
    float *gf = grad_f + ((size_t)n * T + t) * U1;
    float blank = 0.0f;
    for (int u = lane; u < U1; u += 64) {
        const float g0 = row[u * 3], g1 = row[u * 3 + 1], g2 = row[u * 3 + 2];
        blank += g0;
        if (grad_den) grad_den[((size_t)n * T + t) * U1 + u] = -(g0 + g1 + g2);
        if (u >= 1) gf[u] = g1 + row[(u - 1) * 3 + 2];
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) blank += __shfl_xor(blank, off, 64);
    if (lane == 0) gf[0] = blank;
}

// Per context: grad_g[u,k] = sum_t g_k[t,u].  One wavefront per (n,u).
__global__ __launch_bounds__(kBlock) void simple_reduce_contexts_kernel(
    const float *__restrict__ ug, float *__restrict__ grad_g, int T, int U) {
    const int U1 = U + 1;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int u = blockIdx.x * 4 + wave;
    const int n = blockIdx.y;
    if (u >= U1) return;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
    for (int t = lane; t < T; t += 64) {
        const float *p = ug + (((size_t)n * T + t) * U1 + u) * 3;
        s0 += p[0];
        s1 += p[1];
        s2 += p[2];
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        s0 += __shfl_xor(s0, off, 64);
        s1 += __shfl_xor(s1, off, 64);
        s2 += __shfl_xor(s2, off, 64);
    }
    if (lane == 0) {
        float *o = grad_g + ((size_t)n * U1 + u) * 3;
        o[0] = s0;
        o[1] = s1;
        o[2] = s2;
    }
}

// Unit gradients and their reductions in one pass over the lattices: what
// unit_grads_kernel + simple_reduce_frames_kernel + simple_reduce_contexts_kernel
// produce, without the (N,T,U+1,3) tensor in between.  One workgroup per
// (n, block of kFramesPerBlock frames), one thread per context:
//   grad_den[t,u] = -(g0+g1+g2),  grad_f[t,u>=1] = g1[t,u] + g2[t,u-1],
//   grad_f[t,0] = sum_u g0[t,u]                          (per frame)
//   partial[n,block,u,k] = sum over the block's frames of g_k[t,u]
// and simple_sum_partials_kernel adds the blocks up in a fixed order.
constexpr int kFramesPerBlock = 8;
// how far the posteriors of a frame may be from adding up to 1 before the
// linear lattices are given up (their own rounding stays below 1e-6)
constexpr float kPosteriorSlack = 2e-5f;

// LIN: the lattices are those of lattice_lin.hip (linear domain; `scales` as
// launch_lattice_lin describes them), and the kernel checks what it hands out:
// the posteriors of every frame add up to 1 (every alignment consumes exactly
// one unit per frame; lost mass and anything not finite fail that), and no unit
// is so large that a chunk of frames could overflow.  Where a check fails it raises *flag, and the
// log-domain kernels launched behind it (only_if) compute the batch again.
// only_if (may be null): return at once while *only_if is 0.
template <bool LIN>
__global__ __launch_bounds__(512) void simple_grads_kernel(
    const double *__restrict__ units, const int *__restrict__ ys, const int *__restrict__ lx,
    const int *__restrict__ ly, const double *__restrict__ alphas,
    const double *__restrict__ betas, float *__restrict__ grad_f, float *__restrict__ grad_den,
    float *__restrict__ partial, int T, int U, int P, const int *__restrict__ scales,
    unsigned *__restrict__ flag, const unsigned *__restrict__ only_if) {
    if (only_if && *only_if == 0u) return;
    constexpr int F = kFramesPerBlock;
    __shared__ float s_g2[F][512];
    __shared__ float s_blank[F][8];
    __shared__ float s_all[F][8];
    const int U1 = U + 1;
    const int n = blockIdx.y, u = threadIdx.x;
    const int lane = u & 63, wave = u >> 6, waves = P >> 6;
    const int Tn = clampi(lx[n], 0, T), Un = clampi(ly[n], 0, U);
    // columns per row of the work buffers (LIN: those of the linear sweeps)
    const int Pw = LIN ? lin_padded(U) : P;
    const size_t lat = (size_t)(T + 1) * Pw * 2;
    const double *units_n = units + (size_t)n * T * Pw * (LIN ? kLinUnit : 3);
    const double *alpha_n = alphas + (size_t)n * lat, *beta_n = betas + (size_t)n * lat;
    // LIN: rows of high words (lattice_lin.hip)
    const unsigned *alpha_w = reinterpret_cast<const unsigned *>(alphas) + (size_t)n * lat;
    const unsigned *beta_w = reinterpret_cast<const unsigned *>(betas) + (size_t)n * lat;
    const int *y = ys + (size_t)n * U;
    const int t_begin = blockIdx.x * F;
    // LIN: the scales of this context's wavefront (of the sweeps) and of the next
    // context's, and the lattice's total mass: beta(0, state 0)
    const int chunks1 = lin_chunks(T) + 1;
    const int *sc_beta = nullptr, *sc_beta_next = nullptr, *sc_alpha = nullptr;
    double inv_ll = 0.0;
    int s_ll = 0;
    if (LIN) {
        const int lw = lin_waves(U);
        const int w_own = min(u / kLinReal, lw - 1), w_next = min((u + 1) / kLinReal, lw - 1);
        sc_beta = scales + (((size_t)n * 2 + 0) * lw + w_own) * chunks1;
        sc_beta_next = scales + (((size_t)n * 2 + 0) * lw + w_next) * chunks1;
        sc_alpha = scales + (((size_t)n * 2 + 1) * lw + w_own) * chunks1;
        const double ll = lin_state(beta_w[lin_column(0) * 2 + 1]);
        const int ex = (ll > 0.0 && ll < __builtin_huge_val()) ? __builtin_amdgcn_frexp_exp(ll) : 0;
        inv_ll = 1.0 / __builtin_amdgcn_ldexp(ll, -ex);   // (0 or inf: NaN below, caught by the check)
        // row 0 of beta was stored by step Tn - 1 of context 0's wavefront
        s_ll = ex + scales[(((size_t)n * 2 + 0) * lw + 0) * chunks1 + (Tn > 0 ? 1 + (Tn - 1) / kLinChunk : 0)];
    }
    // all frames of the block first (their loads are independent), then one exchange
    UnitGrad g[F];
    float a0 = 0.0f, a1 = 0.0f, a2 = 0.0f;
    bool bad_unit = false;
#pragma unroll
    for (int f = 0; f < F; ++f) {
        const int t = t_begin + f;
        g[f] = UnitGrad{0.0f, 0.0f, 0.0f};
        // padding and cells outside the band of complete alignments: exactly zero
        if (t < Tn && u <= Un && !outside_band(t, u, Tn, Un)) {
            if (LIN) {
                // row t of alpha: step t - 1; row t + 1 of beta: step Tn - 2 - t
                const int ia = t > 0 ? 1 + (t - 1) / kLinChunk : 0;
                const int ib = t + 1 < Tn ? 1 + (Tn - 2 - t) / kLinChunk : 0;
                bool bad;
                g[f] = unit_grad_cell_lin(units_n, alpha_w, beta_w, y, t, u, Un, Pw, sc_alpha[ia],
                                          sc_beta[ib], sc_beta_next[ib], inv_ll, s_ll, bad);
                bad_unit = bad_unit || bad;
            } else {
                g[f] = unit_grad_cell(units_n, alpha_n, beta_n, y, t, u, Un, P);
            }
        }
        a0 += g[f].g0;
        a1 += g[f].g1;
        a2 += g[f].g2;
    }
#pragma unroll
    for (int f = 0; f < F; ++f) {
        float blank = g[f].g0;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) blank += __shfl_xor(blank, off, 64);
        s_g2[f][u] = g[f].g2;
        if (lane == 0) s_blank[f][wave] = blank;
        // The check, on every frame: mass that the linear sweeps have lost is
        // missing from every later frame's posteriors (alpha) or shows in them as a
        // surplus (beta: the total they are divided by came out too small); a
        // product that left the range of a double on the way to one posterior
        // shows in that frame only.
        if (LIN) {
            float all = g[f].g0 + g[f].g1 + g[f].g2;
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) all += __shfl_xor(all, off, 64);
            if (lane == 0) s_all[f][wave] = all;
        }
    }
    __syncthreads();
    if (LIN) {
        if (u < F) {
            const int t = t_begin + u;
            float all = 0.0f;
            for (int w = 0; w < waves; ++w) all += s_all[u][w];
            // (a NaN fails the comparison too)
            if (t < Tn && !(__builtin_fabsf(all + 1.0f) <= kPosteriorSlack)) atomicOr(flag, 1u);
        }
        if (__ballot(bad_unit) != 0ULL && lane == 0) atomicOr(flag, 1u);
    }
    if (u >= U1) return;
#pragma unroll
    for (int f = 0; f < F; ++f) {
        const int t = t_begin + f;
        if (t >= T) break;
        const size_t at = ((size_t)n * T + t) * U1 + u;
        if (grad_den) grad_den[at] = -(g[f].g0 + g[f].g1 + g[f].g2);
        if (u >= 1) {
            grad_f[at] = g[f].g1 + s_g2[f][u - 1];
        } else {
            float b = 0.0f;
            for (int w = 0; w < waves; ++w) b += s_blank[f][w];
            grad_f[at] = b;
        }
    }
    float *o = partial + (((size_t)n * gridDim.x + blockIdx.x) * U1 + u) * 3;
    o[0] = a0;
    o[1] = a1;
    o[2] = a2;
}

// grad_g[n,u,k] = sum over the frame blocks of partial[n,block,u,k]; one
// wavefront per (n,u), lanes over the blocks, summed in a fixed order.
__global__ __launch_bounds__(kBlock) void simple_sum_partials_kernel(
    const float *__restrict__ partial, float *__restrict__ grad_g, int blocks, int U1) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int u = blockIdx.x * 4 + wave;
    const int n = blockIdx.y;
    if (u >= U1) return;
    float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f;
    for (int b = lane; b < blocks; b += 64) {
        const float *p = partial + (((size_t)n * blocks + b) * U1 + u) * 3;
        s0 += p[0];
        s1 += p[1];
        s2 += p[2];
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        s0 += __shfl_xor(s0, off, 64);
        s1 += __shfl_xor(s1, off, 64);
        s2 += __shfl_xor(s2, off, 64);
    }
    if (lane == 0) {
        float *o = grad_g + ((size_t)n * U1 + u) * 3;
        o[0] = s0;
        o[1] = s1;
        o[2] = s2;
    }
}

// dense_f[n,t,idx(u)] += w[n] * grad_f[n,t,u],  idx = [0, y0 .. y_{U-1}]: the
// backward of f.gather (warp_ctct/__init__.py:205-208).  The same label may
// occur at several u, so the adds are atomic.  Padding holds zeros: skipped.
__device__ __forceinline__ void scatter_f_cell(
    int cell, const float *__restrict__ grad_f, const int *__restrict__ ys,
    const int *__restrict__ lx, const int *__restrict__ ly, const float *__restrict__ grad_out,
    float *__restrict__ dense_f, int T, int U, int V) {
    const int U1 = U + 1;
    const int n = blockIdx.y;
    if (cell >= T * U1) return;
    const int t = cell / U1, u = cell - t * U1;
    const int Tn = clampi(lx[n], 0, T), Un = clampi(ly[n], 0, U);
    if (t >= Tn || u > Un) return;
    // (all three loads requested before the first is looked at)
    const float gv = grad_f[((size_t)n * T + t) * U1 + u];
    const float w = grad_out ? grad_out[n] : 1.0f;
    const int col = U > 0 ? clampi(ys[(size_t)n * U + max(u - 1, 0)], 0, V - 1) : 0;   // (no labels: ys may be null)
    // cells that no complete alignment passes through hold exact zeros: no add
    if (gv == 0.0f) return;
    atomicAdd(dense_f + ((size_t)n * T + t) * V + (u == 0 ? 0 : col), w * gv);
}

__global__ __launch_bounds__(kBlock) void simple_scatter_f_kernel(
    const float *__restrict__ grad_f, const int *__restrict__ ys, const int *__restrict__ lx,
    const int *__restrict__ ly, const float *__restrict__ grad_out, float *__restrict__ dense_f,
    int T, int U, int V) {
    scatter_f_cell(blockIdx.x * kBlock + threadIdx.x, grad_f, ys, lx, ly, grad_out, dense_f, T, U, V);
}

// dense_f[n,t,:] as a whole row: zeros plus w[n] * grad_f[n,t,u] at idx(u), the
// zero-fill and the scatter-add of simple_scatter_f_kernel in one pass.  One
// workgroup per frame builds the row in LDS (repeated labels add there) and
// writes it out with full-width stores, so no element of the row is touched
// twice in memory and no partially written line is left behind.
// The rows of dense_g ride in the same launch (workgroups f_rows.. of a sample,
// one per context): zeros plus w[n] * grad_g[n,u,k] at columns 0, y[u-1], y[u].
// A row of dense_g has at most three non-zero elements, so every thread
// decides for its own columns what to store and LDS is not used.
__global__ __launch_bounds__(kBlock) void simple_dense_rows_kernel(
    const float *__restrict__ grad_f, const float *__restrict__ grad_g,
    const int *__restrict__ ys, const int *__restrict__ lx, const int *__restrict__ ly,
    const Weight weight, float *__restrict__ dense_f, float *__restrict__ dense_g,
    int T, int U, int V, int f_rows) {
    extern __shared__ __attribute__((aligned(16))) float row[];   // V floats (f rows only)
    typedef float v4f __attribute__((ext_vector_type(4)));
    const int U1 = U + 1;
    const int n = blockIdx.y;
    const int Un = clampi(ly[n], 0, U);
    const float w = sample_weight(weight, n, lx[n]);
    if ((int)blockIdx.x >= f_rows) {
        const int u = blockIdx.x - f_rows;
        float *out = dense_g + ((size_t)n * U1 + u) * V;
        // entry k of the row: column and value; a column of -1 takes no part
        int col[3] = {-1, -1, -1};
        float val[3] = {0.0f, 0.0f, 0.0f};
        if (u <= Un) {
            const float *gg = grad_g + ((size_t)n * U1 + u) * 3;
            col[0] = 0, val[0] = w * gg[0];
            if (u >= 1) col[1] = clampi(ys[(size_t)n * U + u - 1], 0, V - 1), val[1] = w * gg[1];
            if (u < Un) col[2] = clampi(ys[(size_t)n * U + u], 0, V - 1), val[2] = w * gg[2];
        }
        if ((V & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
            for (int k = threadIdx.x * 4; k < V; k += kBlock * 4) {
                v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                for (int e = 0; e < 3; ++e)
                    if ((col[e] >> 2) == (k >> 2)) {   // (-1 >> 2 is -1: never a vector of the row)
#pragma unroll
                        for (int q = 0; q < 4; ++q) v[q] += ((col[e] & 3) == q) ? val[e] : 0.0f;
                    }
                __builtin_nontemporal_store(v, reinterpret_cast<v4f *>(out + k));
            }
        } else {
            for (int k = threadIdx.x; k < V; k += kBlock) {
                float v = 0.0f;
#pragma unroll
                for (int e = 0; e < 3; ++e) v += (col[e] == k) ? val[e] : 0.0f;
                out[k] = v;
            }
        }
        return;
    }
    const int t = blockIdx.x;
    const int Tn = clampi(lx[n], 0, T);
    float *out = dense_f + ((size_t)n * T + t) * V;
    const bool live = t < Tn;
    if (live) {
        for (int k = threadIdx.x; k < V; k += kBlock) row[k] = 0.0f;
        __syncthreads();
        for (int u = threadIdx.x; u <= Un; u += kBlock) {
            const float gv = grad_f[((size_t)n * T + t) * U1 + u];
            if (gv == 0.0f) continue;
            const int col = (u == 0) ? 0 : clampi(ys[(size_t)n * U + u - 1], 0, V - 1);
            atomicAdd(row + col, w * gv);
        }
        __syncthreads();
    }
    if ((V & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
        const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
        for (int k = threadIdx.x * 4; k < V; k += kBlock * 4)
            // (non-temporal: nothing of this path reads the rows again, and their
            // write-back would run into the next step's gather)
            __builtin_nontemporal_store(live ? *reinterpret_cast<const v4f *>(row + k) : zero,
                                        reinterpret_cast<v4f *>(out + k));
    } else {
        for (int k = threadIdx.x; k < V; k += kBlock) out[k] = live ? row[k] : 0.0f;
    }
}

// dense_g[n,u,{0,y[u-1],y[u]}] += w[n] * grad_g[n,u,k]: backward of g.gather
// (warp_ctct/__init__.py:211-215).  One thread per (n,u,k).
__device__ __forceinline__ void scatter_g_entry(
    int e, const float *__restrict__ grad_g, const int *__restrict__ ys,
    const int *__restrict__ ly, const float *__restrict__ grad_out, float *__restrict__ dense_g,
    int U, int V) {
    const int U1 = U + 1;
    const int n = blockIdx.y;
    if (e >= U1 * 3) return;
    const int u = e / 3, k = e - u * 3;
    const int Un = clampi(ly[n], 0, U);
    if (u > Un || (k == 1 && u == 0) || (k == 2 && u >= Un)) return;
    const float w = grad_out ? grad_out[n] : 1.0f;
    int col = 0;
    if (k == 1) col = clampi(ys[(size_t)n * U + u - 1], 0, V - 1);
    if (k == 2) col = clampi(ys[(size_t)n * U + u], 0, V - 1);
    atomicAdd(dense_g + ((size_t)n * U1 + u) * V + col, w * grad_g[((size_t)n * U1 + u) * 3 + k]);
}

__global__ __launch_bounds__(kBlock) void simple_scatter_g_kernel(
    const float *__restrict__ grad_g, const int *__restrict__ ys, const int *__restrict__ ly,
    const float *__restrict__ grad_out, float *__restrict__ dense_g, int U, int V) {
    scatter_g_entry(blockIdx.x * kBlock + threadIdx.x, grad_g, ys, ly, grad_out, dense_g, U, V);
}

// Both scatters in one launch: the first f_blocks workgroups of a sample take
// the cells of f, the rest the entries of g.
__global__ __launch_bounds__(kBlock) void simple_scatter_fg_kernel(
    const float *__restrict__ grad_f, const float *__restrict__ grad_g,
    const int *__restrict__ ys, const int *__restrict__ lx, const int *__restrict__ ly,
    const float *__restrict__ grad_out, float *__restrict__ dense_f, float *__restrict__ dense_g,
    int T, int U, int V, int f_blocks) {
    if ((int)blockIdx.x < f_blocks)
        scatter_f_cell(blockIdx.x * kBlock + threadIdx.x, grad_f, ys, lx, ly, grad_out, dense_f, T,
                       U, V);
    else
        scatter_g_entry((blockIdx.x - f_blocks) * kBlock + threadIdx.x, grad_g, ys, ly, grad_out,
                        dense_g, U, V);
}

// weights[n] = grad_out[n * stride] * scale (/ lx[n]): what the kernels that take a
// plain array of per-sample weights read after a reduction over the batch
__global__ __launch_bounds__(kBlock) void sample_weights_kernel(const Weight weight,
                                                                const int *__restrict__ lx,
                                                                float *__restrict__ weights, int N) {
    const int n = blockIdx.x * kBlock + threadIdx.x;
    if (n < N) weights[n] = sample_weight(weight, n, lx[n]);
}

inline dim3 cell_grid(int N, int T, int U) {
    const long cells = (long)T * (U + 1);
    return dim3((unsigned)((cells + kBlock - 1) / kBlock), (unsigned)N);
}

}  // namespace

hipError_t launch_simple_gather_units(const float *f, const float *g, float *den, const int *ys,
                                      const int *lx, const int *ly, double *units, int N, int T,
                                      int U, int V, const RelaySlots &relay,
                                      const LogmmDeferred &deferred, float *fmax,
                                      unsigned *counter, hipStream_t stream,
                                      const unsigned *only_if) {
    const int P = padded_contexts(U);
    const long cells = (long)T * P;
    const dim3 grid((unsigned)((cells + kBlock - 1) / kBlock), (unsigned)N);
    if (deferred.partial && (!den || !fmax || deferred.splits < 1 || deferred.splits > 8 ||
                             deferred.B != N || deferred.Nn != U + 1))
        return hipErrorInvalidValue;
    unsigned *status = device_status_word();
    if (deferred.partial)
        TIMED_LAUNCH(simple_gather_units_kernel<true>, grid, dim3(kBlock), 0, stream, f, g, den, ys, lx,
                     ly, units, T, U, V, P, relay, deferred, fmax, counter, status, only_if);
    else
        TIMED_LAUNCH(simple_gather_units_kernel<false>, grid, dim3(kBlock), 0, stream, f, g, den, ys, lx,
                     ly, units, T, U, V, P, relay, deferred, fmax, counter, status, only_if);
    return hipGetLastError();
}

hipError_t launch_simple_gather_units_lin(const float *f, const float *g, float *den, const int *ys,
                                          const int *lx, const int *ly, double *units, int N, int T,
                                          int U, int V, const LogmmDeferred &deferred, float *fmax,
                                          unsigned *counter, unsigned *flag, hipStream_t stream) {
    if (!simple_grads_lin_applies(T, U) || !flag) return hipErrorInvalidValue;
    const int Pl = lin_padded(U);
    const long cells = (long)T * Pl;
    const dim3 grid((unsigned)((cells + kBlock - 1) / kBlock), (unsigned)N);
    if (deferred.partial && (!den || !fmax || deferred.splits < 1 || deferred.splits > 8 ||
                             deferred.B != N || deferred.Nn != U + 1))
        return hipErrorInvalidValue;
    unsigned *status = device_status_word();
    if (deferred.partial)
        TIMED_LAUNCH(simple_gather_units_lin_kernel<true>, grid, dim3(kBlock), 0, stream, f, g, den, ys,
                     lx, ly, units, T, U, V, Pl, deferred, fmax, counter, status, flag);
    else
        TIMED_LAUNCH(simple_gather_units_lin_kernel<false>, grid, dim3(kBlock), 0, stream, f, g, den, ys,
                     lx, ly, units, T, U, V, Pl, deferred, fmax, counter, status, flag);
    return hipGetLastError();
}

// The first half of launch_simple_grads for lattices in the linear domain (see
// simple_grads_kernel<true>): grad_f, grad_den and the partial sums of grad_g;
// the caller adds those up with launch_simple_grads' second half afterwards.
bool simple_grads_lin_applies(int T, int U) {
    // (the linear sweeps address a sample's units through 32-bit byte offsets)
    return T > 0 && padded_contexts(U) <= 512 &&
           (size_t)T * lin_padded(U) * kLinUnit * sizeof(double) < (1ULL << 31);
}

hipError_t launch_simple_grads_lin(const double *units, const int *ys, const int *lx, const int *ly,
                                   const double *alphas, const double *betas, const int *scales,
                                   float *partial, float *grad_f, float *grad_den, int N, int T,
                                   int U, unsigned *flag, hipStream_t stream) {
    if (!simple_grads_lin_applies(T, U) || !scales || !flag) return hipErrorInvalidValue;
    const int P = padded_contexts(U);
    const int blocks = (T + kFramesPerBlock - 1) / kFramesPerBlock;
    TIMED_LAUNCH(simple_grads_kernel<true>, dim3(blocks, N), dim3(P), 0, stream, units, ys, lx, ly,
                 alphas, betas, grad_f, grad_den, partial, T, U, P, scales, flag, nullptr);
    return hipGetLastError();
}

hipError_t launch_simple_grads(const double *units, const int *ys, const int *lx, const int *ly,
                               const double *alphas, const double *betas, float *partial,
                               float *grad_f, float *grad_g, float *grad_den, int N, int T, int U,
                               hipStream_t stream, const unsigned *only_if) {
    const int P = padded_contexts(U);
    if (P > 512) {
        if (only_if) return hipErrorInvalidValue;
        // more contexts than one workgroup of the fused kernel holds: unit
        // gradients into `partial` (it has room for all of them), then the two
        // reductions over them
        hipError_t e = launch_unit_grads(units, ys, lx, ly, alphas, betas, partial, N, T, U, stream);
        if (e != hipSuccess) return e;
        return launch_simple_reduce(partial, grad_f, grad_g, grad_den, N, T, U, stream);
    }
    const int blocks = (T + kFramesPerBlock - 1) / kFramesPerBlock;
    if (T > 0) {
        TIMED_LAUNCH(simple_grads_kernel<false>, dim3(blocks, N), dim3(P), 0, stream, units, ys, lx,
                           ly, alphas, betas, grad_f, grad_den, partial, T, U, P, nullptr, nullptr,
                           only_if);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    TIMED_LAUNCH(simple_sum_partials_kernel, dim3((U + 1 + 3) / 4, N), dim3(kBlock), 0,
                       stream, partial, grad_g, blocks, U + 1);
    return hipGetLastError();
}

hipError_t launch_simple_reduce(const float *unit_grads, float *grad_f, float *grad_g,
                                float *grad_den, int N, int T, int U, hipStream_t stream) {
    TIMED_LAUNCH(simple_reduce_frames_kernel, dim3((T + 3) / 4, N), dim3(kBlock), 0, stream,
                       unit_grads, grad_f, grad_den, T, U);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    TIMED_LAUNCH(simple_reduce_contexts_kernel, dim3((U + 1 + 3) / 4, N), dim3(kBlock), 0,
                       stream, unit_grads, grad_g, T, U);
    return hipGetLastError();
}

bool simple_dense_rows_fit(int V) { return (size_t)V * sizeof(float) <= 64 * 1024; }

// Either dense pointer may be null: its rows are then left out of the launch.
hipError_t launch_simple_dense_rows(const float *grad_f, const float *grad_g, const int *ys,
                                    const int *lx, const int *ly, const Weight &weight,
                                    float *dense_f, float *dense_g, int N, int T, int U, int V,
                                    hipStream_t stream) {
    const int f_rows = dense_f ? T : 0, g_rows = dense_g ? U + 1 : 0;
    if (N == 0 || f_rows + g_rows == 0) return hipSuccess;
    TIMED_LAUNCH(simple_dense_rows_kernel, dim3(f_rows + g_rows, N), dim3(kBlock),
                 f_rows ? (size_t)V * sizeof(float) : 0, stream, grad_f, grad_g, ys, lx, ly,
                 weight, dense_f, dense_g, T, U, V, f_rows);
    return hipGetLastError();
}

hipError_t launch_sample_weights(const Weight &weight, const int *lx, float *weights, int N,
                                 hipStream_t stream) {
    if (N == 0) return hipSuccess;
    TIMED_LAUNCH(sample_weights_kernel, dim3((N + kBlock - 1) / kBlock), dim3(kBlock), 0, stream,
                 weight, lx, weights, N);
    return hipGetLastError();
}

hipError_t launch_simple_scatter(const float *grad_f, const float *grad_g, const int *ys,
                                 const int *lx, const int *ly, const float *grad_out,
                                 float *dense_f, float *dense_g, int N, int T, int U, int V,
                                 hipStream_t stream) {
    if (dense_f && dense_g) {
        const dim3 fg = cell_grid(N, T, U);
        const unsigned g_blocks = ((U + 1) * 3 + kBlock - 1) / kBlock;
        TIMED_LAUNCH(simple_scatter_fg_kernel, dim3(fg.x + g_blocks, N), dim3(kBlock), 0, stream,
                     grad_f, grad_g, ys, lx, ly, grad_out, dense_f, dense_g, T, U, V, (int)fg.x);
        return hipGetLastError();
    }
    if (dense_f) {
        TIMED_LAUNCH(simple_scatter_f_kernel, cell_grid(N, T, U), dim3(kBlock), 0, stream,
                           grad_f, ys, lx, ly, grad_out, dense_f, T, U, V);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (dense_g) {
        TIMED_LAUNCH(simple_scatter_g_kernel, dim3(((U + 1) * 3 + kBlock - 1) / kBlock, N),
                           dim3(kBlock), 0, stream, grad_g, ys, ly, grad_out, dense_g, U, V);
        return hipGetLastError();
    }
    return hipSuccess;
}

}  // namespace wctct
