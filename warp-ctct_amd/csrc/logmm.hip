// Log-semiring matrix product and its backward on gfx950:
//     res[b,i,j] = log sum_k exp(lhs[b,i,k] + rhs[b,k,j])
// (csrc/logmatmul.cu:44-146 of the reference; all-(-inf) rows give -inf,
// :142-144), and
//     grad_lhs[b,i,k] = sum_j go[b,i,j] * exp(lhs[b,i,k] + rhs[b,k,j] - res[b,i,j])
//     grad_rhs[b,k,j] = sum_i go[b,i,j] * exp(lhs[b,i,k] + rhs[b,k,j] - res[b,i,j])
// which is what the reference's log_matmul_backward (csrc/binding.cpp:247-324)
// evaluates through four more log-matmuls on the positive and negative parts
// of grad_out; here the sum is taken directly, signed, in one pass.
//
// The reference launches one block per output element and evaluates two
// exponentials per term.  Here every operand row is shifted by its own
// maximum m and exponentiated ONCE while it is staged in LDS,
//     E_l[i,k] = exp(lhs[i,k] - ml[i]),   E_r[k,j] = exp(rhs[k,j] - mr[j]),
// all in [0,1], and the contraction becomes a plain fp32 GEMM on the FMA
// units: 64x64 output tile per workgroup, 4x4 per thread, operands read from
// LDS as 16-byte vectors; the next chunk of the reduction is fetched into
// registers while the current one is multiplied (two LDS buffers, one barrier
// per chunk).
//     res[i,j]      = ml[i] + mr[j] + log(sum_k E_l[i,k] E_r[k,j])
//     grad_lhs[i,k] = E_l[i,k] * sum_j C[i,j] E_r[k,j],
//     C[i,j]        = go[i,j] * exp(ml[i] + mr[j] - res[i,j])     (likewise rhs)
// The shift cannot overflow.  It can underflow when the maxima of a row and a
// column sit at far-apart k: an output whose shifted sum falls below 2^-60 is
// recomputed exactly with its own maximum, and in the backward a pair (i,j)
// whose C would exceed 2^60 is left out of the GEMM and added by an exact
// per-term pass (taken only by tiles that contain such a pair).  Results never
// depend on the shift beyond fp32 rounding.
#include "device_utils.h"
#include "launch.h"

namespace wctct {

namespace {

constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kLn2F = 0.6931471805599453f;
constexpr float kTiny = 8.6736174e-19f;   // 2^-60
constexpr float kMaxShiftLog2 = 60.0f;

__device__ __forceinline__ float neg_inf_f() { return -__builtin_huge_valf(); }
__device__ __forceinline__ float finite_or_zero(float m) { return m == neg_inf_f() ? 0.0f : m; }

// ---- maxima over the reduction dimension -----------------------------------
// out[b, r] = max_k x[b*sb + r*sr + k*sk], one wavefront per (b, r).
__global__ __launch_bounds__(256) void reduce_max_kernel(const float *__restrict__ x, long sb,
                                                         long sr, long sk, int R, int K,
                                                         float *__restrict__ out) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + wave;
    const int b = blockIdx.y;
    if (r >= R) return;
    const float *p = x + (size_t)b * sb + (size_t)r * sr;
    float m = neg_inf_f();
    for (int k = lane; k < K; k += 64) m = fmaxf(m, p[(size_t)k * sk]);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) out[(size_t)b * R + r] = m;
}

// ---- shared 64x64 GEMM tile -------------------------------------------------
constexpr int TM = 64;        // outputs along the first index of the tile
constexpr int TN = 64;        // outputs along the second index
constexpr int TQ = 32;        // reduction chunk
constexpr int LD = TM + 4;    // LDS row stride (floats): 16-byte aligned rows

typedef float v4f __attribute__((ext_vector_type(4)));

// acc[a][c] += sum_q sa[q][tp*4+a] * sb[q][tk*4+c]
__device__ __forceinline__ void tile_fma(const float (*sa)[LD], const float (*sb)[LD], int tp,
                                         int tk, float (&acc)[4][4]) {
    // partial unroll: a full unroll lets the compiler hoist all 64 LDS reads and
    // costs > 350 VGPRs, i.e. one workgroup per CU
#pragma unroll 4
    for (int q = 0; q < TQ; ++q) {
        const v4f av = *reinterpret_cast<const v4f *>(&sa[q][tp * 4]);
        const v4f bv = *reinterpret_cast<const v4f *>(&sb[q][tk * 4]);
        const float a[4] = {av.x, av.y, av.z, av.w};
        const float b[4] = {bv.x, bv.y, bv.z, bv.w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
}

// ---- forward ----------------------------------------------------------------
__device__ float exact_lse(const float *lrow, long lsk, const float *rcol, long rsk, int K) {
    float mx = neg_inf_f();
    for (int k = 0; k < K; ++k) mx = fmaxf(mx, lrow[(size_t)k * lsk] + rcol[(size_t)k * rsk]);
    if (mx == neg_inf_f()) return mx;
    float s = 0.0f;
    for (int k = 0; k < K; ++k)
        s += exp2_hw((lrow[(size_t)k * lsk] + rcol[(size_t)k * rsk] - mx) * kLog2eF);
    return mx + log2_hw(s) * kLn2F;
}

// grid (ceil(M/64), ceil(Nn/64), B), block 256: thread (tp, tk) = (tid/16, tid%16)
// owns rows i0 + tp*4 .. +3 and cols j0 + tk*4 .. +3.
__global__ __launch_bounds__(256) void logmm_fwd_kernel(
    const float *__restrict__ lhs, long lsb, long lsm, long lsk, const float *__restrict__ rhs,
    long rsb, long rsk, long rsn, const float *__restrict__ lmax, const float *__restrict__ rmax,
    float *__restrict__ res, int M, int K, int Nn, const int *__restrict__ row_len,
    const int *__restrict__ col_len) {
    __shared__ __attribute__((aligned(16))) float sa[2][TQ][LD];   // E_l[k][i]
    __shared__ __attribute__((aligned(16))) float sb_[2][TQ][LD];  // E_r[k][j]
    const int b = blockIdx.z;
    const int i0 = blockIdx.x * TM, j0 = blockIdx.y * TN;
    // lengths-aware: rows >= row_len[b] and cols > col_len[b] are padding
    const int Mb = row_len ? min(max(row_len[b], 0), M) : M;
    const int Nb = col_len ? min(max(col_len[b], 0) + 1, Nn) : Nn;
    if (i0 >= Mb || j0 >= Nb) return;
    const int tid = threadIdx.x;
    const int tp = tid >> 4, tk = tid & 15;
    const float *lb = lhs + (size_t)b * lsb;
    const float *rb = rhs + (size_t)b * rsb;
    const float *lm = lmax + (size_t)b * M;
    const float *rm = rmax + (size_t)b * Nn;

    // staging assignment: element e = tid + 256*s of a (64 x TQ) slab, k fast
    // (contiguous in memory for a row-major lhs and a transposed-view rhs)
    constexpr int kStage = TM * TQ / 256;
    int sr[kStage], sq[kStage];
    float shl[kStage], shr[kStage];      // per staged row: its shift (0 if the row is all -inf)
    bool okl[kStage], okr[kStage];
#pragma unroll
    for (int s2 = 0; s2 < kStage; ++s2) {
        const int e = tid + 256 * s2;
        sr[s2] = e / TQ;
        sq[s2] = e % TQ;
        okl[s2] = (i0 + sr[s2]) < Mb;
        okr[s2] = (j0 + sr[s2]) < Nb;
        shl[s2] = okl[s2] ? finite_or_zero(lm[i0 + sr[s2]]) : 0.0f;
        shr[s2] = okr[s2] ? finite_or_zero(rm[j0 + sr[s2]]) : 0.0f;
    }
    float rl[kStage], rr[kStage];
    auto fetch = [&](int k0) {
#pragma unroll
        for (int s2 = 0; s2 < kStage; ++s2) {
            // loads are unconditional from clamped (always valid) addresses and
            // the padding is selected afterwards: no branch separates the loads
            // from the FMAs that are meant to hide their latency
            const int k = k0 + sq[s2];
            const int kc = min(k, K - 1);
            const float vl = lb[(size_t)min(i0 + sr[s2], M - 1) * lsm + (size_t)kc * lsk];
            const float vr = rb[(size_t)kc * rsk + (size_t)min(j0 + sr[s2], Nn - 1) * rsn];
            rl[s2] = (okl[s2] && k < K) ? vl : neg_inf_f();
            rr[s2] = (okr[s2] && k < K) ? vr : neg_inf_f();
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int s2 = 0; s2 < kStage; ++s2) {
            sa[buf][sq[s2]][sr[s2]] = exp2_hw((rl[s2] - shl[s2]) * kLog2eF);
            sb_[buf][sq[s2]][sr[s2]] = exp2_hw((rr[s2] - shr[s2]) * kLog2eF);
        }
    };

    float acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[a][c] = 0.0f;

    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += TQ) {
        const bool more = (k0 + TQ) < K;
        if (more) fetch(k0 + TQ);              // global loads in flight during the FMAs
        tile_fma(sa[buf], sb_[buf], tp, tk, acc);
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int i = i0 + tp * 4 + a, j = j0 + tk * 4 + c;
            if (i >= Mb || j >= Nb) continue;
            const float s = acc[a][c];
            float out;
            if (s >= kTiny && s < __builtin_huge_valf()) {
                out = lm[i] + rm[j] + log2_hw(s) * kLn2F;
            } else {
                out = exact_lse(lb + (size_t)i * lsm, lsk, rb + (size_t)j * rsn, rsk, K);
            }
            res[((size_t)b * M + i) * Nn + j] = out;
        }
    }
}

// ---- backward ----------------------------------------------------------------
// One kernel serves both operands.  "own" is the operand whose gradient is
// produced, own[b, p, k] with p = i (lhs) or j (rhs); "oth" is the other one,
// oth[b, q, k].  go/res are addressed as [b, p*gp + q*gq].
//   grad_own[b,p,k] = sum_q go[p,q] * exp(own[p,k] + oth[q,k] - res[p,q])
//                   = E_own[p,k] * sum_q C[p,q] * E_oth[q,k]
// grid (ceil(P/64), ceil(K/64), B): thread (tp, tk) owns p0+tp*4.., k0+tk*4...
__global__ __launch_bounds__(256) void logmm_bwd_kernel(
    const float *__restrict__ own, long osb, long osp, long osk, const float *__restrict__ oth,
    long tsb, long tsq, long tsk, const float *__restrict__ own_max,
    const float *__restrict__ oth_max, const float *__restrict__ go,
    const float *__restrict__ res, long gsb, long gp, long gq, float *__restrict__ grad, long dsb,
    long dsp, long dsk, int P, int Q, int K, const int *__restrict__ p_len, int p_extra,
    const int *__restrict__ q_len, int q_extra, const float *__restrict__ batch_scale) {
    __shared__ __attribute__((aligned(16))) float s_c[2][TQ][LD];   // C[q][p]
    __shared__ __attribute__((aligned(16))) float s_e[2][TQ][LD];   // E_oth[q][k]
    __shared__ int s_unsafe;
    const int b = blockIdx.z;
    const int p0 = blockIdx.x * TM, k0 = blockIdx.y * TN;
    const int Pb = p_len ? min(max(p_len[b], 0) + p_extra, P) : P;
    const int Qb = q_len ? min(max(q_len[b], 0) + q_extra, Q) : Q;
    const int tid = threadIdx.x;
    const int tp = tid >> 4, tk = tid & 15;
    const float *ob = own + (size_t)b * osb;
    const float *tb = oth + (size_t)b * tsb;
    const float *om = own_max + (size_t)b * P;
    const float *tm = oth_max + (size_t)b * Q;
    const float *gb = go + (size_t)b * gsb;
    const float *rb = res + (size_t)b * gsb;
    float *db = grad + (size_t)b * dsb;
    const float scale = batch_scale ? batch_scale[b] : 1.0f;

    float acc[4][4], fix[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[a][c] = fix[a][c] = 0.0f;
    if (tid == 0) s_unsafe = 0;
    __syncthreads();

    if (p0 < Pb) {
        constexpr int kStage = TM * TQ / 256;
        // E_oth slab (TQ x 64): k fast.  C slab (64 x TQ): q fast (contiguous for lhs).
        float re[kStage], rg[kStage], rres[kStage], rom[kStage];
        auto fetch = [&](int q0) {
#pragma unroll
            for (int s2 = 0; s2 < kStage; ++s2) {
                const int e = tid + 256 * s2;
                const int q = e / TN, c = e % TN;
                // unconditional loads from clamped addresses, padding selected after
                const int qq = q0 + q, k = k0 + c;
                const int qv = min(qq, Q - 1);
                const float ve = tb[(size_t)qv * tsq + (size_t)min(k, K - 1) * tsk] -
                                 finite_or_zero(tm[qv]);
                re[s2] = (qq < Qb && k < K) ? ve : neg_inf_f();
                const int r = e / TQ, q2 = e % TQ;
                const int p = p0 + r, qc = q0 + q2;
                const int pv = min(p, P - 1), qcv = min(qc, Q - 1);
                const bool ok = (p < Pb && qc < Qb);
                const float vres = rb[(size_t)pv * gp + (size_t)qcv * gq];
                const float vg = gb[(size_t)pv * gp + (size_t)qcv * gq] * scale;
                const float vm = om[pv] + tm[qcv];
                rres[s2] = ok ? vres : neg_inf_f();
                rg[s2] = ok ? vg : 0.0f;
                rom[s2] = ok ? vm : 0.0f;
            }
        };
        auto stash = [&](int buf) {
#pragma unroll
            for (int s2 = 0; s2 < kStage; ++s2) {
                const int e = tid + 256 * s2;
                s_e[buf][e / TN][e % TN] = exp2_hw(re[s2] * kLog2eF);
                float cv = 0.0f;
                // an all -inf row has no gradient; a zero grad_out needs no work
                if (rg[s2] != 0.0f && rres[s2] != neg_inf_f()) {
                    const float ex = (rom[s2] - rres[s2]) * kLog2eF;
                    if (ex <= kMaxShiftLog2)
                        cv = rg[s2] * exp2_hw(ex);
                    else
                        s_unsafe = 1;   // handled exactly below
                }
                s_c[buf][e % TQ][e / TQ] = cv;
            }
        };
        fetch(0);
        stash(0);
        __syncthreads();
        int buf = 0;
        for (int q0 = 0; q0 < Qb; q0 += TQ) {
            const bool more = (q0 + TQ) < Qb;
            if (more) fetch(q0 + TQ);
            tile_fma(s_c[buf], s_e[buf], tp, tk, acc);
            if (more) stash(buf ^ 1);
            __syncthreads();
            buf ^= 1;
        }
    }
    const bool slow = s_unsafe != 0;
    if (slow && p0 < Pb) {
        // exact per-term pass over the pairs the GEMM left out
        for (int a = 0; a < 4; ++a) {
            const int p = p0 + tp * 4 + a;
            if (p >= Pb) continue;
            for (int qq = 0; qq < Qb; ++qq) {
                const float rr = rb[(size_t)p * gp + (size_t)qq * gq];
                const float gv = gb[(size_t)p * gp + (size_t)qq * gq] * scale;
                if (gv == 0.0f || rr == neg_inf_f()) continue;
                if ((om[p] + tm[qq] - rr) * kLog2eF <= kMaxShiftLog2) continue;
                for (int c = 0; c < 4; ++c) {
                    const int k = k0 + tk * 4 + c;
                    if (k >= K) continue;
                    const float x = ob[(size_t)p * osp + (size_t)k * osk] +
                                    tb[(size_t)qq * tsq + (size_t)k * tsk] - rr;
                    fix[a][c] += gv * exp2_hw(x * kLog2eF);
                }
            }
        }
    }
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int p = p0 + tp * 4 + a, k = k0 + tk * 4 + c;
            if (p < P && k < K) {
                float v = 0.0f;
                if (p < Pb) {
                    const float e_own =
                        exp2_hw((ob[(size_t)p * osp + (size_t)k * osk] - finite_or_zero(om[p])) *
                                kLog2eF);
                    // acc is 0 where nothing was added: avoid 0 * inf for a +inf operand
                    v = (acc[a][c] != 0.0f ? e_own * acc[a][c] : 0.0f) + fix[a][c];
                }
                db[(size_t)p * dsp + (size_t)k * dsk] = v;
            }
        }
}

}  // namespace

hipError_t launch_reduce_max(const float *x, long sb, long sr, long sk, int B, int R, int K,
                             float *out, hipStream_t stream) {
    if (B == 0 || R == 0) return hipSuccess;
    hipLaunchKernelGGL(reduce_max_kernel, dim3((R + 3) / 4, B), dim3(256), 0, stream, x, sb, sr,
                       sk, R, K, out);
    return hipGetLastError();
}

hipError_t launch_logmm_max(const LogmmOperand &lhs, const LogmmOperand &rhs, float *lmax,
                            float *rmax, int B, int M, int K, int Nn, hipStream_t stream) {
    hipError_t e = launch_reduce_max(lhs.p, lhs.sb, lhs.s1, lhs.s2, B, M, K, lmax, stream);
    if (e != hipSuccess) return e;
    // rhs[b,k,j]: the rows to reduce are j (stride s2), k has stride s1
    return launch_reduce_max(rhs.p, rhs.sb, rhs.s2, rhs.s1, B, Nn, K, rmax, stream);
}

hipError_t launch_logmm_fwd(const LogmmOperand &lhs, const LogmmOperand &rhs, float *lmax,
                            float *rmax, float *res, int B, int M, int K, int Nn,
                            const int *row_len, const int *col_len, hipStream_t stream) {
    if (B == 0 || M == 0 || Nn == 0) return hipSuccess;
    hipError_t e = launch_logmm_max(lhs, rhs, lmax, rmax, B, M, K, Nn, stream);
    if (e != hipSuccess) return e;
    dim3 grid((M + TM - 1) / TM, (Nn + TN - 1) / TN, B);
    hipLaunchKernelGGL(logmm_fwd_kernel, grid, dim3(256), 0, stream, lhs.p, lhs.sb, lhs.s1, lhs.s2,
                       rhs.p, rhs.sb, rhs.s1, rhs.s2, lmax, rmax, res, M, K, Nn, row_len, col_len);
    return hipGetLastError();
}

hipError_t launch_logmm_bwd_lhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const float *lmax, const float *rmax, const float *go,
                                const float *res, const LogmmGrad &grad, int B, int M, int K,
                                int Nn, const int *row_len, const int *col_len,
                                const float *batch_scale, hipStream_t stream) {
    if (B == 0 || M == 0 || K == 0) return hipSuccess;
    dim3 grid((M + TM - 1) / TM, (K + TN - 1) / TN, B);
    // own = lhs[b,i,k]; oth[q=j][k] = rhs[b,k,j]; go/res[i,j]: p stride Nn, q stride 1
    hipLaunchKernelGGL(logmm_bwd_kernel, grid, dim3(256), 0, stream, lhs.p, lhs.sb, lhs.s1, lhs.s2,
                       rhs.p, rhs.sb, rhs.s2, rhs.s1, lmax, rmax, go, res, (long)M * Nn, (long)Nn,
                       1L, grad.p, grad.sb, grad.s1, grad.s2, M, Nn, K, row_len, 0, col_len, 1,
                       batch_scale);
    return hipGetLastError();
}

hipError_t launch_logmm_bwd_rhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const float *lmax, const float *rmax, const float *go,
                                const float *res, const LogmmGrad &grad, int B, int M, int K,
                                int Nn, const int *row_len, const int *col_len,
                                const float *batch_scale, hipStream_t stream) {
    if (B == 0 || Nn == 0 || K == 0) return hipSuccess;
    dim3 grid((Nn + TM - 1) / TM, (K + TN - 1) / TN, B);
    // own[p=j][k] = rhs[b,k,j]; oth[q=i][k] = lhs[b,i,k]; go/res[i,j]: p stride 1, q stride Nn.
    // grad is addressed [b, j, k] through (s2, s1) of the (B,K,Nn) gradient layout.
    hipLaunchKernelGGL(logmm_bwd_kernel, grid, dim3(256), 0, stream, rhs.p, rhs.sb, rhs.s2, rhs.s1,
                       lhs.p, lhs.sb, lhs.s1, lhs.s2, rmax, lmax, go, res, (long)M * Nn, 1L,
                       (long)Nn, grad.p, grad.sb, grad.s2, grad.s1, Nn, M, K, col_len, 1, row_len,
                       0, batch_scale);
    return hipGetLastError();
}

}  // namespace wctct
