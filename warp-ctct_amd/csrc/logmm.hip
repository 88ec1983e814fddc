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
// The reference launches one block per output element and re-reads 2K values
// for each.  Here a workgroup owns an output tile and streams the reduction
// dimension through LDS once per tile.  Forward: every operand is shifted by
// its row (column) maximum and scaled to log2 when it is staged in LDS, so the
// inner loop is one add, one v_exp_f32 and one accumulate per term and cannot
// overflow; an output whose shifted sum falls below 2^-60 (the maxima of its
// row and column sit at far-apart k) is recomputed exactly with its own
// maximum, so the result never depends on the shift.
#include "device_utils.h"
#include "launch.h"

namespace wctct {

namespace {

constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kLn2F = 0.6931471805599453f;

__device__ __forceinline__ float neg_inf_f() { return -__builtin_huge_valf(); }

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

// ---- forward ----------------------------------------------------------------
constexpr int FM = 64;   // tile rows (i)
constexpr int FN = 32;   // tile cols (j)
constexpr int FK = 32;   // reduction chunk
constexpr int FPAD = 1;

__device__ float exact_lse(const float *lrow, long lsk, const float *rcol, long rsk, int K) {
    float mx = neg_inf_f();
    for (int k = 0; k < K; ++k) mx = fmaxf(mx, lrow[(size_t)k * lsk] + rcol[(size_t)k * rsk]);
    if (mx == neg_inf_f()) return mx;
    float s = 0.0f;
    for (int k = 0; k < K; ++k)
        s += exp2_hw((lrow[(size_t)k * lsk] + rcol[(size_t)k * rsk] - mx) * kLog2eF);
    return mx + log2_hw(s) * kLn2F;
}

// grid (ceil(M/FM), ceil(Nn/FN), B), block 256: thread (ty, tx) = (tid/16, tid%16)
// owns rows ty*4..ty*4+3 and cols tx*2, tx*2+1 of the tile.
__global__ __launch_bounds__(256) void logmm_fwd_kernel(
    const float *__restrict__ lhs, long lsb, long lsm, long lsk, const float *__restrict__ rhs,
    long rsb, long rsk, long rsn, const float *__restrict__ lmax, const float *__restrict__ rmax,
    float *__restrict__ res, int M, int K, int Nn, const int *__restrict__ row_len,
    const int *__restrict__ col_len) {
    __shared__ float sa[FM][FK + FPAD];
    __shared__ float sb_[FN][FK + FPAD];
    const int b = blockIdx.z;
    const int i0 = blockIdx.x * FM, j0 = blockIdx.y * FN;
    // lengths-aware: rows >= row_len[b] and cols > col_len[b] are padding
    const int Mb = row_len ? min(max(row_len[b], 0), M) : M;
    const int Nb = col_len ? min(max(col_len[b], 0) + 1, Nn) : Nn;
    if (i0 >= Mb || j0 >= Nb) return;
    const int tid = threadIdx.x;
    const int ty = tid >> 4, tx = tid & 15;
    const float *lb = lhs + (size_t)b * lsb;
    const float *rb = rhs + (size_t)b * rsb;
    const float *lm = lmax + (size_t)b * M;
    const float *rm = rmax + (size_t)b * Nn;

    float acc[4][2];
#pragma unroll
    for (int a = 0; a < 4; ++a) acc[a][0] = acc[a][1] = 0.0f;

    for (int k0 = 0; k0 < K; k0 += FK) {
        // stage shifted, log2-scaled operands; out-of-range entries as -inf (2^-inf = 0)
        for (int e = tid; e < FM * FK; e += 256) {
            const int r = e / FK, c = e % FK;
            const int i = i0 + r, k = k0 + c;
            float v = neg_inf_f();
            if (i < Mb && k < K) {
                const float m = lm[i];
                v = (lb[(size_t)i * lsm + (size_t)k * lsk] - (m == neg_inf_f() ? 0.0f : m)) * kLog2eF;
            }
            sa[r][c] = v;
        }
        for (int e = tid; e < FN * FK; e += 256) {
            const int r = e / FK, c = e % FK;
            const int j = j0 + r, k = k0 + c;
            float v = neg_inf_f();
            if (j < Nb && k < K) {
                const float m = rm[j];
                v = (rb[(size_t)k * rsk + (size_t)j * rsn] - (m == neg_inf_f() ? 0.0f : m)) * kLog2eF;
            }
            sb_[r][c] = v;
        }
        __syncthreads();
#pragma unroll 8
        for (int c = 0; c < FK; ++c) {
            float av[4], bv[2];
#pragma unroll
            for (int a = 0; a < 4; ++a) av[a] = sa[ty * 4 + a][c];
            bv[0] = sb_[tx * 2][c];
            bv[1] = sb_[tx * 2 + 1][c];
#pragma unroll
            for (int a = 0; a < 4; ++a) {
                acc[a][0] += exp2_hw(av[a] + bv[0]);
                acc[a][1] += exp2_hw(av[a] + bv[1]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int a = 0; a < 4; ++a) {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            const int i = i0 + ty * 4 + a, j = j0 + tx * 2 + c;
            if (i >= Mb || j >= Nb) continue;
            const float s = acc[a][c];
            float out;
            if (s >= 8.6736174e-19f /* 2^-60 */ && s < __builtin_huge_valf()) {
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
constexpr int BP = 32;   // tile over p
constexpr int BK = 64;   // tile over k
constexpr int BQ = 16;   // chunk over q (the reduced index)

__global__ __launch_bounds__(256) void logmm_bwd_kernel(
    const float *__restrict__ own, long osb, long osp, long osk, const float *__restrict__ oth,
    long tsb, long tsq, long tsk, const float *__restrict__ go, const float *__restrict__ res,
    long gsb, long gp, long gq, float *__restrict__ grad, long dsb, long dsp, long dsk, int P,
    int Q, int K, const int *__restrict__ p_len, int p_extra, const int *__restrict__ q_len,
    int q_extra, const float *__restrict__ batch_scale) {
    __shared__ float s_oth[BQ][BK + 1];   // oth[q][k] * log2e
    __shared__ float s_c[BP][BQ + 1];     // -res[p][q] * log2e (or -inf when excluded)
    __shared__ float s_g[BP][BQ + 1];     // go[p][q]
    const int b = blockIdx.z;
    const int p0 = blockIdx.x * BP, k0 = blockIdx.y * BK;
    const int Pb = p_len ? min(max(p_len[b], 0) + p_extra, P) : P;
    const int Qb = q_len ? min(max(q_len[b], 0) + q_extra, Q) : Q;
    const int tid = threadIdx.x;
    const int tp = tid >> 4, tk = tid & 15;   // thread owns p = tp*2+{0,1}, k = tk + 16*{0..3}
    const float *ob = own + (size_t)b * osb;
    const float *tb = oth + (size_t)b * tsb;
    const float *gb = go + (size_t)b * gsb;
    const float *rb = res + (size_t)b * gsb;
    float *db = grad + (size_t)b * dsb;
    const float scale = batch_scale ? batch_scale[b] : 1.0f;

    float l2[2][4], acc[2][4];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int p = p0 + tp * 2 + a, k = k0 + tk + 16 * c;
            acc[a][c] = 0.0f;
            l2[a][c] = (p < Pb && k < K) ? ob[(size_t)p * osp + (size_t)k * osk] * kLog2eF
                                         : neg_inf_f();
        }

    if (p0 < Pb) {
        for (int q0 = 0; q0 < Qb; q0 += BQ) {
            for (int e = tid; e < BQ * BK; e += 256) {
                const int r = e / BK, c = e % BK;
                const int q = q0 + r, k = k0 + c;
                s_oth[r][c] = (q < Qb && k < K) ? tb[(size_t)q * tsq + (size_t)k * tsk] * kLog2eF
                                                : neg_inf_f();
            }
            for (int e = tid; e < BP * BQ; e += 256) {
                const int r = e / BQ, c = e % BQ;
                const int p = p0 + r, q = q0 + c;
                float cv = neg_inf_f(), gv = 0.0f;
                if (p < Pb && q < Qb) {
                    const float rr = rb[(size_t)p * gp + (size_t)q * gq];
                    gv = gb[(size_t)p * gp + (size_t)q * gq] * scale;
                    // an all -inf row has no gradient; a zero grad_out needs no work
                    cv = (rr == neg_inf_f() || gv == 0.0f) ? neg_inf_f() : -rr * kLog2eF;
                }
                s_c[r][c] = cv;
                s_g[r][c] = gv;
            }
            __syncthreads();
#pragma unroll 4
            for (int q = 0; q < BQ; ++q) {
                float ov[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) ov[c] = s_oth[q][tk + 16 * c];
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    const float cv = s_c[tp * 2 + a][q];
                    const float gv = s_g[tp * 2 + a][q];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        // -inf operands give 2^-inf = 0; cv = -inf masks the whole (p,q) pair.
                        // (l2 + ov) may be -inf + (-inf) = -inf, never NaN, since cv is never +inf.
                        acc[a][c] += gv * exp2_hw((l2[a][c] + ov[c]) + cv);
                    }
                }
            }
            __syncthreads();
        }
    }
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const int p = p0 + tp * 2 + a, k = k0 + tk + 16 * c;
            if (p < P && k < K)
                db[(size_t)p * dsp + (size_t)k * dsk] = (p < Pb) ? acc[a][c] : 0.0f;
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

hipError_t launch_logmm_fwd(const LogmmOperand &lhs, const LogmmOperand &rhs, float *lmax,
                            float *rmax, float *res, int B, int M, int K, int Nn,
                            const int *row_len, const int *col_len, hipStream_t stream) {
    if (B == 0 || M == 0 || Nn == 0) return hipSuccess;
    hipError_t e = launch_reduce_max(lhs.p, lhs.sb, lhs.s1, lhs.s2, B, M, K, lmax, stream);
    if (e != hipSuccess) return e;
    // rhs[b,k,j]: rows of the reduction are j (stride s2), k has stride s1
    e = launch_reduce_max(rhs.p, rhs.sb, rhs.s2, rhs.s1, B, Nn, K, rmax, stream);
    if (e != hipSuccess) return e;
    dim3 grid((M + FM - 1) / FM, (Nn + FN - 1) / FN, B);
    hipLaunchKernelGGL(logmm_fwd_kernel, grid, dim3(256), 0, stream, lhs.p, lhs.sb, lhs.s1, lhs.s2,
                       rhs.p, rhs.sb, rhs.s1, rhs.s2, lmax, rmax, res, M, K, Nn, row_len, col_len);
    return hipGetLastError();
}

hipError_t launch_logmm_bwd_lhs(const LogmmOperand &lhs, const LogmmOperand &rhs, const float *go,
                                const float *res, const LogmmGrad &grad, int B, int M, int K,
                                int Nn, const int *row_len, const int *col_len,
                                const float *batch_scale, hipStream_t stream) {
    if (B == 0 || M == 0 || K == 0) return hipSuccess;
    dim3 grid((M + BP - 1) / BP, (K + BK - 1) / BK, B);
    // own = lhs[b,i,k]; oth[q=j][k] = rhs[b,k,j]; go/res[i,j]: p stride Nn, q stride 1
    hipLaunchKernelGGL(logmm_bwd_kernel, grid, dim3(256), 0, stream, lhs.p, lhs.sb, lhs.s1, lhs.s2,
                       rhs.p, rhs.sb, rhs.s2, rhs.s1, go, res, (long)M * Nn, (long)Nn, 1L, grad.p,
                       grad.sb, grad.s1, grad.s2, M, Nn, K, row_len, 0, col_len, 1, batch_scale);
    return hipGetLastError();
}

hipError_t launch_logmm_bwd_rhs(const LogmmOperand &lhs, const LogmmOperand &rhs, const float *go,
                                const float *res, const LogmmGrad &grad, int B, int M, int K,
                                int Nn, const int *row_len, const int *col_len,
                                const float *batch_scale, hipStream_t stream) {
    if (B == 0 || Nn == 0 || K == 0) return hipSuccess;
    dim3 grid((Nn + BP - 1) / BP, (K + BK - 1) / BK, B);
    // own[p=j][k] = rhs[b,k,j]; oth[q=i][k] = lhs[b,i,k]; go/res[i,j]: p stride 1, q stride Nn.
    // grad is addressed [b, j, k] through (s2, s1) of the (B,K,Nn) gradient layout.
    hipLaunchKernelGGL(logmm_bwd_kernel, grid, dim3(256), 0, stream, rhs.p, rhs.sb, rhs.s2, rhs.s1,
                       lhs.p, lhs.sb, lhs.s1, lhs.s2, go, res, (long)M * Nn, 1L, (long)Nn, grad.p,
                       grad.sb, grad.s2, grad.s1, Nn, M, K, col_len, 1, row_len, 0, batch_scale);
    return hipGetLastError();
}

}  // namespace wctct
