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
// all in [0,1], and the contraction becomes a plain fp32 GEMM on the matrix
// cores (v_mfma_f32_16x16x4_f32): a workgroup owns a tile of the output, each
// of its wavefronts RB x CB blocks of 16x16; operands are read from LDS; the
// next chunk of the reduction is fetched into registers while the current one
// is multiplied (two LDS buffers, one barrier per chunk).
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

// ---- shared MFMA tile ----------------------------------------------------------
constexpr int TQ = 32;        // reduction chunk
constexpr int LDK = TQ + 4;   // LDS row stride (floats) of a [row][q] slab: 16-byte aligned rows

typedef float v4f __attribute__((ext_vector_type(4)));

// A workgroup of WR x WC wavefronts owns a (16*RB*WR) x (16*CB*WC) tile; the
// wavefront at (wr, wc) owns RB x CB blocks of 16x16 starting at row
// wr*16*RB, column wc*16*CB.  Both operands lie in LDS as [row or column][q].
// v_mfma_f32_16x16x4_f32: lane l supplies A[l%16][l/16] and B[l/16][l%16] and
// holds D[4*(l/16) + r][l%16] in register r of the accumulator.  The order of
// summation over q is free, so lane group g = l/16 takes q = 8g .. 8g+7 of the
// chunk, which it reads as two 16-byte vectors per block.
template <int RB, int CB>
__device__ __forceinline__ void tile_mfma(const float (*sa)[LDK], const float (*sb)[LDK], int row0,
                                          int col0, int lane, v4f (&acc)[RB][CB]) {
    const int r = lane & 15, g = lane >> 4;
    v4f a[RB][2], b[CB][2];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        a[rb][0] = *reinterpret_cast<const v4f *>(&sa[row0 + rb * 16 + r][g * 8]);
        a[rb][1] = *reinterpret_cast<const v4f *>(&sa[row0 + rb * 16 + r][g * 8 + 4]);
    }
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) {
        b[cb][0] = *reinterpret_cast<const v4f *>(&sb[col0 + cb * 16 + r][g * 8]);
        b[cb][1] = *reinterpret_cast<const v4f *>(&sb[col0 + cb * 16 + r][g * 8 + 4]);
    }
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                acc[rb][cb] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[rb][s >> 2][s & 3],
                                                                   b[cb][s >> 2][s & 3],
                                                                   acc[rb][cb], 0, 0, 0);
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

// grid (ceil(M/TM), ceil(Nn/TN), B) with TM = 16*RB*WR rows i and TN = 16*CB*WC
// columns j per workgroup of 64*WR*WC threads.
template <int RB, int CB, int WR, int WC>
__global__ __launch_bounds__(64 * WR * WC) void logmm_fwd_kernel(
    const float *__restrict__ lhs, long lsb, long lsm, long lsk, const float *__restrict__ rhs,
    long rsb, long rsk, long rsn, const float *__restrict__ lmax, const float *__restrict__ rmax,
    float *__restrict__ res, int M, int K, int Nn, const int *__restrict__ row_len,
    const int *__restrict__ col_len) {
    constexpr int TM = 16 * RB * WR, TN = 16 * CB * WC, NT = 64 * WR * WC;
    constexpr int SA = TM * TQ / NT, SB = TN * TQ / NT;   // staged elements per thread
    static_assert(TM * TQ % NT == 0 && TN * TQ % NT == 0, "slabs must divide over the threads");
    __shared__ __attribute__((aligned(16))) float sa[2][TM][LDK];   // E_l[i][k]
    __shared__ __attribute__((aligned(16))) float sb_[2][TN][LDK];  // E_r[j][k]
    const int b = blockIdx.z;
    const int i0 = blockIdx.x * TM, j0 = blockIdx.y * TN;
    // lengths-aware: rows >= row_len[b] and cols > col_len[b] are padding
    const int Mb = row_len ? min(max(row_len[b], 0), M) : M;
    const int Nb = col_len ? min(max(col_len[b], 0) + 1, Nn) : Nn;
    if (i0 >= Mb || j0 >= Nb) return;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int row0 = (wave % WR) * 16 * RB, col0 = (wave / WR) * 16 * CB;
    const float *lb = lhs + (size_t)b * lsb;
    const float *rb = rhs + (size_t)b * rsb;
    const float *lm = lmax + (size_t)b * M;
    const float *rm = rmax + (size_t)b * Nn;

    // staging: thread tid takes q = tid % 32 of rows tid/32 + (NT/32)*s: the 32
    // lanes of a row read 128 contiguous bytes (k is contiguous for a row-major
    // lhs and for the transposed view that is the rhs of the joiner)
    const int sq = tid & (TQ - 1), sr0 = tid / TQ;
    float shl[SA], shr[SB];              // per staged row: its shift (0 if the row is all -inf)
    bool okl[SA], okr[SB];
    const float *pl[SA], *pr[SB];
#pragma unroll
    for (int s2 = 0; s2 < SA; ++s2) {
        const int i = i0 + sr0 + (NT / TQ) * s2;
        okl[s2] = i < Mb;
        shl[s2] = okl[s2] ? finite_or_zero(lm[i]) : 0.0f;
        pl[s2] = lb + (size_t)min(i, M - 1) * lsm;
    }
#pragma unroll
    for (int s2 = 0; s2 < SB; ++s2) {
        const int j = j0 + sr0 + (NT / TQ) * s2;
        okr[s2] = j < Nb;
        shr[s2] = okr[s2] ? finite_or_zero(rm[j]) : 0.0f;
        pr[s2] = rb + (size_t)min(j, Nn - 1) * rsn;
    }
    float rl[SA], rr[SB];
    auto fetch = [&](int k0) {
        // loads are unconditional from clamped (always valid) addresses and the
        // padding is selected afterwards: no branch separates the loads from
        // the matrix instructions that are meant to hide their latency
        const int k = k0 + sq;
        const bool kin = k < K;
        const size_t kc = (size_t)min(k, K - 1);
#pragma unroll
        for (int s2 = 0; s2 < SA; ++s2) {
            const float v = pl[s2][kc * lsk];
            rl[s2] = (okl[s2] && kin) ? v : neg_inf_f();
        }
#pragma unroll
        for (int s2 = 0; s2 < SB; ++s2) {
            const float v = pr[s2][kc * rsk];
            rr[s2] = (okr[s2] && kin) ? v : neg_inf_f();
        }
    };
    auto stash = [&](int buf) {
#pragma unroll
        for (int s2 = 0; s2 < SA; ++s2)
            sa[buf][sr0 + (NT / TQ) * s2][sq] = exp2_hw((rl[s2] - shl[s2]) * kLog2eF);
#pragma unroll
        for (int s2 = 0; s2 < SB; ++s2)
            sb_[buf][sr0 + (NT / TQ) * s2][sq] = exp2_hw((rr[s2] - shr[s2]) * kLog2eF);
    };

    v4f acc[RB][CB];
#pragma unroll
    for (int a = 0; a < RB; ++a)
#pragma unroll
        for (int c = 0; c < CB; ++c) acc[a][c] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    fetch(0);
    stash(0);
    __syncthreads();
    int buf = 0;
    for (int k0 = 0; k0 < K; k0 += TQ) {
        const bool more = (k0 + TQ) < K;
        if (more) fetch(k0 + TQ);              // global loads in flight during the MFMAs
        tile_mfma<RB, CB>(sa[buf], sb_[buf], row0, col0, lane, acc);
        if (more) stash(buf ^ 1);
        __syncthreads();
        buf ^= 1;
    }
#pragma unroll
    for (int a = 0; a < RB; ++a) {
#pragma unroll
        for (int c = 0; c < CB; ++c) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = i0 + row0 + a * 16 + 4 * (lane >> 4) + r;
                const int j = j0 + col0 + c * 16 + (lane & 15);
                if (i >= Mb || j >= Nb) continue;
                const float s = acc[a][c][r];
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
}

// ---- backward ----------------------------------------------------------------
// C[b,i,j] = scale[b] * go[b,i,j] * exp(ml[i] + mr[j] - res[b,i,j]), the factor
// that a pair (i,j) contributes to both gradients; 0 for padding, for a zero
// grad_out and for an all -inf row (no gradient).  A pair whose exponent
// exceeds 2^60 is stored as 0 and its row is flagged: flags[b,i] = 1 makes the
// gradient kernels add such pairs term by term.  One wavefront per row i.
__global__ __launch_bounds__(256) void logmm_pair_factor_kernel(
    const float *__restrict__ go, const float *__restrict__ res, const float *__restrict__ lmax,
    const float *__restrict__ rmax, const float *__restrict__ batch_scale,
    const int *__restrict__ row_len, const int *__restrict__ col_len, float *__restrict__ C,
    int *__restrict__ flags, int M, int Nn) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = blockIdx.x * 4 + wave, b = blockIdx.y;
    if (i >= M) return;
    const int Mb = row_len ? min(max(row_len[b], 0), M) : M;
    const int Nb = col_len ? min(max(col_len[b], 0) + 1, Nn) : Nn;
    const float scale = batch_scale ? batch_scale[b] : 1.0f;
    const size_t row = ((size_t)b * M + i) * Nn;
    const float ml = lmax[(size_t)b * M + i];
    int unsafe = 0;
    for (int j = lane; j < Nn; j += 64) {
        float cv = 0.0f;
        if (i < Mb && j < Nb) {
            const float gv = go[row + j] * scale, rr = res[row + j];
            if (gv != 0.0f && rr != neg_inf_f()) {
                const float ex = (ml + rmax[(size_t)b * Nn + j] - rr) * kLog2eF;
                if (ex <= kMaxShiftLog2)
                    cv = gv * exp2_hw(ex);
                else
                    unsafe = 1;
            }
        }
        C[row + j] = cv;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) unsafe |= __shfl_xor(unsafe, off, 64);
    if (lane == 0) flags[(size_t)b * M + i] = unsafe;
}

// One kernel serves both operands.  "own" is the operand whose gradient is
// produced, own[b, p, k] with p = i (lhs) or j (rhs); "oth" is the other one,
// oth[b, q, k].  C / go / res are addressed as [b, p*gp + q*gq].
//   grad_own[b,p,k] = sum_q go[p,q] * exp(own[p,k] + oth[q,k] - res[p,q])
//                   = E_own[p,k] * sum_q C[p,q] * E_oth[q,k]
// grid (ceil(P/TP), ceil(K/TK), B) with TP = 16*RB*WR rows p and TK = 16*CB*WC
// columns k per workgroup of 64*WR*WC threads.  Offsets inside one batch are
// 32-bit (the launcher checks the extents).
struct BwdArgs {
    const float *own, *oth, *own_max, *oth_max, *C, *go, *res, *batch_scale;
    const int *flags;       // (B, rows i): 1 = the row holds a pair left out of C
    float *grad;
    long osb, tsb, gsb, dsb;   // batch strides
    int osp, osk, tsq, tsk, gp, gq, dsp, dsk;
    int P, Q, K;
    const int *p_len, *q_len;
    int p_extra, q_extra;
    int flags_follow_p;     // rows i are p (lhs gradient) or q (rhs gradient)
};

template <int RB, int CB, int WR, int WC>
__global__ __launch_bounds__(64 * WR * WC) void logmm_bwd_kernel(const BwdArgs a) {
    constexpr int TP = 16 * RB * WR, TK = 16 * CB * WC, NT = 64 * WR * WC;
    constexpr int SC = TP * TQ / NT, SE = TK * TQ / NT;   // staged elements per thread
    static_assert(TP * TQ % NT == 0 && TK * TQ % NT == 0, "slabs must divide over the threads");
    static_assert(NT % TK == 0, "a thread stages one column k of the E slab");
    __shared__ __attribute__((aligned(16))) float s_c[2][TP][LDK];   // C[p][q]
    __shared__ __attribute__((aligned(16))) float s_e[2][TK][LDK];   // E_oth[k][q]
    const int b = blockIdx.z;
    const int p0 = blockIdx.x * TP, k0 = blockIdx.y * TK;
    const int P = a.P, Q = a.Q, K = a.K;
    const int Pb = a.p_len ? min(max(a.p_len[b], 0) + a.p_extra, P) : P;
    const int Qb = a.q_len ? min(max(a.q_len[b], 0) + a.q_extra, Q) : Q;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int row0 = (wave % WR) * 16 * RB, col0 = (wave / WR) * 16 * CB;
    const float *ob = a.own + (size_t)b * a.osb;
    const float *tb = a.oth + (size_t)b * a.tsb;
    const float *om = a.own_max + (size_t)b * P;
    const float *tm = a.oth_max + (size_t)b * Q;
    const float *cb = a.C + (size_t)b * a.gsb;
    float *db = a.grad + (size_t)b * a.dsb;

    v4f acc[RB][CB];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int c = 0; c < CB; ++c) acc[r][c] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    int unsafe = 0;
    if (p0 < Pb) {
        // rows flagged by the pair-factor kernel that this tile depends on
        const int *fl = a.flags + (size_t)b * (a.flags_follow_p ? P : Q);
        if (a.flags_follow_p) {
            for (int r = tid; r < TP; r += NT) unsafe |= (p0 + r < Pb) ? fl[p0 + r] : 0;
        } else {
            for (int r = tid; r < Qb; r += NT) unsafe |= fl[r];
        }
        // E_oth slab (TQ x TK): thread takes column k0 + tid % TK (contiguous in
        // memory over the lanes) of rows q = tid / TK + (NT/TK)*s.
        // C slab (TP x TQ): element e = tid + NT*s is (p, q) = (e / TQ, e % TQ)
        // when q is the contiguous index of C (gq == 1), else (e % TP, e / TP):
        // consecutive lanes read consecutive addresses.
        // fetch() only loads (clamped, always valid addresses; nothing is
        // computed from the values, so no wait separates the loads from the
        // matrix instructions); stash() selects the padding and does the math.
        const int ek = tid % TK, eq0 = tid / TK;
        const bool ek_ok = (k0 + ek) < K;
        const float *pe = tb + min(k0 + ek, K - 1) * a.tsk;
        const int q_last = (Q - 1) * a.tsq, c_last = (Q - 1) * a.gq;
        int cp[SC], cq[SC];
        bool cp_ok[SC];
        const float *c_row[SC];
#pragma unroll
        for (int s2 = 0; s2 < SC; ++s2) {
            const int e = tid + NT * s2;
            cp[s2] = (a.gq == 1) ? e / TQ : e % TP;
            cq[s2] = (a.gq == 1) ? e % TQ : e / TP;
            cp_ok[s2] = (p0 + cp[s2]) < Pb;
            c_row[s2] = cb + min(p0 + cp[s2], P - 1) * a.gp;
        }
        float re[SE], rtm[SE], rc[SC];
        auto fetch = [&](int q0) {
#pragma unroll
            for (int s2 = 0; s2 < SE; ++s2) {
                const int q = q0 + eq0 + (NT / TK) * s2;
                re[s2] = pe[min(q * a.tsq, q_last)];
                rtm[s2] = tm[min(q, Q - 1)];
            }
#pragma unroll
            for (int s2 = 0; s2 < SC; ++s2) rc[s2] = c_row[s2][min((q0 + cq[s2]) * a.gq, c_last)];
        };
        auto stash = [&](int buf, int q0) {
#pragma unroll
            for (int s2 = 0; s2 < SE; ++s2) {
                const int qq = q0 + eq0 + (NT / TK) * s2;
                const float x = (qq < Qb && ek_ok) ? re[s2] - finite_or_zero(rtm[s2]) : neg_inf_f();
                s_e[buf][ek][eq0 + (NT / TK) * s2] = exp2_hw(x * kLog2eF);
            }
#pragma unroll
            for (int s2 = 0; s2 < SC; ++s2)
                s_c[buf][cp[s2]][cq[s2]] = (cp_ok[s2] && (q0 + cq[s2]) < Qb) ? rc[s2] : 0.0f;
        };
        fetch(0);
        stash(0, 0);
        __syncthreads();
        int buf = 0;
        for (int q0 = 0; q0 < Qb; q0 += TQ) {
            const bool more = (q0 + TQ) < Qb;
            if (more) fetch(q0 + TQ);
            tile_mfma<RB, CB>(s_c[buf], s_e[buf], row0, col0, lane, acc);
            if (more) stash(buf ^ 1, q0 + TQ);
            __syncthreads();
            buf ^= 1;
        }
    }
    const bool slow = __syncthreads_or(unsafe) != 0;
    const float scale = a.batch_scale ? a.batch_scale[b] : 1.0f;
#pragma unroll
    for (int r4 = 0; r4 < RB; ++r4)
#pragma unroll
        for (int c = 0; c < CB; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int p = p0 + row0 + r4 * 16 + 4 * (lane >> 4) + r;
                const int k = k0 + col0 + c * 16 + (lane & 15);
                if (p >= P || k >= K) continue;
                float v = 0.0f;
                if (p < Pb) {
                    const float x_own = ob[p * a.osp + k * a.osk];
                    const float e_own = exp2_hw((x_own - finite_or_zero(om[p])) * kLog2eF);
                    const float s = acc[r4][c][r];
                    // s is 0 where nothing was added: avoid 0 * inf for a +inf operand
                    v = (s != 0.0f) ? e_own * s : 0.0f;
                    if (slow) {
                        // exact per-term pass over the pairs that C left out
                        const float *gb = a.go + (size_t)b * a.gsb, *rb = a.res + (size_t)b * a.gsb;
                        for (int qq = 0; qq < Qb; ++qq) {
                            const float rr = rb[p * a.gp + qq * a.gq];
                            const float gv = gb[p * a.gp + qq * a.gq] * scale;
                            if (gv == 0.0f || rr == neg_inf_f()) continue;
                            if ((om[p] + tm[qq] - rr) * kLog2eF <= kMaxShiftLog2) continue;
                            const float x = x_own + tb[qq * a.tsq + k * a.tsk] - rr;
                            v += gv * exp2_hw(x * kLog2eF);
                        }
                    }
                }
                db[p * a.dsp + k * a.dsk] = v;
            }
}

// Tiles: 64 x 64 or 96 x 64 outputs, whichever pads the tiled extent less.
inline bool prefer_96(int extent) {
    return (extent + 95) / 96 * 96 < (extent + 63) / 64 * 64;
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
    // 8 wavefronts per workgroup: 64 rows i by 96 or 64 columns j
    if (prefer_96(Nn)) {
        dim3 grid((M + 63) / 64, (Nn + 95) / 96, B);
        hipLaunchKernelGGL((logmm_fwd_kernel<1, 3, 4, 2>), grid, dim3(512), 0, stream, lhs.p,
                           lhs.sb, lhs.s1, lhs.s2, rhs.p, rhs.sb, rhs.s1, rhs.s2, lmax, rmax, res,
                           M, K, Nn, row_len, col_len);
    } else {
        dim3 grid((M + 63) / 64, (Nn + 63) / 64, B);
        hipLaunchKernelGGL((logmm_fwd_kernel<1, 2, 4, 2>), grid, dim3(512), 0, stream, lhs.p,
                           lhs.sb, lhs.s1, lhs.s2, rhs.p, rhs.sb, rhs.s1, rhs.s2, lmax, rmax, res,
                           M, K, Nn, row_len, col_len);
    }
    return hipGetLastError();
}

namespace {

bool fits_int(long extent) { return extent >= 0 && extent < 0x7fffffffL; }

// 4 wavefronts per workgroup: 64 rows p (one 16-row block per wavefront, all 64
// columns) or 96 rows p (all rows, 16 columns per wavefront) by 64 columns k
hipError_t launch_bwd(const BwdArgs &a, int B, hipStream_t stream) {
    // offsets inside one batch are 32-bit in the kernel
    if (!fits_int((long)(a.P - 1) * a.osp + (long)(a.K - 1) * a.osk + 1) ||
        !fits_int((long)(a.Q - 1) * a.tsq + (long)(a.K - 1) * a.tsk + 1) ||
        !fits_int((long)(a.P - 1) * a.dsp + (long)(a.K - 1) * a.dsk + 1) ||
        !fits_int((long)a.P * a.Q))
        return hipErrorInvalidValue;
    if (prefer_96(a.P)) {
        dim3 grid((a.P + 95) / 96, (a.K + 63) / 64, B);
        hipLaunchKernelGGL((logmm_bwd_kernel<6, 1, 1, 4>), grid, dim3(256), 0, stream, a);
    } else {
        dim3 grid((a.P + 63) / 64, (a.K + 63) / 64, B);
        hipLaunchKernelGGL((logmm_bwd_kernel<1, 4, 4, 1>), grid, dim3(256), 0, stream, a);
    }
    return hipGetLastError();
}

bool stride_ok(long s) { return s >= 0 && s < 0x7fffffffL; }

}  // namespace

hipError_t launch_logmm_pair_factor(const float *go, const float *res, const float *lmax,
                                    const float *rmax, const float *batch_scale,
                                    const int *row_len, const int *col_len, float *C, int *flags,
                                    int B, int M, int Nn, hipStream_t stream) {
    if (B == 0 || M == 0) return hipSuccess;
    hipLaunchKernelGGL(logmm_pair_factor_kernel, dim3((M + 3) / 4, B), dim3(256), 0, stream, go,
                       res, lmax, rmax, batch_scale, row_len, col_len, C, flags, M, Nn);
    return hipGetLastError();
}

hipError_t launch_logmm_bwd_lhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const float *lmax, const float *rmax, const float *go,
                                const float *res, const float *C, const int *flags,
                                const LogmmGrad &grad, int B, int M, int K, int Nn,
                                const int *row_len, const int *col_len, const float *batch_scale,
                                hipStream_t stream) {
    if (B == 0 || M == 0 || K == 0) return hipSuccess;
    if (!stride_ok(lhs.s1) || !stride_ok(lhs.s2) || !stride_ok(rhs.s1) || !stride_ok(rhs.s2) ||
        !stride_ok(grad.s1) || !stride_ok(grad.s2))
        return hipErrorInvalidValue;
    // own = lhs[b,i,k]; oth[q=j][k] = rhs[b,k,j]; C/go/res[i,j]: p stride Nn, q stride 1
    BwdArgs a;
    a.own = lhs.p, a.osb = lhs.sb, a.osp = (int)lhs.s1, a.osk = (int)lhs.s2;
    a.oth = rhs.p, a.tsb = rhs.sb, a.tsq = (int)rhs.s2, a.tsk = (int)rhs.s1;
    a.own_max = lmax, a.oth_max = rmax;
    a.C = C, a.go = go, a.res = res, a.gsb = (long)M * Nn, a.gp = Nn, a.gq = 1;
    a.flags = flags, a.flags_follow_p = 1;
    a.grad = grad.p, a.dsb = grad.sb, a.dsp = (int)grad.s1, a.dsk = (int)grad.s2;
    a.P = M, a.Q = Nn, a.K = K;
    a.p_len = row_len, a.p_extra = 0, a.q_len = col_len, a.q_extra = 1;
    a.batch_scale = batch_scale;
    return launch_bwd(a, B, stream);
}

hipError_t launch_logmm_bwd_rhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const float *lmax, const float *rmax, const float *go,
                                const float *res, const float *C, const int *flags,
                                const LogmmGrad &grad, int B, int M, int K, int Nn,
                                const int *row_len, const int *col_len, const float *batch_scale,
                                hipStream_t stream) {
    if (B == 0 || Nn == 0 || K == 0) return hipSuccess;
    if (!stride_ok(lhs.s1) || !stride_ok(lhs.s2) || !stride_ok(rhs.s1) || !stride_ok(rhs.s2) ||
        !stride_ok(grad.s1) || !stride_ok(grad.s2))
        return hipErrorInvalidValue;
    // own[p=j][k] = rhs[b,k,j]; oth[q=i][k] = lhs[b,i,k]; C/go/res[i,j]: p stride 1, q stride Nn.
    // grad is addressed [b, j, k] through (s2, s1) of the (B,K,Nn) gradient layout.
    BwdArgs a;
    a.own = rhs.p, a.osb = rhs.sb, a.osp = (int)rhs.s2, a.osk = (int)rhs.s1;
    a.oth = lhs.p, a.tsb = lhs.sb, a.tsq = (int)lhs.s1, a.tsk = (int)lhs.s2;
    a.own_max = rmax, a.oth_max = lmax;
    a.C = C, a.go = go, a.res = res, a.gsb = (long)M * Nn, a.gp = 1, a.gq = Nn;
    a.flags = flags, a.flags_follow_p = 0;
    a.grad = grad.p, a.dsb = grad.sb, a.dsp = (int)grad.s2, a.dsk = (int)grad.s1;
    a.P = Nn, a.Q = M, a.K = K;
    a.p_len = col_len, a.p_extra = 1, a.q_len = row_len, a.q_extra = 0;
    a.batch_scale = batch_scale;
    return launch_bwd(a, B, stream);
}

}  // namespace wctct
