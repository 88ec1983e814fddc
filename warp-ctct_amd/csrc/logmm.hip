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
// maximum m and exponentiated ONCE, by a kernel that reads the operand and
// writes
//     E_l[i,k] = exp(lhs[i,k] - ml[i]),   E_r[j,k] = exp(rhs[k,j] - mr[j]),
// all in [0,1], k contiguous, rows padded with zeros to a multiple of 32.
// Forward and both gradients are then plain fp32 GEMMs on the matrix cores
// (v_mfma_f32_16x16x4_f32) whose operands are copied global -> LDS as 16-byte
// vectors while the previous chunk is multiplied:
//     res[i,j]      = ml[i] + mr[j] + log(sum_k E_l[i,k] E_r[j,k])
//     grad_lhs[i,k] = E_l[i,k] * sum_j C[i,j] E_r[j,k],
//     C[i,j]        = go[i,j] * exp(ml[i] + mr[j] - res[i,j])     (likewise rhs)
// The shift cannot overflow.  It can underflow when the maxima of a row and a
// column sit at far-apart k: an output whose shifted sum falls below 2^-60 is
// recomputed exactly with its own maximum, and in the backward a pair (i,j)
// whose C would exceed 2^60 is left out of the GEMM and added by an exact
// per-term pass (taken only by tiles that depend on such a pair).  Results
// never depend on the shift beyond fp32 rounding.
#include <algorithm>

#include "device_utils.h"
#include "launch.h"
#include "unit_grad.h"

namespace wctct {

namespace {

constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kLn2F = 0.6931471805599453f;
constexpr float kTiny = 8.6736174e-19f;   // 2^-60
constexpr float kMaxShiftLog2 = 60.0f;

typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float neg_inf_f() { return -__builtin_huge_valf(); }
__device__ __forceinline__ float finite_or_zero(float m) { return m == neg_inf_f() ? 0.0f : m; }

// ---- shifted exponentials of an operand --------------------------------------
// One wavefront per row r of x[b, r, k] (element strides sb, sr, sk):
//   mx[b,r]  = max_k x[b,r,k]
//   E[b,r,k] = exp(x[b,r,k] - mx[b,r])  for k < K,  0 for K <= k < Kp
// (the shift is 0 for an all -inf row).  Rows r >= len[b] + extra are padding:
// mx = -inf, E = 0.  E is (B, R, Kp) contiguous.  The row is read twice; the
// second read comes from cache.
__global__ __launch_bounds__(256) void shift_exp_kernel(const float *__restrict__ x, long sb,
                                                        long sr, long sk, int R, int K, int Kp,
                                                        const int *__restrict__ len, int extra,
                                                        float *__restrict__ mx,
                                                        float *__restrict__ E) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + wave;
    const int b = blockIdx.y;
    if (r >= R) return;
    const int Rb = len ? min(max(len[b], 0) + extra, R) : R;
    float *e = E + ((size_t)b * R + r) * Kp;
    const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
    if (r >= Rb) {
        for (int k = lane * 4; k < Kp; k += 256) *reinterpret_cast<v4f *>(e + k) = zero;
        if (lane == 0) mx[(size_t)b * R + r] = neg_inf_f();
        return;
    }
    const float *p = x + (size_t)b * sb + (size_t)r * sr;
    // 16-byte loads when the row is contiguous and aligned
    const bool vec = sk == 1 && (K & 3) == 0 && (reinterpret_cast<uintptr_t>(p) & 15u) == 0;
    float m = neg_inf_f();
    if (vec) {
        for (int k = lane * 4; k < K; k += 256) {
            const v4f v = *reinterpret_cast<const v4f *>(p + k);
            m = fmaxf(fmaxf(m, fmaxf(v.x, v.y)), fmaxf(v.z, v.w));
        }
    } else {
        for (int k = lane; k < K; k += 64) m = fmaxf(m, p[(size_t)k * sk]);
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) mx[(size_t)b * R + r] = m;
    const float shift = finite_or_zero(m);
    if (vec) {
        for (int k = lane * 4; k < Kp; k += 256) {
            v4f o = zero;
            if (k < K) {
                const v4f v = *reinterpret_cast<const v4f *>(p + k);
                o.x = exp2_hw((v.x - shift) * kLog2eF);
                o.y = exp2_hw((v.y - shift) * kLog2eF);
                o.z = exp2_hw((v.z - shift) * kLog2eF);
                o.w = exp2_hw((v.w - shift) * kLog2eF);
            }
            *reinterpret_cast<v4f *>(e + k) = o;
        }
    } else {
        for (int k = lane; k < Kp; k += 64)
            e[k] = (k < K) ? exp2_hw((p[(size_t)k * sk] - shift) * kLog2eF) : 0.0f;
    }
}

// The same with the whole row held in registers (NV 16-byte vectors per lane,
// K <= 256*NV): the operand is read once.  Requires contiguous, 16-byte
// aligned rows (the launcher checks).
template <int NV>
__global__ __launch_bounds__(256) void shift_exp_rows_kernel(const float *__restrict__ x, long sb,
                                                             long sr, int R, int K, int Kp,
                                                             const int *__restrict__ len,
                                                             int extra, float *__restrict__ mx,
                                                             float *__restrict__ E) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int r = blockIdx.x * 4 + wave;
    const int b = blockIdx.y;
    if (r >= R) return;
    const int Rb = len ? min(max(len[b], 0) + extra, R) : R;
    float *e = E + ((size_t)b * R + r) * Kp;
    const v4f zero = {0.0f, 0.0f, 0.0f, 0.0f};
    if (r >= Rb) {
        for (int k = lane * 4; k < Kp; k += 256) *reinterpret_cast<v4f *>(e + k) = zero;
        if (lane == 0) mx[(size_t)b * R + r] = neg_inf_f();
        return;
    }
    const float *p = x + (size_t)b * sb + (size_t)r * sr;
    v4f v[NV];
#pragma unroll
    for (int j = 0; j < NV; ++j)
        v[j] = *reinterpret_cast<const v4f *>(p + min(j * 256 + lane * 4, K - 4));
    float m = neg_inf_f();
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        if (j * 256 + lane * 4 < K)
            m = fmaxf(fmaxf(m, fmaxf(v[j].x, v[j].y)), fmaxf(v[j].z, v[j].w));
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
    if (lane == 0) mx[(size_t)b * R + r] = m;
    const float shift = finite_or_zero(m);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
        const int k = j * 256 + lane * 4;
        if (k >= Kp) continue;
        v4f o = zero;
        if (k < K) {
            o.x = exp2_hw((v[j].x - shift) * kLog2eF);
            o.y = exp2_hw((v[j].y - shift) * kLog2eF);
            o.z = exp2_hw((v[j].z - shift) * kLog2eF);
            o.w = exp2_hw((v[j].w - shift) * kLog2eF);
        }
        *reinterpret_cast<v4f *>(e + k) = o;
    }
}

// ---- MFMA tiles ----------------------------------------------------------------
// v_mfma_f32_16x16x4_f32: lane l supplies A[l%16][l/16] and B[l/16][l%16] and
// holds D[4*(l/16) + r][l%16] in register r of the accumulator.
// A workgroup of WR x WC wavefronts owns a (16*RB*WR) x (16*CB*WC) tile; the
// wavefront at (wr, wc) owns RB x CB blocks of 16x16 starting at row
// wr*16*RB, column wc*16*CB.  The reduction runs in chunks of TQ = 32.
constexpr int TQ = 32;
constexpr int kDepth = 4;     // chunks of global loads in flight in the forward (even)
constexpr int LDK = TQ + 4;   // row stride (floats) of a [row][q] slab: 16-byte aligned rows

// Both operands in LDS as [row or column][q].  The order of summation over q
// is free, so lane group g = l/16 takes q = 8g .. 8g+7 of the chunk, which it
// reads as two 16-byte vectors per block.
template <int RB, int CB>
__device__ __forceinline__ void tile_mfma_qq(const float (*sa)[LDK], const float (*sb)[LDK],
                                             int row0, int col0, int lane, v4f (&acc)[RB][CB]) {
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

// A in LDS as [row][q] (stride LDA), B as [q][column] (stride LDB): lane group
// g takes q = 4s + g in step s; 4-byte reads, free of bank conflicts for
// LDA = 36 and LDB = 16 (mod 64).  With SWAP the two values change places in
// the instruction, which transposes the product: the lane then holds
// D[row = l%16 of A's block][4 consecutive columns 4*(l/16) + r of B's block],
// i.e. 16 contiguous bytes of a row-major output instead of 4 rows of one column.
template <int RB, int CB, int LDA, int LDB, bool SWAP = false>
__device__ __forceinline__ void tile_mfma_qc(const float (*sa)[LDA], const float (*sb)[LDB],
                                             int row0, int col0, int lane, v4f (&acc)[RB][CB]) {
    const int r = lane & 15, g = lane >> 4;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
        float a[RB], b[CB];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb) a[rb] = sa[row0 + rb * 16 + r][4 * s + g];
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) b[cb] = sb[4 * s + g][col0 + cb * 16 + r];
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
#pragma unroll
            for (int cb = 0; cb < CB; ++cb)
                acc[rb][cb] = SWAP ? __builtin_amdgcn_mfma_f32_16x16x4f32(b[cb], a[rb],
                                                                          acc[rb][cb], 0, 0, 0)
                                   : __builtin_amdgcn_mfma_f32_16x16x4f32(a[rb], b[cb],
                                                                          acc[rb][cb], 0, 0, 0);
    }
}

// ---- placement of the workgroups --------------------------------------------
// The 8 XCDs of the GPU, each with its own 4 MB L2, receive the workgroups of a
// launch round-robin by linear index.  Every workgroup of a batch entry re-reads
// that entry's second operand, so the batch entries are dealt to the XCDs (entry
// b runs on XCD b % 8) instead of being spread over all of them: an L2 then
// serves 1/8 of the operands, not every one.  The grid is one-dimensional,
// 8 * ceil(B/8) * tiles_x * tiles_y workgroups; tiles with b >= B do not exist.
struct TileId {
    int x, y, b;
};
__device__ __forceinline__ TileId xcd_tile(int tiles_x, int tiles_y) {
    const int per_batch = tiles_x * tiles_y;
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int w = slot % per_batch;
    TileId t;
    t.b = (slot / per_batch) * 8 + xcd;
    t.x = w % tiles_x;
    t.y = w / tiles_x;
    return t;
}
inline unsigned xcd_grid(int tiles_x, int tiles_y, int B) {
    return (unsigned)((B + 7) / 8 * 8) * tiles_x * tiles_y;
}
inline bool xcd_grid_fits(long tiles_x, long tiles_y, int B) {
    return (long)((B + 7) / 8 * 8) * tiles_x * tiles_y < 0x7fffffffL;
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

struct FwdArgs {
    const float *El, *Er;     // (B,M,Kp), (B,Nn,Kp): shifted exponentials
    const float *lmax, *rmax; // (B,M), (B,Nn)
    const float *lhs, *rhs;   // the operands themselves, for the exact fallback
    long lsb, lsm, lsk, rsb, rsk, rsn;
    float *res;               // (B,M,Nn)
    // the reduction may be split over `splits` workgroups (more of them than a
    // small output has tiles); then each writes its partial sums to
    // partial (splits,B,M,Nn) and logmm_fwd_finish_kernel adds them up
    float *partial;
    int splits, chunks_per_split;
    int pM, pN;               // rows and row length of one partial sum (>= M, Nn)
    // the slab kernel reading lhs itself: every slab shifts a row by the row's
    // maximum inside the slab, slab_max (splits,B,pM); the caller's next kernel
    // brings the partial sums to the row's maximum (LogmmDeferred)
    float *slab_max = nullptr;
    int M, K, Kp, Nn;
    int B, tiles_x, tiles_y;  // batch entries, row tiles, column tiles * splits
    const int *row_len, *col_len;
};

// res from a sum s of shifted exponentials; the exact fallback for sums that
// underflowed (or overflowed)
__device__ __forceinline__ float fwd_result(const FwdArgs &a, int b, int i, int j, float s) {
    if (s >= kTiny && s < __builtin_huge_valf())
        return a.lmax[(size_t)b * a.M + i] + a.rmax[(size_t)b * a.Nn + j] + log2_hw(s) * kLn2F;
    return exact_lse(a.lhs + (size_t)b * a.lsb + (size_t)i * a.lsm, a.lsk,
                     a.rhs + (size_t)b * a.rsb + (size_t)j * a.rsn, a.rsk, a.K);
}

// grid (ceil(M/TM), ceil(Nn/TN) * splits, B) with TM = 16*RB*WR rows i and
// TN = 16*CB*WC columns j per workgroup of 64*WR*WC threads.
template <int RB, int CB, int WR, int WC>
__global__ __launch_bounds__(64 * WR * WC) void logmm_fwd_kernel(const FwdArgs a) {
    constexpr int TM = 16 * RB * WR, TN = 16 * CB * WC, NT = 64 * WR * WC;
    constexpr int VA = TM * TQ / 4, VB = TN * TQ / 4;   // 16-byte vectors per slab
    constexpr int SA = VA / NT, SB = VB / NT;           // ... per thread
    static_assert(VA % NT == 0 && VB % NT == 0, "slabs must divide over the threads");
    __shared__ __attribute__((aligned(16))) float sa[2][TM][LDK];   // E_l[i][k]
    __shared__ __attribute__((aligned(16))) float sb_[2][TN][LDK];  // E_r[j][k]
    const TileId tile = xcd_tile(a.tiles_x, a.tiles_y);
    const int b = tile.b;
    if (b >= a.B) return;
    const int split = tile.y % a.splits;
    const int i0 = tile.x * TM, j0 = (tile.y / a.splits) * TN;
    const int M = a.M, Nn = a.Nn, Kp = a.Kp;
    // lengths-aware: rows >= row_len[b] and cols > col_len[b] are padding
    const int Mb = a.row_len ? min(max(a.row_len[b], 0), M) : M;
    const int Nb = a.col_len ? min(max(a.col_len[b], 0) + 1, Nn) : Nn;
    if (i0 >= Mb || j0 >= Nb) return;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int row0 = (wave % WR) * 16 * RB, col0 = (wave / WR) * 16 * CB;

    // staging: vector e = tid + NT*s of a slab is (row, 4 k's) = (e / 8, e % 8);
    // rows beyond the operand are clamped (their outputs are not stored)
    const float *pa[SA], *pb[SB];
#pragma unroll
    for (int s = 0; s < SA; ++s) {
        const int e = tid + NT * s;
        pa[s] = a.El + ((size_t)b * M + min(i0 + e / 8, M - 1)) * Kp + (e % 8) * 4;
    }
#pragma unroll
    for (int s = 0; s < SB; ++s) {
        const int e = tid + NT * s;
        pb[s] = a.Er + ((size_t)b * Nn + min(j0 + e / 8, Nn - 1)) * Kp + (e % 8) * 4;
    }
    // The reduction is pipelined kDepth chunks deep: a chunk's global loads are
    // issued kDepth - 1 iterations before they are copied to LDS (a round trip
    // to memory takes several times the ~770 cycles of one chunk's MFMAs).
    // No load or LDS store sits behind a branch or a lane mask, so that the
    // compiler can wait for exactly the oldest chunk (a masked load makes it
    // wait for all of them); chunks past the end are clamped duplicates.
    v4f ra[kDepth][SA], rb[kDepth][SB];
    auto fetch = [&](int set, int k0) {
#pragma unroll
        for (int s = 0; s < SA; ++s)
            ra[set][s] = *reinterpret_cast<const v4f *>(pa[s] + k0);
#pragma unroll
        for (int s = 0; s < SB; ++s)
            rb[set][s] = *reinterpret_cast<const v4f *>(pb[s] + k0);
    };
    auto stash = [&](int set, int buf) {
#pragma unroll
        for (int s = 0; s < SA; ++s) {
            const int e = tid + NT * s;
            *reinterpret_cast<v4f *>(&sa[buf][e / 8][(e % 8) * 4]) = ra[set][s];
        }
#pragma unroll
        for (int s = 0; s < SB; ++s) {
            const int e = tid + NT * s;
            *reinterpret_cast<v4f *>(&sb_[buf][e / 8][(e % 8) * 4]) = rb[set][s];
        }
    };

    v4f acc[RB][CB];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int c = 0; c < CB; ++c) acc[r][c] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

    // chunk j lives in register set j % kDepth and in LDS buffer j % 2; an empty
    // reduction leaves the sums at 0: log 0 below
    // this workgroup's share of the reduction: chunks [c_begin, c_begin + n)
    const int c_begin = split * a.chunks_per_split;
    const int n = max(min(Kp / TQ - c_begin, a.chunks_per_split), 0);
    const int k_first = c_begin * TQ, k_last = max(k_first + (n - 1) * TQ, 0);
    if (n > 0) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) fetch(d, min(k_first + d * TQ, k_last));
        stash(0, 0);
        fetch(0, min(k_first + kDepth * TQ, k_last));
        __syncthreads();
    }
    for (int j0 = 0; j0 < n; j0 += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            const int j = j0 + d;
            if (j < n) {   // uniform over the workgroup
                tile_mfma_qq<RB, CB>(sa[d & 1], sb_[d & 1], row0, col0, lane, acc);
                stash((d + 1) % kDepth, (d + 1) & 1);
                // set (d+1) % kDepth is free again: refill it kDepth chunks ahead
                fetch((d + 1) % kDepth, min(k_first + (j + 1 + kDepth) * TQ, k_last));
                __syncthreads();
            }
        }
    }
#pragma unroll
    for (int r4 = 0; r4 < RB; ++r4) {
#pragma unroll
        for (int c = 0; c < CB; ++c) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = i0 + row0 + r4 * 16 + 4 * (lane >> 4) + r;
                const int j = j0 + col0 + c * 16 + (lane & 15);
                if (i >= Mb || j >= Nb) continue;
                const float s = acc[r4][c][r];
                const size_t at = ((size_t)b * M + i) * Nn + j;
                if (a.splits > 1)
                    a.partial[(size_t)split * a.B * M * Nn + at] = s;
                else
                    a.res[at] = fwd_result(a, b, i, j, s);
            }
        }
    }
}

// ---- fp32 products on the bfloat16 matrix cores -------------------------------
// An fp32 value x is split into three bfloat16 values h + m + l (each rounded to
// nearest even from what the ones before left over): 24 bits of mantissa, i.e.
// all of x but for values near the bottom of the fp32 range.  A product of two
// such sums, cut after the terms of order 2^-16 (lh, hl, mm, mh, hm, hh; small
// ones first), is as accurate as an fp32 product: measured relative error of a
// dot product of length 2048: 4e-8 (plain fp32 accumulation: 2e-6).  Six
// v_mfma_f32_16x16x32_bf16 do per 32 reduction indices what eight
// v_mfma_f32_16x16x4_f32 do per 32 in fp32, in 96 instead of 256 cycles.
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

struct Split3 {
    __bf16 h, m, l;
};
__device__ __forceinline__ Split3 split3(float x) {
    Split3 s;
    s.h = (__bf16)x;
    const float r1 = x - (float)s.h;
    s.m = (__bf16)r1;
    s.l = (__bf16)(r1 - (float)s.m);
    return s;
}
// Two values -> their three planes by truncation, each plane as two packed
// bfloat16 (integer instructions only; x = h + m + l exactly, as with rounding,
// since three 8-bit pieces cover the 24 bits of an fp32 significand)
struct Pair3 {
    unsigned h, m, l;
};
__device__ __forceinline__ Pair3 split3_pair(float x0, float x1) {
    const unsigned top = 0xffff0000u;
    const float h0 = __uint_as_float(__float_as_uint(x0) & top), h1 = __uint_as_float(__float_as_uint(x1) & top);
    const float r0 = x0 - h0, r1 = x1 - h1;
    const float m0 = __uint_as_float(__float_as_uint(r0) & top), m1 = __uint_as_float(__float_as_uint(r1) & top);
    const float s0 = r0 - m0, s1 = r1 - m1;
    Pair3 p;
    p.h = __builtin_amdgcn_perm(__float_as_uint(x1), __float_as_uint(x0), 0x07060302u);
    p.m = __builtin_amdgcn_perm(__float_as_uint(r1), __float_as_uint(r0), 0x07060302u);
    p.l = __builtin_amdgcn_perm(__float_as_uint(s1), __float_as_uint(s0), 0x07060302u);
    return p;
}
// acc += x * y for 16x16 outputs over 32 reduction indices, x and y given as
// their three planes (each lane holds 8 consecutive reduction indices of its
// row / column)
__device__ __forceinline__ v4f mfma6(const bf16x8 (&x)[3], const bf16x8 (&y)[3], v4f acc) {
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[2], y[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[0], y[2], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[1], y[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[1], y[0], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[0], y[1], acc, 0, 0, 0);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(x[0], y[0], acc, 0, 0, 0);
    return acc;
}

// The forward for few columns (Nn up to a few hundred: the label axis of a
// joiner) and a long reduction: the product is bound by streaming E_l once, as
// long as E_r stays on the chip.  A workgroup of 4 wavefronts takes one batch
// entry, one tile of 16*CB columns and one slab of kSlab reduction indices;
// that slab of E_r is split into its three bfloat16 planes and put into LDS
// once (3 x 16*CB x kSlab bfloat16, ~150 KB), and all rows of E_l pass through
// registers against it: a wavefront walks over blocks of 16 rows, a lane loads
// its 8 consecutive k of a row and chunk of 32 as two 16-byte vectors of fp32
// and splits them in registers, and half a block's vectors (4 chunks) are
// requested again as soon as they have been multiplied.  No barrier and no LDS
// write inside the loop.  Each slab writes its partial sums;
// logmm_fwd_finish_kernel adds them in a fixed order.
constexpr int kSlab = 256;
constexpr int kSlabLd = kSlab + 8;   // bfloat16 per LDS row: 16-byte aligned, rows 4 banks apart
constexpr int kSlabWaves = 8;        // two wavefronts per SIMD: one's matrix instructions cover the other's waits

// RAW: E_l is not in memory; the kernel reads lhs itself (k contiguous, K a
// multiple of 32) and forms exp(lhs - lmax) in registers on the way to the
// split (the maxima come from a pass of their own).  E_l is then never
// written: one pass over lhs less per step, and its memory.
template <int CB, bool RAW>
__global__ __launch_bounds__(64 * kSlabWaves) void logmm_fwd_slab_kernel(const FwdArgs a, int slabs) {
    constexpr int TN = 16 * CB, NW = kSlabWaves, NT = 64 * NW;
    constexpr int CH = kSlab / TQ / 2;                  // chunks of 32 per half slab
    constexpr int GB = CB / 2;                          // column blocks per group
    extern __shared__ __attribute__((aligned(16))) __bf16 s_b[];   // [3][TN][kSlabLd]
    // the slabs of one batch entry on one XCD, next to each other in time (see
    // xcd_tile): together they read whole rows of E_l, through one L2
    const TileId tile = xcd_tile(a.tiles_x, a.tiles_y);
    const int b = tile.b;
    if (b >= a.B) return;
    const int slab = tile.x, j0 = tile.y * TN;
    const int M = a.M, Nn = a.Nn, Kp = a.Kp;
    const int Mb = a.row_len ? min(max(a.row_len[b], 0), M) : M;
    const int Nb = a.col_len ? min(max(a.col_len[b], 0) + 1, Nn) : Nn;
    if (Mb <= 0 || j0 >= Nb) return;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int r = lane & 15, g = lane >> 4;
    const int row_blocks = (Mb + 15) / 16;
    const int steps = (row_blocks - wave + NW - 1) / NW;   // row blocks of this wavefront
    // one partial sum is (pM, pN) floats, whole row blocks and column tiles: the
    // stores below need no conditions (and are then counted exactly by the
    // compiler when it waits for the loads in flight around them)
    float *part = a.partial + ((size_t)slab * a.B + b) * a.pM * a.pN;
    const int k0 = slab * kSlab;
    for (int e = tid; e < TN * (kSlab / 4); e += NT) {
        const int row = e / (kSlab / 4), c4 = e - row * (kSlab / 4);
        const int k = k0 + c4 * 4;
        v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (k < Kp)
            v = *reinterpret_cast<const v4f *>(a.Er + ((size_t)b * Nn + min(j0 + row, Nn - 1)) * Kp + k);
        bf16x4 h, m, l;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const Split3 sp = split3(v[i]);
            h[i] = sp.h, m[i] = sp.m, l[i] = sp.l;
        }
        __bf16 *at = s_b + (size_t)row * kSlabLd + c4 * 4;
        *reinterpret_cast<bf16x4 *>(at) = h;
        *reinterpret_cast<bf16x4 *>(at + (size_t)TN * kSlabLd) = m;
        *reinterpret_cast<bf16x4 *>(at + (size_t)2 * TN * kSlabLd) = l;
    }
    __syncthreads();
    if (steps <= 0) return;
    // Two register sets, each one half (4 chunks = 8 vectors per lane) of a row
    // block's share of the slab; a half is requested for the next row block as
    // soon as it has been multiplied, so both are always in flight, and a row
    // block is walked without a branch (the waits are then counted exactly).
    // Vectors past the reduction are clamped into it (they meet zeros of the
    // slab), row blocks past the last repeat it (and are dropped).
    auto request = [&](int st, int half, v4f (&A)[2 * CH]) {
        const int rb = wave + NW * min(st, steps - 1);
        const int i = min(rb * 16 + r, M - 1);
        const float *row = RAW ? a.lhs + (size_t)b * a.lsb + (size_t)i * a.lsm
                               : a.El + ((size_t)b * M + i) * Kp;
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int k = min(k0 + TQ * (half * CH + c) + 8 * g, Kp - 8);
            A[2 * c] = *reinterpret_cast<const v4f *>(row + k);
            A[2 * c + 1] = *reinterpret_cast<const v4f *>(row + k + 4);
        }
    };
    v4f acc[CB];
    // E_r's planes are read from LDS right before the matrix instructions that
    // use them, one group of GB column blocks at a time (the scheduler is held to
    // that: left alone it hoists all reads of a half and spills); the other
    // wavefront of the SIMD covers the wait.
    auto multiply = [&](int half, const v4f (&A)[2 * CH], float shift) {
        bf16x8 xp[3];
#pragma unroll
        for (int item = 0; item < 2 * CH; ++item) {
            const int c = item >> 1, grp = item & 1;
            bf16x8 bq[GB][3];
#pragma unroll
            for (int cb = 0; cb < GB; ++cb)
#pragma unroll
                for (int p = 0; p < 3; ++p)
                    bq[cb][p] = *reinterpret_cast<const bf16x8 *>(
                        s_b + ((size_t)p * TN + (grp * GB + cb) * 16 + r) * kSlabLd +
                        TQ * (half * CH + c) + 8 * g);
            if (grp == 0) {
#pragma unroll
                for (int i = 0; i < 8; ++i) {
                    float x = i < 4 ? A[2 * c][i] : A[2 * c + 1][i - 4];
                    if (RAW) x = exp2_hw((x - shift) * kLog2eF);
                    const Split3 sp = split3(x);
                    xp[0][i] = sp.h, xp[1][i] = sp.m, xp[2][i] = sp.l;
                }
            }
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int cb = 0; cb < GB; ++cb)
                acc[grp * GB + cb] = mfma6(xp, bq[cb], acc[grp * GB + cb]);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    v4f A0[2 * CH], A1[2 * CH];
    request(0, 0, A0);
    // (the two halves in this order, as in the loop: the waits for a half are
    // counted from the loads issued after it)
    __builtin_amdgcn_sched_barrier(0);
    request(0, 1, A1);
    __builtin_amdgcn_sched_barrier(0);
    float *slab_max = RAW ? a.slab_max + ((size_t)slab * a.B + b) * a.pM : nullptr;
    for (int st = 0; st < steps; ++st) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) acc[cb] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        float shift = 0.0f;
        if (RAW) {
            // the row's maximum inside the slab: this lane's 64 values, then the
            // 4 lanes of the row (vectors clamped into the reduction repeat
            // values of the same row: the maximum may only come out larger than
            // the slab's own, and any shift >= it serves)
            float m = neg_inf_f();
#pragma unroll
            for (int v = 0; v < 2 * CH; ++v) {
                m = fmaxf(fmaxf(m, fmaxf(A0[v][0], A0[v][1])), fmaxf(A0[v][2], A0[v][3]));
                m = fmaxf(fmaxf(m, fmaxf(A1[v][0], A1[v][1])), fmaxf(A1[v][2], A1[v][3]));
            }
            m = fmaxf(m, __shfl_xor(m, 16, 64));
            m = fmaxf(m, __shfl_xor(m, 32, 64));
            if (g == 0) slab_max[(wave + NW * st) * 16 + r] = m;
            shift = finite_or_zero(m);
        }
        multiply(0, A0, shift);
        request(st + 1, 0, A0);
        multiply(1, A1, shift);
        // lane l holds D[4*(l/16) + q][l%16] of each block in register q; the
        // stores come before the second request, so that at the head of the
        // loop nothing but the two halves is outstanding
        const int i0 = (wave + NW * st) * 16 + 4 * g;
        float *at = part + (size_t)i0 * a.pN + j0 + r;
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
#pragma unroll
            for (int q = 0; q < 4; ++q) at[(size_t)q * a.pN + cb * 16] = acc[cb][q];
        __builtin_amdgcn_sched_barrier(0);
        request(st + 1, 1, A1);
    }
}

// res from the partial sums of a split reduction, added in a fixed order.
__global__ __launch_bounds__(256) void logmm_fwd_finish_kernel(const FwdArgs a, int B) {
    const int b = blockIdx.y;
    const int e = blockIdx.x * 256 + threadIdx.x;
    if (e >= a.M * a.Nn) return;
    const int i = e / a.Nn, j = e - i * a.Nn;
    const int Mb = a.row_len ? min(max(a.row_len[b], 0), a.M) : a.M;
    const int Nb = a.col_len ? min(max(a.col_len[b], 0) + 1, a.Nn) : a.Nn;
    if (i >= Mb || j >= Nb) return;
    const size_t per = (size_t)a.pM * a.pN;
    const float *p = a.partial + (size_t)b * per + (size_t)i * a.pN + j;
    float s = 0.0f;
    for (int sp = 0; sp < a.splits; ++sp) s += p[(size_t)sp * B * per];
    a.res[(size_t)b * a.M * a.Nn + e] = fwd_result(a, b, i, j, s);
}

// ---- backward ----------------------------------------------------------------
// C[b,i,j] = scale[b] * go[b,i,j] * exp(ml[i] + mr[j] - res[b,i,j]), the factor
// that a pair (i,j) contributes to both gradients; scale[b] is the sample's
// weight (Weight, with row_len as the frame counts), which the kernel also
// leaves in weights_out[b] (if not null) for the kernels that follow; 0 for padding, for a zero
// grad_out and for an all -inf row (no gradient).  A pair whose exponent
// exceeds 2^60 is stored as 0 and its row is flagged: flags[b,i] = 1 makes the
// gradient kernels add such pairs term by term.  Rows of C are logmm_pair_row(Nn)
// floats long, zeros in the padding.  One wavefront per row i.
__global__ __launch_bounds__(256) void logmm_pair_factor_kernel(
    const float *__restrict__ go, const float *__restrict__ res, const float *__restrict__ lmax,
    const float *__restrict__ rmax, const Weight weight, float *__restrict__ weights_out,
    const int *__restrict__ row_len, const int *__restrict__ col_len, float *__restrict__ C,
    int *__restrict__ flags, int M, int Nn) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int i = blockIdx.x * 4 + wave, b = blockIdx.y;
    if (i >= M) return;
    const int Mb = row_len ? min(max(row_len[b], 0), M) : M;
    const int Nb = col_len ? min(max(col_len[b], 0) + 1, Nn) : Nn;
    const float scale = sample_weight(weight, b, row_len ? row_len[b] : 1);
    if (weights_out && blockIdx.x == 0 && threadIdx.x == 0) weights_out[b] = scale;
    const size_t row = ((size_t)b * M + i) * Nn;
    const int Cq = logmm_pair_row(Nn);
    float *crow = C + ((size_t)b * M + i) * Cq;
    const float ml = lmax[(size_t)b * M + i];
    int unsafe = 0;
    for (int j = lane; j < Cq; j += 64) {
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
        crow[j] = cv;
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) unsafe |= __shfl_xor(unsafe, off, 64);
    if (lane == 0) flags[(size_t)b * M + i] = unsafe;
}

// The same, 8 rows i per workgroup, which also writes the pair factors transposed
// and split into three bfloat16 planes, planes[pl][b][j][i] with ct_frames =
// logmm_pair_frames(M) entries per row (8 consecutive i of one j: one 16-byte
// store per plane), zeros for i >= M, and shifts[b][i] = the finite maximum of
// row i of lhs, +inf for rows that are padding (their exponentials are then 0).
// Requires logmm_pair_row(Nn) <= 96.  A workgroup of 8 wavefronts takes 32 rows
// (the padded frame count is a multiple of 32), 4 per wavefront; grid
// (ct_frames / 32, B), 512 threads.
constexpr int kPairRowsPerWave = 4;
__global__ __launch_bounds__(512) void logmm_pair_factor_planes_kernel(
    const float *__restrict__ go, const float *__restrict__ res, const float *__restrict__ lmax,
    const float *__restrict__ rmax, const Weight weight, float *__restrict__ weights_out,
    const int *__restrict__ row_len, const int *__restrict__ col_len, float *__restrict__ C,
    int *__restrict__ flags, unsigned short *__restrict__ planes, float *__restrict__ shifts,
    int B, int M, int Nn, int ct_frames) {
    constexpr int R = kPairRowsPerWave;
    __shared__ float s_c[8 * R][96];
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int b = blockIdx.y, i0 = blockIdx.x * 8 * R;
    const int Mb = row_len ? min(max(row_len[b], 0), M) : M;
    const int Nb = col_len ? min(max(col_len[b], 0) + 1, Nn) : Nn;
    const float scale = sample_weight(weight, b, row_len ? row_len[b] : 1);
    if (weights_out && blockIdx.x == 0 && threadIdx.x == 0) weights_out[b] = scale;
    const int Cq = logmm_pair_row(Nn);
    // row r of this wavefront is local row 8*r + wave.  (A row has at most 96
    // entries; all of a lane's loads are requested before the first is used.)
    float gv[R][2], rr[R][2], rm[2], ml[R];
#pragma unroll
    for (int t = 0; t < 2; ++t) rm[t] = rmax[(size_t)b * Nn + min(lane + 64 * t, Nn - 1)];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int i = min(i0 + 8 * r + wave, M - 1);
        const size_t row = ((size_t)b * M + i) * Nn;
        ml[r] = lmax[(size_t)b * M + i];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int j = min(lane + 64 * t, Nn - 1);
            gv[r][t] = go[row + j], rr[r][t] = res[row + j];
        }
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int i = i0 + 8 * r + wave;
        const bool in_rows = i < M;
        float *crow = C + ((size_t)b * M + min(i, M - 1)) * Cq;
        int unsafe = 0;
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int j = lane + 64 * t;
            if (j >= Cq) break;
            float cv = 0.0f;
            if (i < Mb && j < Nb) {
                const float gs = gv[r][t] * scale;
                if (gs != 0.0f && rr[r][t] != neg_inf_f()) {
                    const float ex = (ml[r] + rm[t] - rr[r][t]) * kLog2eF;
                    if (ex <= kMaxShiftLog2)
                        cv = gs * exp2_hw(ex);
                    else
                        unsafe = 1;
                }
            }
            if (in_rows) crow[j] = cv;
            s_c[8 * r + wave][j] = cv;
        }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) unsafe |= __shfl_xor(unsafe, off, 64);
        if (lane == 0) {
            if (in_rows) flags[(size_t)b * M + i] = unsafe;
            shifts[(size_t)b * ct_frames + i] = (i < Mb) ? finite_or_zero(ml[r]) : __builtin_huge_valf();
        }
    }
    __syncthreads();
    // thread (group of 8 frames, row j of the planes)
    for (int e = tid; e < R * Cq; e += 512) {
        const int grp = e / Cq, j = e - grp * Cq;
        float x[8];
#pragma unroll
        for (int w = 0; w < 8; ++w) x[w] = s_c[8 * grp + w][j];
        const Pair3 p0 = split3_pair(x[0], x[1]), p1 = split3_pair(x[2], x[3]);
        const Pair3 p2 = split3_pair(x[4], x[5]), p3 = split3_pair(x[6], x[7]);
        const size_t plane = (size_t)B * Cq * ct_frames;
        unsigned short *at = planes + ((size_t)b * Cq + j) * ct_frames + i0 + 8 * grp;
        *reinterpret_cast<uint4 *>(at) = make_uint4(p0.h, p1.h, p2.h, p3.h);
        *reinterpret_cast<uint4 *>(at + plane) = make_uint4(p0.m, p1.m, p2.m, p3.m);
        *reinterpret_cast<uint4 *>(at + 2 * plane) = make_uint4(p0.l, p1.l, p2.l, p3.l);
    }
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
    const float *Eown, *Eoth;  // (B,P,Kp), (B,Q,Kp): shifted exponentials
    const float *C;            // pair factors
    const int *flags;          // (B, rows i): 1 = the row holds a pair left out of C
    // for the exact pass only: the operands, their maxima, grad_out and res
    const float *own, *oth, *own_max, *oth_max, *go, *res, *batch_scale;
    float *grad;
    long osb, tsb, gsb, dsb;   // batch strides
    int osp, osk, tsq, tsk, gp, gq, dsp, dsk;
    long csb;                  // C: batch stride and element strides along p and q (its rows
    int cgp, cgq;              // are padded to logmm_pair_row(Nn) floats, zeros in the padding)
    int P, Q, K, Kp;
    const int *p_len, *q_len;
    int p_extra, q_extra;
    int flags_follow_p;        // rows i are p (lhs gradient) or q (rhs gradient)
    int B, tiles_x, tiles_y;   // batch entries, p tiles, k tiles (or groups of k tiles)
    // logmm_bwd_rhs_planes_kernel only: C transposed and split (3, B, ct_rows, ct_frames)
    // and the shifts of the rows of oth (B, ct_frames), see LogmmPairPlanes
    const unsigned short *ct = nullptr;
    const float *ct_shift = nullptr;
    int ct_rows = 0, ct_frames = 0;
};

// E_own * sum; the sum is 0 where nothing was added: avoid 0 * inf or 0 * nan
__device__ __forceinline__ float scaled_sum(float s, float e_own) {
    return (s != 0.0f) ? e_own * s : 0.0f;
}

// Exact per-term pass over the pairs (p, q) that C left out (exponent > 2^60).
__device__ float exact_pairs(const BwdArgs &a, int b, int p, int k, int Qb) {
    const float *ob = a.own + (size_t)b * a.osb;
    const float *tb = a.oth + (size_t)b * a.tsb;
    const float *om = a.own_max + (size_t)b * a.P;
    const float *tm = a.oth_max + (size_t)b * a.Q;
    const float *gb = a.go + (size_t)b * a.gsb;
    const float *rb = a.res + (size_t)b * a.gsb;
    const float scale = a.batch_scale ? a.batch_scale[b] : 1.0f;
    const float x_own = ob[p * a.osp + k * a.osk];
    float v = 0.0f;
    for (int qq = 0; qq < Qb; ++qq) {
        const float rr = rb[p * a.gp + qq * a.gq];
        const float gv = gb[p * a.gp + qq * a.gq] * scale;
        if (gv == 0.0f || rr == neg_inf_f()) continue;
        if ((om[p] + tm[qq] - rr) * kLog2eF <= kMaxShiftLog2) continue;
        const float x = x_own + tb[qq * a.tsq + k * a.tsk] - rr;
        v += gv * exp2_hw(x * kLog2eF);
    }
    return v;
}

template <int RB, int CB, int WR, int WC, int DEPTH, bool REFILL>
__global__ __launch_bounds__(64 * WR * WC) void logmm_bwd_kernel(const BwdArgs a) {
    constexpr int TP = 16 * RB * WR, TK = 16 * CB * WC, NT = 64 * WR * WC;
    constexpr int LDE = TK + 16;                        // 16 (mod 64): see tile_mfma_qc
    constexpr int SC = TP * TQ / NT;                    // C elements per thread and chunk
    constexpr int VE = TQ * TK / 4, SE = VE / NT;       // E vectors per chunk / thread
    static_assert(TP * TQ % NT == 0 && VE % NT == 0, "slabs must divide over the threads");
    __shared__ __attribute__((aligned(16))) float s_c[2][TP][LDK];   // C[p][q]
    __shared__ __attribute__((aligned(16))) float s_e[2][TQ][LDE];   // E_oth[q][k]
    const TileId tile = xcd_tile(a.tiles_x, a.tiles_y);
    const int b = tile.b;
    if (b >= a.B) return;
    const int p0 = tile.x * TP, k0 = tile.y * TK;
    const int P = a.P, Q = a.Q, K = a.K, Kp = a.Kp;
    const int Pb = a.p_len ? min(max(a.p_len[b], 0) + a.p_extra, P) : P;
    const int Qb = a.q_len ? min(max(a.q_len[b], 0) + a.q_extra, Q) : Q;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int row0 = (wave % WR) * 16 * RB, col0 = (wave / WR) * 16 * CB;
    const float *cb = a.C + (size_t)b * a.csb;
    const float *eo = a.Eoth + (size_t)b * Q * Kp;
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
        // E_oth slab (TQ x TK): vector e = tid + NT*s is (q, 4 k's) = (e / (TK/4),
        // e % (TK/4)).  Columns beyond Kp and rows beyond Q are clamped to valid
        // memory: such columns are never stored, and such rows meet C = 0.
        // C slab (TP x TQ): element e is (p, q) = (e / TQ, e % TQ) when q is
        // the contiguous index of C (gq == 1), else (e % TP, e / TP):
        // consecutive lanes read consecutive addresses.
        const float *pe[SE];
        int eq[SE], ek[SE];
#pragma unroll
        for (int s = 0; s < SE; ++s) {
            const int e = tid + NT * s;
            eq[s] = e / (TK / 4);
            ek[s] = (e % (TK / 4)) * 4;
            pe[s] = eo + min(k0 + ek[s], Kp - 4);
        }
        const int c_last = (Q - 1) * a.cgq;
        int cp[SC], cq[SC];
        bool cp_ok[SC];
        const float *c_row[SC];
#pragma unroll
        for (int s = 0; s < SC; ++s) {
            const int e = tid + NT * s;
            cp[s] = (a.cgq == 1) ? e / TQ : e % TP;
            cq[s] = (a.cgq == 1) ? e % TQ : e / TP;
            cp_ok[s] = (p0 + cp[s]) < Pb;
            c_row[s] = cb + min(p0 + cp[s], P - 1) * a.cgp;
        }
        v4f re[DEPTH][SE];
        float rc[DEPTH][SC];
        auto fetch = [&](int set, int q0) {
#pragma unroll
            for (int s = 0; s < SE; ++s)
                re[set][s] = *reinterpret_cast<const v4f *>(
                    pe[s] + (size_t)min(q0 + eq[s], Q - 1) * Kp);
#pragma unroll
            for (int s = 0; s < SC; ++s)
                rc[set][s] = c_row[s][min((q0 + cq[s]) * a.cgq, c_last)];
        };
        auto stash = [&](int set, int buf, int q0) {
#pragma unroll
            for (int s = 0; s < SE; ++s)
                *reinterpret_cast<v4f *>(&s_e[buf][eq[s]][ek[s]]) = re[set][s];
#pragma unroll
            for (int s = 0; s < SC; ++s)
                s_c[buf][cp[s]][cq[s]] = (cp_ok[s] && (q0 + cq[s]) < Qb) ? rc[set][s] : 0.0f;
        };
        // Pipelined like the forward: chunk j in register set j % DEPTH and in
        // LDS buffer j % 2.  REFILL = false is for reductions of at most DEPTH
        // chunks: everything is fetched up front, each chunk once.  With
        // REFILL a set is loaded again as soon as it has been copied to LDS,
        // unconditionally (chunks past the end read clamped addresses and are
        // never multiplied), so that the compiler can wait for exactly the
        // oldest chunk.
        const int n = (Qb + TQ - 1) / TQ;
        if (n > 0) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d)
                if (REFILL || d < n) fetch(d, d * TQ);
            stash(0, 0, 0);
            if (REFILL) fetch(0, DEPTH * TQ);
            __syncthreads();
        }
        for (int j0 = 0; j0 < n; j0 += DEPTH) {
#pragma unroll
            for (int d = 0; d < DEPTH; ++d) {
                const int j = j0 + d;
                if (j < n) {   // uniform over the workgroup
                    tile_mfma_qc<RB, CB, LDK, LDE>(s_c[j & 1], s_e[j & 1], row0, col0, lane, acc);
                    if (REFILL) {
                        stash((d + 1) % DEPTH, (j + 1) & 1, (j + 1) * TQ);
                        fetch((d + 1) % DEPTH, (j + 1 + DEPTH) * TQ);
                    } else if (j + 1 < n) {
                        stash((d + 1) % DEPTH, (j + 1) & 1, (j + 1) * TQ);
                    }
                    __syncthreads();
                }
            }
        }
    }
    const bool slow = __syncthreads_or(unsafe) != 0;
    const float *eown = a.Eown + (size_t)b * P * Kp;
    // E_own of all this lane's outputs first (clamped addresses, no branches),
    // then one select, multiply and store per output; the exact pass is a
    // separate, workgroup-uniform branch
    float ev[RB][CB][4];
#pragma unroll
    for (int r4 = 0; r4 < RB; ++r4)
#pragma unroll
        for (int c = 0; c < CB; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int p = p0 + row0 + r4 * 16 + 4 * (lane >> 4) + r;
                const int k = k0 + col0 + c * 16 + (lane & 15);
                ev[r4][c][r] = eown[(size_t)min(p, P - 1) * Kp + min(k, Kp - 1)];
            }
#pragma unroll
    for (int r4 = 0; r4 < RB; ++r4)
#pragma unroll
        for (int c = 0; c < CB; ++c)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int p = p0 + row0 + r4 * 16 + 4 * (lane >> 4) + r;
                const int k = k0 + col0 + c * 16 + (lane & 15);
                float v = (p < Pb) ? scaled_sum(acc[r4][c][r], ev[r4][c][r]) : 0.0f;
                if (slow && p < Pb && k < K) v += exact_pairs(a, b, p, k, Qb);
                if (p < P && k < K) db[p * a.dsp + k * a.dsk] = v;
            }
}

// The same for short reductions (Q <= 96, e.g. the gradient wrt f of the
// joiner, where q runs over the U+1 contexts): the C slab of a 64-row tile is
// loaded into LDS once and the workgroup then walks over `tiles_per_wg`
// 64-column tiles of k, fetching the next tile's E_oth rows and this tile's
// E_own values while the current tile is multiplied.  Set-up, the C slab and
// the load latency are paid once per workgroup instead of once per tile.
// grid (ceil(P/64), ceil(ceil(K/64) / tiles_per_wg), B), 256 threads.
constexpr int QR = 96;        // longest resident reduction
constexpr int LDC = QR + 4;   // 36 (mod 64), like LDK

__global__ __launch_bounds__(256) void logmm_bwd_resident_kernel(const BwdArgs a,
                                                                 int tiles_per_wg) {
    constexpr int TP = 64, TK = 64, NT = 256, LDE = TK + 16, CB = 4;
    constexpr int SC = TP * QR / NT;           // C elements per thread
    constexpr int SE = QR * TK / 4 / NT;       // E vectors per thread and tile
    __shared__ __attribute__((aligned(16))) float s_c[TP][LDC];   // C[p][q]
    __shared__ __attribute__((aligned(16))) float s_e[QR][LDE];   // E_oth[q][k]
    const TileId tile = xcd_tile(a.tiles_x, a.tiles_y);
    const int b = tile.b;
    if (b >= a.B) return;
    const int p0 = tile.x * TP;
    const int P = a.P, Q = a.Q, K = a.K, Kp = a.Kp;
    const int ktiles = (K + TK - 1) / TK;
    const int kt_begin = tile.y * tiles_per_wg;
    const int kt_end = min(kt_begin + tiles_per_wg, ktiles);
    const int Pb = a.p_len ? min(max(a.p_len[b], 0) + a.p_extra, P) : P;
    const int Qb = a.q_len ? min(max(a.q_len[b], 0) + a.q_extra, Q) : Q;
    const int tid = threadIdx.x;
    const int wave = tid >> 6, lane = tid & 63;
    const int row0 = wave * 16;
    float *db = a.grad + (size_t)b * a.dsb;
    // The product is formed transposed (see tile_mfma_qc): this lane owns row
    // my_p and, in each of the 4 column blocks, 4 consecutive columns from my_k
    const int my_p = p0 + row0 + (lane & 15);
    const int my_k = 4 * (lane >> 4);
    // 16-byte accesses to the gradient need unit stride along k and aligned rows
    const bool vec = a.dsk == 1 && (a.dsp & 3) == 0 && (a.dsb & 3) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.grad) & 15u) == 0;

    if (p0 >= Pb) {   // a tile of padding rows: zeros
        for (int kt = kt_begin; kt < kt_end; ++kt)
#pragma unroll
            for (int c = 0; c < CB; ++c)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int k = kt * TK + c * 16 + my_k + r;
                    if (my_p < P && k < K) db[my_p * a.dsp + k * a.dsk] = 0.0f;
                }
        return;
    }

    int unsafe = 0;
    {
        const int *fl = a.flags + (size_t)b * (a.flags_follow_p ? P : Q);
        if (a.flags_follow_p) {
            for (int r = tid; r < TP; r += NT) unsafe |= (p0 + r < Pb) ? fl[p0 + r] : 0;
        } else {
            for (int r = tid; r < Qb; r += NT) unsafe |= fl[r];
        }
    }
    // C slab, whole reduction: element e = tid + NT*s is (p, q) = (e / QR, e % QR)
    // when q is the contiguous index of C, else (e % TP, e / TP)
    {
        const float *cb = a.C + (size_t)b * a.csb;
        const int c_last = (Q - 1) * a.cgq;
        float rc[SC];
#pragma unroll
        for (int s = 0; s < SC; ++s) {
            const int e = tid + NT * s;
            const int cp = (a.cgq == 1) ? e / QR : e % TP, cq = (a.cgq == 1) ? e % QR : e / TP;
            rc[s] = cb[min(p0 + cp, P - 1) * a.cgp + min(cq * a.cgq, c_last)];
        }
#pragma unroll
        for (int s = 0; s < SC; ++s) {
            const int e = tid + NT * s;
            const int cp = (a.cgq == 1) ? e / QR : e % TP, cq = (a.cgq == 1) ? e % QR : e / TP;
            s_c[cp][cq] = ((p0 + cp) < Pb && cq < Qb) ? rc[s] : 0.0f;
        }
    }
    // E_oth rows of one tile: vector e = tid + NT*s is (q, 4 k's) = (e / 16, e % 16);
    // rows beyond Q and columns beyond Kp are clamped to valid memory (they
    // meet C = 0, or are never stored)
    const float *eo = a.Eoth + (size_t)b * Q * Kp;
    const float *eown = a.Eown + (size_t)b * P * Kp + (size_t)min(my_p, P - 1) * Kp;
    v4f re[SE];
    auto fetch = [&](int kt) {
#pragma unroll
        for (int s = 0; s < SE; ++s) {
            const int e = tid + NT * s;
            re[s] = *reinterpret_cast<const v4f *>(eo + (size_t)min(e / 16, Q - 1) * Kp +
                                                   min(kt * TK + (e % 16) * 4, Kp - 4));
        }
    };
    fetch(kt_begin);
    const bool slow = __syncthreads_or(unsafe) != 0;   // also: the C slab is in LDS
    const int nq = (Qb + TQ - 1) / TQ;
    for (int kt = kt_begin; kt < kt_end; ++kt) {
        const int k0 = kt * TK;
#pragma unroll
        for (int s = 0; s < SE; ++s) {
            const int e = tid + NT * s;
            *reinterpret_cast<v4f *>(&s_e[e / 16][(e % 16) * 4]) = re[s];
        }
        __syncthreads();
        if (kt + 1 < kt_end) fetch(kt + 1);
        // E_own of this lane's outputs, in flight during the MFMAs (Kp is a
        // multiple of 32: the 4 columns are one aligned vector, clamped into the row)
        v4f ev[CB];
#pragma unroll
        for (int c = 0; c < CB; ++c)
            ev[c] = *reinterpret_cast<const v4f *>(eown + min(k0 + c * 16 + my_k, Kp - 4));
        v4f acc[1][CB];
#pragma unroll
        for (int c = 0; c < CB; ++c) acc[0][c] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        for (int c3 = 0; c3 < nq; ++c3)
            tile_mfma_qc<1, CB, LDC, LDE, true>(
                reinterpret_cast<const float (*)[LDC]>(&s_c[0][c3 * TQ]), &s_e[c3 * TQ], row0, 0,
                lane, acc);
#pragma unroll
        for (int c = 0; c < CB; ++c) {
            const int k = k0 + c * 16 + my_k;
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                v[r] = (my_p < Pb) ? scaled_sum(acc[0][c][r], ev[c][r]) : 0.0f;
                if (slow && my_p < Pb && k + r < K) v[r] += exact_pairs(a, b, my_p, k + r, Qb);
            }
            if (my_p >= P) continue;
            float *dst = db + my_p * a.dsp + k * a.dsk;
            if (vec && k + 3 < K) {
                *reinterpret_cast<v4f *>(dst) = v4f{v[0], v[1], v[2], v[3]};
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (k + r < K) dst[r * a.dsk] = v[r];
            }
        }
        __syncthreads();   // everyone is done with s_e
    }
}

// The gradient of the operand with many rows and a SHORT reduction (the f of a
// joiner: P = frames, Q = labels + 1 <= 96, K = vocabulary):
//   grad[b,p,k] = E_own[p,k] * sum_q C[p,q] * E_oth[q,k].
// The product is bound by reading E_own and writing the gradient once, as long
// as E_oth stays on the chip.  A workgroup of 4 wavefronts takes one batch entry
// and kBwdSlab columns k; that slab of E_oth is split into three bfloat16
// planes and put into LDS once, transposed ([k][q]: the reduction index is then
// contiguous for the matrix instruction).  A wavefront walks over blocks of 16
// rows p: it splits the block's rows of C in registers (QC chunks of 32) and
// multiplies them with every 16 columns of the slab.  The product is formed
// transposed (E_oth^T first), so that a lane ends up with 4 consecutive k of one
// row p: one 16-byte load of E_own and one 16-byte store of the gradient.
constexpr int kBwdSlab = 128;

constexpr int kBwdWaves = 4;

// RAW: E_own is not in memory; the kernel reads the operand itself (k contiguous,
// K a multiple of 32) and forms exp(own - own_max) where it needs it.
template <int QC, bool FAST, bool RAW>
__global__ __launch_bounds__(64 * kBwdWaves) void logmm_bwd_lhs_slab_kernel(const BwdArgs a) {
    constexpr int QLD = QC * TQ + 8;            // bfloat16 per LDS row: rows 4 banks apart
    constexpr int KB = kBwdSlab / 16, NW = kBwdWaves, NT = 64 * NW;
    extern __shared__ __attribute__((aligned(16))) __bf16 s_e[];   // [3][kBwdSlab][QLD]
    // the slabs of one batch entry on one XCD, next to each other in time (see
    // xcd_tile): together they read whole rows of E_own and write whole rows of
    // the gradient, through one L2
    const TileId tile = xcd_tile(a.tiles_x, 1);
    const int b = tile.b, k0 = tile.x * kBwdSlab;
    if (b >= a.B) return;
    const int P = a.P, Q = a.Q, K = a.K, Kp = a.Kp;
    const int Pb = a.p_len ? min(max(a.p_len[b], 0) + a.p_extra, P) : P;
    const int Qb = a.q_len ? min(max(a.q_len[b], 0) + a.q_extra, Q) : Q;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    float *db = a.grad + (size_t)b * a.dsb;
    const bool vec = a.dsk == 1 && (a.dsp & 3) == 0 && (a.dsb & 3) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.grad) & 15u) == 0;
    // the slab of E_oth, transposed and split: element e is (row q, 4 columns k),
    // q the fast index: neighbouring lanes then write neighbouring bfloat16 of an
    // LDS row (with k the fast index all lanes of a store hit 4 banks)
    for (int e = tid; e < QC * TQ * (kBwdSlab / 4); e += NT) {
        const int k4 = (e / (QC * TQ)) * 4, q = e % (QC * TQ);
        v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
        if (q < Qb && k0 + k4 < Kp)
            v = *reinterpret_cast<const v4f *>(a.Eoth + ((size_t)b * Q + q) * Kp + k0 + k4);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const Split3 sp = split3(v[i]);
            __bf16 *at = s_e + (size_t)(k4 + i) * QLD + q;
            at[0] = sp.h;
            at[(size_t)kBwdSlab * QLD] = sp.m;
            at[(size_t)2 * kBwdSlab * QLD] = sp.l;
        }
    }
    __syncthreads();
    const int row_blocks = (P + 15) / 16;
    const int *fl = a.flags + (size_t)b * P;
    const int Cq = a.cgp;                       // row length of C
    // A wavefront asks for everything a block of rows needs (its rows of C, and
    // E_own at its lane's 4 columns of every 16) at the top of the block; the
    // second workgroup of the CU covers the wait.  Measured and dropped: a second
    // set of registers, so that a block's rows are requested while the block
    // before it is worked on (64 us instead of 62: what a wavefront waits for is
    // mostly its own earlier stores, which retire in order with its loads), and
    // 8 wavefronts with E_own requested per 16 columns (73 us), and slabs of 64
    // columns, which let three workgroups share a compute unit (71 us).
    for (int rb = wave; rb < row_blocks; rb += NW) {
        const int p = rb * 16 + c, pl = min(p, P - 1);
        const float *crow = a.C + (size_t)b * a.csb + (size_t)pl * Cq + 8 * g;
        v4f cv[2 * QC], ev[KB];
#pragma unroll
        for (int ch = 0; ch < QC; ++ch) {
            cv[2 * ch] = *reinterpret_cast<const v4f *>(crow + TQ * ch);
            cv[2 * ch + 1] = *reinterpret_cast<const v4f *>(crow + TQ * ch + 4);
        }
        const float *erow = RAW ? a.own + (size_t)b * a.osb + (size_t)pl * a.osp
                                : a.Eown + ((size_t)b * P + pl) * Kp;
        const float own_max = RAW ? a.own_max[(size_t)b * P + pl] : 0.0f;
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
            ev[kb] = *reinterpret_cast<const v4f *>(erow + min(k0 + kb * 16 + 4 * g, Kp - 4));
        bf16x8 cp[QC][3];
#pragma unroll
        for (int ch = 0; ch < QC; ++ch)
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const Split3 sp = split3(i < 4 ? cv[2 * ch][i] : cv[2 * ch + 1][i - 4]);
                cp[ch][0][i] = sp.h, cp[ch][1][i] = sp.m, cp[ch][2][i] = sp.l;
            }
        const float own_shift = finite_or_zero(own_max);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb) {
            v4f acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int ch = 0; ch < QC; ++ch) {
                bf16x8 ep[3];
#pragma unroll
                for (int pn = 0; pn < 3; ++pn)
                    ep[pn] = *reinterpret_cast<const bf16x8 *>(
                        s_e + ((size_t)pn * kBwdSlab + kb * 16 + c) * QLD + TQ * ch + 8 * g);
                acc = mfma6(ep, cp[ch], acc);
            }
            // register q holds (k = k0 + kb*16 + 4g + q, row p)
            const int k = k0 + kb * 16 + 4 * g;
            v4f v;
#pragma unroll
            for (int q = 0; q < 4; ++q)
                v[q] = scaled_sum(acc[q], RAW ? exp2_hw((ev[kb][q] - own_shift) * kLog2eF) : ev[kb][q]);
            float *dst = db + (size_t)p * a.dsp + (size_t)k * a.dsk;
            if (FAST) {
                *reinterpret_cast<v4f *>(dst) = v;
            } else if (p < P && k < K) {
                if (vec && k + 3 < K) {
                    *reinterpret_cast<v4f *>(dst) = v;
                } else {
#pragma unroll
                    for (int q = 0; q < 4; ++q)
                        if (k + q < K) dst[(size_t)q * a.dsk] = v[q];
                }
            }
            // (left alone the scheduler hoists the LDS reads of all 16-column
            // blocks to the top and spills)
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // rows with pairs that C left out (exponent beyond the shifted range): their
    // terms are added one by one, to what this lane has stored
    for (int rb = wave; rb < row_blocks; rb += NW) {
        const int p = rb * 16 + c;
        const int flagged = (p < Pb) ? fl[min(p, P - 1)] : 0;
        if (!__any(flagged)) continue;
        if (!flagged) continue;
        for (int kb = 0; kb < KB; ++kb)
            for (int q = 0; q < 4; ++q) {
                const int k = k0 + kb * 16 + 4 * g + q;
                if (k < K) db[(size_t)p * a.dsp + (size_t)k * a.dsk] += exact_pairs(a, b, p, k, Qb);
            }
    }
}

// The end of the kernel below: the sums of a wavefront (lane l holds
// D[p = ub*16 + 4*(l/16) + q][k = kb*16 + l%16] in register q) times E_own, to
// the gradient.  All of a lane's values of E_own are requested before the first
// is used (one round trip to memory; asked for one by one, inside the
// conditions, each load was waited for by itself: 48 round trips, 15 us).
template <int UB>
__device__ __forceinline__ void rhs_store_sums(const BwdArgs &a, int b, int k0, int wave, int c,
                                               int g, const v4f (&acc)[2][UB], bool slow, int Pb,
                                               int Qb) {
    const int P = a.P, K = a.K, Kp = a.Kp;
    float eo[2][UB][4];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
        const int k = min(k0 + (2 * wave + kk) * 16 + c, Kp - 1);
#pragma unroll
        for (int ub = 0; ub < UB; ++ub)
#pragma unroll
            for (int q = 0; q < 4; ++q)
                eo[kk][ub][q] = a.Eown[((size_t)b * P + min(ub * 16 + 4 * g + q, P - 1)) * Kp + k];
    }
    float *db = a.grad + (size_t)b * a.dsb;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
        const int k = k0 + (2 * wave + kk) * 16 + c;
        if (k >= K) continue;
#pragma unroll
        for (int ub = 0; ub < UB; ++ub)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int p = ub * 16 + 4 * g + q;
                if (p >= P) continue;
                float v = (p < Pb) ? scaled_sum(acc[kk][ub][q], eo[kk][ub][q]) : 0.0f;
                if (slow && p < Pb) v += exact_pairs(a, b, p, k, Qb);
                db[(size_t)p * a.dsp + (size_t)k * a.dsk] = v;
            }
    }
}

// The gradient of the operand with FEW rows and a LONG reduction (the g of a
// joiner: P = labels + 1 <= 96, Q = frames, K = vocabulary):
//   grad[b,p,k] = E_own[p,k] * sum_q C[q,p] * E_oth[q,k].
// The output is small; the product is bound by streaming E_oth once.  A
// workgroup of 4 wavefronts takes one batch entry and kRhsSlab columns k and
// keeps its (16*UB x kRhsSlab) sums in registers (a wavefront: 32 columns).  The
// reduction runs in chunks of 32 rows q.  Both operands have q as their ROW
// index in memory, the matrix instruction wants 8 consecutive q per lane.
constexpr int kRhsSlab = 128;
constexpr int kRhsLd = TQ + 8;       // bfloat16 per LDS row (80 bytes: rows 4 banks apart)

// Nothing is split or transposed for C on the way: the pair
// factors arrive as bfloat16 planes with the frames contiguous (written once by
// logmm_pair_factor_planes_kernel), and a lane takes its 8 frames of one column
// k of the long operand straight from memory, one 4-byte load per frame (the 16
// lanes of a column block read 64 contiguous bytes of a row), exponentiates
// (RAW) and splits them in registers: they are its share of the matrix
// instruction's second operand as they are.  Only the planes of C pass through
// LDS (a plain copy, two buffers, one barrier per chunk of 32 frames); the long
// operand never does, and no value is split more than once per workgroup.
// Per chunk a lane issues ~150 vector instructions and 72 matrix instructions.
// (Before: both operands loaded row-wise as 16-byte vectors, split, and written
// to LDS transposed, two barriers per chunk: ~350 vector instructions per chunk
// and lane, 52 us where this kernel takes 39.)
template <int UB, bool RAW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void logmm_bwd_rhs_planes_kernel(const BwdArgs a) {
    constexpr int NT = 256, DEPTH = 2;
    constexpr int ROWS = 16 * UB;
    constexpr int CV = 3 * ROWS * 4;               // 16-byte vectors of one chunk of the planes
    constexpr int CPT = (CV + NT - 1) / NT;        // ... per thread (the last ones repeat)
    __shared__ __attribute__((aligned(16))) __bf16 s_ct[2][3][ROWS][kRhsLd];
    __shared__ int s_unsafe;
    const TileId tile = xcd_tile(a.tiles_x, 1);
    const int b = tile.b, k0 = tile.x * kRhsSlab;
    if (b >= a.B) return;
    const int P = a.P, Q = a.Q, Kp = a.Kp, Tp = a.ct_frames;
    const int Pb = a.p_len ? min(max(a.p_len[b], 0) + a.p_extra, P) : P;
    const int Qb = a.q_len ? min(max(a.q_len[b], 0) + a.q_extra, Q) : Q;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int c = lane & 15, g = lane >> 4;
    if (tid == 0) s_unsafe = 0;
    __syncthreads();
    {
        const int *fl = a.flags + (size_t)b * Q;
        int unsafe = 0;
        for (int q = tid; q < Qb; q += NT) unsafe |= fl[q];
        if (unsafe) s_unsafe = 1;
    }
    const int n = (Qb + TQ - 1) / TQ, last_chunk = Tp / TQ - 1;
    // the planes: vector e of a chunk is (plane, row u, 8 frames j)
    const unsigned short *ct_src[CPT];
    int ct_dst[CPT];
#pragma unroll
    for (int it = 0; it < CPT; ++it) {
        const int e = min(tid + it * NT, CV - 1);
        const int pl = e / (ROWS * 4), u = (e >> 2) % ROWS, j = e & 3;
        ct_src[it] = a.ct + (((size_t)pl * a.B + b) * a.ct_rows + u) * Tp + 8 * j;
        ct_dst[it] = (pl * ROWS + u) * kRhsLd + 8 * j;
    }
    auto ct_fetch = [&](int chunk, u32x4 (&v)[CPT]) {
        const int t0 = min(chunk, last_chunk) * TQ;
#pragma unroll
        for (int it = 0; it < CPT; ++it) v[it] = *reinterpret_cast<const u32x4 *>(ct_src[it] + t0);
    };
    auto ct_put = [&](int buf, const u32x4 (&v)[CPT]) {
        __bf16 *dst = &s_ct[buf][0][0][0];
#pragma unroll
        for (int it = 0; it < CPT; ++it) *reinterpret_cast<u32x4 *>(dst + ct_dst[it]) = v[it];
    };
    // the long operand: this lane's column of each of the wavefront's two blocks
    // of 16 (a pair of blocks beyond the reduction repeats the last pair: its
    // sums are dropped), frames 8g .. 8g+7 of the chunk; frames beyond the
    // entry's length repeat its last one (C is 0 there, and RAW their shift +inf)
    const int kc = min(k0 + 32 * wave, Kp - 32) + c;
    const float *e_base = RAW ? a.oth + (size_t)b * a.tsb : a.Eoth + (size_t)b * Q * Kp;
    const int e_row = RAW ? a.tsq : Kp;
    const int q_last = RAW ? max(Qb - 1, 0) : Q - 1;
    const float *shift_base = a.ct_shift + (size_t)b * Tp + 8 * g;
    auto fetch = [&](int chunk, float (&x)[2][8], v4f (&sf)[2]) {
        const int t0 = min(chunk, last_chunk) * TQ;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            // (offsets inside one batch entry fit 32 bits: the launcher checks)
            const unsigned off = (unsigned)(min(t0 + 8 * g + i, q_last) * e_row + kc);
            x[0][i] = e_base[off];
            x[1][i] = e_base[off + 16];
        }
        if (RAW) {
            sf[0] = *reinterpret_cast<const v4f *>(shift_base + t0);
            sf[1] = *reinterpret_cast<const v4f *>(shift_base + t0 + 4);
        }
    };
    v4f acc[2][UB];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int ub = 0; ub < UB; ++ub) acc[kk][ub] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    float e[DEPTH][2][8];
    v4f sf[DEPTH][2];
    u32x4 cr[CPT];
    // (requested in the order of the loop: the compiler counts the loads in
    // flight at the head of the loop along both ways into it)
    static_assert(DEPTH == 2, "the order of the requests below is that of a loop two chunks deep");
    ct_fetch(0, cr);
    __builtin_amdgcn_sched_barrier(0);
    ct_put(0, cr);
    fetch(0, e[0], sf[0]);
    __builtin_amdgcn_sched_barrier(0);
    ct_fetch(1, cr);
    __builtin_amdgcn_sched_barrier(0);
    fetch(1, e[1], sf[1]);
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    // one chunk: `cur` even works from buffer 0 and register set 0
    auto half = [&](int cur, int buf, float (&ex)[2][8], v4f (&es)[2]) {
        // the next chunk's planes into the buffer that the chunk before read
        // (everyone has passed the barrier behind it), the one after it requested
        ct_put(buf ^ 1, cr);
        ct_fetch(cur + 2, cr);
        // (held in this order: requested behind the loads of the long operand,
        // the planes would be waited for with nothing else left in flight)
        __builtin_amdgcn_sched_barrier(0);
        bf16x8 bk[2][3];
#pragma unroll
        for (int kk = 0; kk < 2; ++kk) {
            float x[8];
#pragma unroll
            for (int i = 0; i < 8; ++i)
                x[i] = RAW ? exp2_hw((ex[kk][i] - es[i >> 2][i & 3]) * kLog2eF) : ex[kk][i];
            const Pair3 p0 = split3_pair(x[0], x[1]), p1 = split3_pair(x[2], x[3]);
            const Pair3 p2 = split3_pair(x[4], x[5]), p3 = split3_pair(x[6], x[7]);
            const u32x4 h = {p0.h, p1.h, p2.h, p3.h};
            const u32x4 m = {p0.m, p1.m, p2.m, p3.m};
            const u32x4 l = {p0.l, p1.l, p2.l, p3.l};
            bk[kk][0] = __builtin_bit_cast(bf16x8, h);
            bk[kk][1] = __builtin_bit_cast(bf16x8, m);
            bk[kk][2] = __builtin_bit_cast(bf16x8, l);
        }
        fetch(cur + DEPTH, ex, es);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ub = 0; ub < UB; ++ub) {
            bf16x8 au[3];
#pragma unroll
            for (int pn = 0; pn < 3; ++pn)
                au[pn] = *reinterpret_cast<const bf16x8 *>(&s_ct[buf][pn][ub * 16 + c][8 * g]);
#pragma unroll
            for (int kk = 0; kk < 2; ++kk) acc[kk][ub] = mfma6(au, bk[kk], acc[kk][ub]);
        }
        __syncthreads();
    };
    // two chunks per trip and no way out of the loop between them: with one, the
    // compiler would count the loads in flight along a path that skips the second
    // chunk, and wait for loads that were only just issued
    int chunk = 0;
    for (; chunk + 1 < n; chunk += 2) {
        half(chunk, 0, e[0], sf[0]);
        half(chunk + 1, 1, e[1], sf[1]);
    }
    if (chunk < n) half(chunk, 0, e[0], sf[0]);
    __syncthreads();
    rhs_store_sums<UB>(a, b, k0, wave, c, g, acc, s_unsafe != 0, Pb, Qb);
}

// Tiles of 64 or 96 along an extent, whichever pads the tiled extent less.
inline bool prefer_96(int extent) {
    return (extent + 95) / 96 * 96 < (extent + 63) / 64 * 64;
}

bool fits_int(long extent) { return extent >= 0 && extent < 0x7fffffffL; }
bool stride_ok(long s) { return s >= 0 && s < 0x7fffffffL; }

// grad[b, p, k] = 0 through the gradient's strides: the gradient of an empty reduction
__global__ __launch_bounds__(256) void logmm_bwd_zero_kernel(BwdArgs a) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= (long)a.P * a.K) return;
    const int p = (int)(i / a.K), k = (int)(i - (long)p * a.K);
    a.grad[(size_t)blockIdx.y * a.dsb + (size_t)p * a.dsp + (size_t)k * a.dsk] = 0.0f;
}

// 4 wavefronts per workgroup: 64 rows p (one 16-row block per wavefront, all 64
// columns) or 96 rows p (all rows, 16 columns per wavefront) by 64 columns k
hipError_t launch_bwd(const BwdArgs &args, int B, hipStream_t stream) {
    BwdArgs a = args;
    a.B = B;
    if (B == 0 || a.P == 0 || a.K == 0) return hipSuccess;
    if (a.Q == 0) {
        const long cells = (long)a.P * a.K;
        if (!fits_int((cells + 255) / 256)) return hipErrorInvalidValue;
        TIMED_LAUNCH(logmm_bwd_zero_kernel, dim3((unsigned)((cells + 255) / 256), B),
                           dim3(256), 0, stream, a);
        return hipGetLastError();
    }
    // offsets inside one batch are 32-bit in the kernel
    if (!fits_int((long)(a.P - 1) * a.osp + (long)(a.K - 1) * a.osk + 1) ||
        !fits_int((long)(a.Q - 1) * a.tsq + (long)(a.K - 1) * a.tsk + 1) ||
        !fits_int((long)(a.P - 1) * a.dsp + (long)(a.K - 1) * a.dsk + 1) ||
        !fits_int((long)a.P * a.Q))
        return hipErrorInvalidValue;
    if (a.cgq == 1 && a.Q <= 3 * TQ && a.Kp >= 2 * kBwdSlab) {
        // short reduction, rows of C contiguous in it (the gradient of the operand
        // with many rows): the slab of E_oth resident, E_own and the gradient
        // streamed once
        const int qc = (a.Q + TQ - 1) / TQ;
        a.tiles_x = (a.Kp + kBwdSlab - 1) / kBwdSlab, a.tiles_y = 1;
        if (!xcd_grid_fits(a.tiles_x, 1, B)) return hipErrorInvalidValue;
        const dim3 grid(xcd_grid(a.tiles_x, 1, B));
        const size_t lds = (size_t)3 * kBwdSlab * (qc * TQ + 8) * sizeof(__bf16);
        // whole blocks of rows and whole slabs of columns, 16-byte stores: no
        // bounds to check in the kernel
        const bool fast = a.P % 16 == 0 && a.K % kBwdSlab == 0 && a.dsk == 1 && (a.dsp & 3) == 0 &&
                          (a.dsb & 3) == 0 && (reinterpret_cast<uintptr_t>(a.grad) & 15u) == 0;
        const bool raw = a.Eown == nullptr;
        if (!a.Eoth || (raw && (a.osk != 1 || a.K != a.Kp))) return hipErrorInvalidValue;
#define LAUNCH_LHS_SLAB(QCN)                                                                   \
    do {                                                                                       \
        if (fast && raw)                                                                       \
            TIMED_LAUNCH((logmm_bwd_lhs_slab_kernel<QCN, true, true>), grid, dim3(64 * kBwdWaves), \
                         lds, stream, a);                                                      \
        else if (fast)                                                                         \
            TIMED_LAUNCH((logmm_bwd_lhs_slab_kernel<QCN, true, false>), grid, dim3(64 * kBwdWaves), \
                         lds, stream, a);                                                      \
        else if (raw)                                                                          \
            TIMED_LAUNCH((logmm_bwd_lhs_slab_kernel<QCN, false, true>), grid, dim3(64 * kBwdWaves), \
                         lds, stream, a);                                                      \
        else                                                                                   \
            TIMED_LAUNCH((logmm_bwd_lhs_slab_kernel<QCN, false, false>), grid, dim3(64 * kBwdWaves), \
                         lds, stream, a);                                                      \
    } while (0)
        if (qc == 1)
            LAUNCH_LHS_SLAB(1);
        else if (qc == 2)
            LAUNCH_LHS_SLAB(2);
        else
            LAUNCH_LHS_SLAB(3);
#undef LAUNCH_LHS_SLAB
        return hipGetLastError();
    }
    if (a.ct && a.ct_shift && a.cgp == 1 && a.P <= 96 && a.Kp >= 2 * kRhsSlab && a.Q >= 4 * TQ &&
        a.Eown && (a.Eoth || (a.tsk == 1 && a.K == a.Kp)) &&
        fits_int((long)(a.Q - 1) * (a.Eoth ? a.Kp : a.tsq) + a.Kp)) {
        // the same shapes with C's planes at hand (the joiner's backward)
        const int ub = (a.P + 15) / 16;
        a.tiles_x = (a.Kp + kRhsSlab - 1) / kRhsSlab, a.tiles_y = 1;
        if (!xcd_grid_fits(a.tiles_x, 1, B)) return hipErrorInvalidValue;
        const dim3 grid(xcd_grid(a.tiles_x, 1, B));
        const bool raw = a.Eoth == nullptr;
#define RHS_PLANES(UBN)                                                                         \
    do {                                                                                        \
        if (raw)                                                                                \
            TIMED_LAUNCH((logmm_bwd_rhs_planes_kernel<UBN, true>), grid, dim3(256), 0, stream, a); \
        else                                                                                    \
            TIMED_LAUNCH((logmm_bwd_rhs_planes_kernel<UBN, false>), grid, dim3(256), 0, stream, a); \
    } while (0)
        switch (ub) {
            case 1: RHS_PLANES(1); break;
            case 2: RHS_PLANES(2); break;
            case 3: RHS_PLANES(3); break;
            case 4: RHS_PLANES(4); break;
            case 5: RHS_PLANES(5); break;
            default: RHS_PLANES(6); break;
        }
#undef RHS_PLANES
        return hipGetLastError();
    }
    if (!a.Eown || !a.Eoth) return hipErrorInvalidValue;   // only the slab kernels read an operand itself
    if (a.Q <= QR && !prefer_96(a.P)) {
        // short reduction, many rows: C slab resident, a few k tiles per workgroup
        const int ptiles = (a.P + 63) / 64, ktiles = (a.K + 63) / 64;
        const long wgs = (long)ptiles * ktiles * B;
        const int per = (int)std::min<long>(8, std::max<long>(1, wgs / 2048));
        a.tiles_x = ptiles, a.tiles_y = (ktiles + per - 1) / per;
        if (!xcd_grid_fits(a.tiles_x, a.tiles_y, B)) return hipErrorInvalidValue;
        TIMED_LAUNCH(logmm_bwd_resident_kernel, dim3(xcd_grid(a.tiles_x, a.tiles_y, B)),
                           dim3(256), 0, stream, a, per);
        return hipGetLastError();
    }
    // a reduction of up to 4 chunks (Q <= 128) is fetched whole, up front;
    // longer ones run a pipeline 3 chunks deep
    const bool short_q = a.Q <= 4 * TQ;
    a.tiles_x = prefer_96(a.P) ? (a.P + 95) / 96 : (a.P + 63) / 64;
    a.tiles_y = (a.K + 63) / 64;
    if (!xcd_grid_fits(a.tiles_x, a.tiles_y, B)) return hipErrorInvalidValue;
    const dim3 grid(xcd_grid(a.tiles_x, a.tiles_y, B));
    if (prefer_96(a.P)) {
        if (short_q)
            TIMED_LAUNCH((logmm_bwd_kernel<6, 1, 1, 4, 4, false>), grid, dim3(256), 0,
                               stream, a);
        else
            TIMED_LAUNCH((logmm_bwd_kernel<6, 1, 1, 4, 3, true>), grid, dim3(256), 0, stream,
                               a);
    } else {
        if (short_q)
            TIMED_LAUNCH((logmm_bwd_kernel<1, 4, 4, 1, 4, false>), grid, dim3(256), 0,
                               stream, a);
        else
            TIMED_LAUNCH((logmm_bwd_kernel<1, 4, 4, 1, 3, true>), grid, dim3(256), 0, stream,
                               a);
    }
    return hipGetLastError();
}

}  // namespace

namespace {

// rows r of x[b, r, k] with strides (sb, sr, sk), see shift_exp_kernel
void launch_shift_exp_rows(const float *x, long sb, long sr, long sk, int B, int R, int K, int Kp,
                           const int *len, int extra, float *mx, float *E, hipStream_t stream) {
    const dim3 grid((R + 3) / 4, B), block(256);
    const bool rows_ok = sk == 1 && K >= 4 && (K & 3) == 0 && (sb & 3) == 0 && (sr & 3) == 0 &&
                         (reinterpret_cast<uintptr_t>(x) & 15u) == 0;
    if (rows_ok && K <= 1024) {
        TIMED_LAUNCH(shift_exp_rows_kernel<4>, grid, block, 0, stream, x, sb, sr, R, K, Kp,
                           len, extra, mx, E);
    } else if (rows_ok && K <= 2048) {
        TIMED_LAUNCH(shift_exp_rows_kernel<8>, grid, block, 0, stream, x, sb, sr, R, K, Kp,
                           len, extra, mx, E);
    } else if (rows_ok && K <= 4096) {
        TIMED_LAUNCH(shift_exp_rows_kernel<16>, grid, block, 0, stream, x, sb, sr, R, K, Kp,
                           len, extra, mx, E);
    } else if (rows_ok && K <= 8192) {
        TIMED_LAUNCH(shift_exp_rows_kernel<32>, grid, block, 0, stream, x, sb, sr, R, K, Kp,
                           len, extra, mx, E);
    } else {
        TIMED_LAUNCH(shift_exp_kernel, grid, block, 0, stream, x, sb, sr, sk, R, K, Kp, len,
                           extra, mx, E);
    }
}

}  // namespace

// Whether all three products of these shapes go to the slab kernels, which can
// read lhs itself: few columns, a reduction of 512..2048 in whole chunks, at
// least 128 rows, lhs contiguous along the reduction in 16-byte aligned rows.
// (Mirrors the conditions in launch_logmm_fwd and launch_bwd.)
bool logmm_reads_lhs_itself(const LogmmOperand &lhs, int M, int K, int Nn) {
    return Nn >= 1 && Nn <= 3 * TQ && K >= 2 * kSlab && K <= 8 * kSlab && K % TQ == 0 &&
           M >= 4 * TQ && lhs.s2 == 1 && (lhs.s1 & 3) == 0 && (lhs.sb & 3) == 0 &&
           (reinterpret_cast<uintptr_t>(lhs.p) & 15u) == 0;
}

hipError_t launch_logmm_shift_exp(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                  const LogmmShifted &sh, int B, int M, int K, int Nn,
                                  const int *row_len, const int *col_len, hipStream_t stream) {
    const int Kp = logmm_padded_reduction(K);
    if (B == 0 || Kp == 0) return hipSuccess;
    // (an operand that the kernels read themselves has its maxima taken by the
    // forward: launch_logmm_fwd must follow)
    if (M > 0 && sh.El) {
        launch_shift_exp_rows(lhs.p, lhs.sb, lhs.s1, lhs.s2, B, M, K, Kp, row_len, 0, sh.lmax,
                              sh.El, stream);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    if (Nn > 0) {
        // rhs[b,k,j]: the rows are j (stride s2), k has stride s1
        launch_shift_exp_rows(rhs.p, rhs.sb, rhs.s2, rhs.s1, B, Nn, K, Kp, col_len, 1, sh.rmax,
                              sh.Er, stream);
    }
    return hipGetLastError();
}

size_t logmm_fwd_partial_floats(int B, int M, int Nn) {
    // up to 8 partial sums of whole row blocks (16) and column tiles (96 or 64)
    // and of 8 slab maxima per row
    const int tn = prefer_96(Nn) ? 96 : 64;
    const size_t pM = (size_t)(M + 15) / 16 * 16;
    return (size_t)8 * B * pM * ((Nn + tn - 1) / tn * tn) + (size_t)8 * B * pM;
}

int logmm_fwd_splits(int B, int M, int K, int Nn) {
    // only when there are fewer tiles than CUs (the extra pass over the partial sums costs as
    // much as it gains otherwise), and at least 2*kDepth chunks each
    const int chunks = logmm_padded_reduction(K) / TQ;
    const long tiles = (long)((M + 31) / 32) * ((Nn + 95) / 96) * B;
    int splits = 1;
    while (splits < 8 && tiles * splits < 256 && chunks / (splits * 2) >= 2 * kDepth) splits *= 2;
    return splits;
}

hipError_t launch_logmm_fwd(const LogmmOperand &lhs, const LogmmOperand &rhs,
                            const LogmmShifted &sh, float *res, float *partial, int B, int M,
                            int K, int Nn, const int *row_len, const int *col_len,
                            LogmmDeferred *defer, hipStream_t stream) {
    if (defer) *defer = LogmmDeferred{};
    if (B == 0 || M == 0 || Nn == 0) return hipSuccess;
    FwdArgs a;
    a.splits = partial ? logmm_fwd_splits(B, M, K, Nn) : 1;
    a.partial = partial;
    a.chunks_per_split = (logmm_padded_reduction(K) / TQ + a.splits - 1) / a.splits;
    if (a.chunks_per_split < 1) a.chunks_per_split = 1;
    a.El = sh.El, a.Er = sh.Er, a.lmax = sh.lmax, a.rmax = sh.rmax;
    a.lhs = lhs.p, a.lsb = lhs.sb, a.lsm = lhs.s1, a.lsk = lhs.s2;
    a.rhs = rhs.p, a.rsb = rhs.sb, a.rsk = rhs.s1, a.rsn = rhs.s2;
    a.res = res, a.M = M, a.K = K, a.Kp = logmm_padded_reduction(K), a.Nn = Nn;
    a.pM = M, a.pN = Nn;
    a.row_len = row_len, a.col_len = col_len;
    a.B = B;
    // few columns, long reduction, room for the partial sums: one slab of E_r
    // resident per workgroup, E_l streamed once
    const bool slab_form = partial && a.Kp >= 2 * kSlab && a.Kp <= 8 * kSlab && Nn <= 8 * 96;
    if (slab_form) {
        const int slabs = (a.Kp + kSlab - 1) / kSlab;   // <= 8: one partial sum each
        a.splits = slabs;
        const bool wide = prefer_96(Nn);
        const int tn = wide ? 96 : 64;
        a.pM = (M + 15) / 16 * 16, a.pN = (Nn + tn - 1) / tn * tn;
        a.tiles_x = slabs, a.tiles_y = (Nn + tn - 1) / tn;
        if (!xcd_grid_fits(a.tiles_x, a.tiles_y, B)) return hipErrorInvalidValue;
        const dim3 grid(xcd_grid(a.tiles_x, a.tiles_y, B));
        const size_t lds = (size_t)3 * tn * kSlabLd * sizeof(__bf16);
        const bool raw = a.El == nullptr;
        if (raw && (a.lsk != 1 || a.K != a.Kp)) return hipErrorInvalidValue;
        if (raw) {
            // the slabs' sums are taken against maxima of their own: only a caller
            // that finishes them itself (logmm_finish_cell) can use this form
            if (!defer) return hipErrorInvalidValue;
            a.slab_max = partial + (size_t)slabs * B * a.pM * a.pN;   // behind the partial sums
        }
        if (wide && raw)
            TIMED_LAUNCH((logmm_fwd_slab_kernel<6, true>), grid, dim3(64 * kSlabWaves), lds, stream, a, slabs);
        else if (wide)
            TIMED_LAUNCH((logmm_fwd_slab_kernel<6, false>), grid, dim3(64 * kSlabWaves), lds, stream, a, slabs);
        else if (raw)
            TIMED_LAUNCH((logmm_fwd_slab_kernel<4, true>), grid, dim3(64 * kSlabWaves), lds, stream, a, slabs);
        else
            TIMED_LAUNCH((logmm_fwd_slab_kernel<4, false>), grid, dim3(64 * kSlabWaves), lds, stream, a, slabs);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
        if (raw) {   // the pass over the slabs' sums is the caller's next kernel's
            *defer = LogmmDeferred{partial, a.slab_max, sh.rmax, slabs, B, a.pM, a.pN, Nn};
            return hipSuccess;
        }
        const long outs = (long)M * Nn;
        TIMED_LAUNCH(logmm_fwd_finish_kernel, dim3((unsigned)((outs + 255) / 256), B), dim3(256),
                     0, stream, a, B);
        return hipGetLastError();
    }
    if (!a.El) return hipErrorInvalidValue;     // only the slab form reads lhs itself
    // 4 wavefronts per workgroup: 32 rows i by 96 or 64 columns j
    a.tiles_x = (M + 31) / 32;
    a.tiles_y = (prefer_96(Nn) ? (Nn + 95) / 96 : (Nn + 63) / 64) * a.splits;
    if (!xcd_grid_fits(a.tiles_x, a.tiles_y, B)) return hipErrorInvalidValue;
    const dim3 grid(xcd_grid(a.tiles_x, a.tiles_y, B));
    if (prefer_96(Nn))
        TIMED_LAUNCH((logmm_fwd_kernel<1, 3, 2, 2>), grid, dim3(256), 0, stream, a);
    else
        TIMED_LAUNCH((logmm_fwd_kernel<1, 2, 2, 2>), grid, dim3(256), 0, stream, a);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || a.splits == 1) return e;
    const long outs = (long)M * Nn;
    TIMED_LAUNCH(logmm_fwd_finish_kernel, dim3((unsigned)((outs + 255) / 256), B), dim3(256),
                       0, stream, a, B);
    return hipGetLastError();
}

// The planes serve the gradient of the operand with few rows where it has at
// most 96 of them and the other at least 128 (the shapes of launch_bwd's branch).
static bool pair_planes_apply(int M, int Nn) { return Nn >= 1 && Nn <= 3 * TQ && M >= 4 * TQ; }
size_t logmm_pair_planes_bytes(int B, int M, int Nn) {
    if (!pair_planes_apply(M, Nn)) return 0;
    const size_t bytes = (size_t)3 * B * logmm_pair_row(Nn) * logmm_pair_frames(M) * sizeof(unsigned short);
    return (bytes + 255) / 256 * 256;
}
size_t logmm_pair_shifts_bytes(int B, int M, int Nn) {
    if (!pair_planes_apply(M, Nn)) return 0;
    return ((size_t)B * logmm_pair_frames(M) * sizeof(float) + 255) / 256 * 256;
}

hipError_t launch_logmm_pair_factor(const float *go, const float *res, const float *lmax,
                                    const float *rmax, const Weight &weight, float *weights_out,
                                    const int *row_len, const int *col_len, float *C, int *flags,
                                    const LogmmPairPlanes &planes, int B, int M, int Nn,
                                    hipStream_t stream) {
    if (B == 0 || M == 0) return hipSuccess;
    if (planes.planes && planes.shifts && pair_planes_apply(M, Nn)) {
        const int frames = logmm_pair_frames(M);
        TIMED_LAUNCH(logmm_pair_factor_planes_kernel, dim3(frames / (8 * kPairRowsPerWave), B),
                     dim3(512), 0, stream, go,
                     res, lmax, rmax, weight, weights_out, row_len, col_len, C, flags, planes.planes,
                     planes.shifts, B, M, Nn, frames);
        return hipGetLastError();
    }
    TIMED_LAUNCH(logmm_pair_factor_kernel, dim3((M + 3) / 4, B), dim3(256), 0, stream, go,
                       res, lmax, rmax, weight, weights_out, row_len, col_len, C, flags, M, Nn);
    return hipGetLastError();
}

hipError_t launch_logmm_bwd_lhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const LogmmShifted &sh, const float *go, const float *res,
                                const float *C, const int *flags, const LogmmGrad &grad, int B,
                                int M, int K, int Nn, const int *row_len, const int *col_len,
                                const float *batch_scale, hipStream_t stream) {
    if (B == 0 || M == 0 || K == 0) return hipSuccess;
    if (!stride_ok(lhs.s1) || !stride_ok(lhs.s2) || !stride_ok(rhs.s1) || !stride_ok(rhs.s2) ||
        !stride_ok(grad.s1) || !stride_ok(grad.s2))
        return hipErrorInvalidValue;
    // own = lhs[b,i,k]; oth[q=j][k] = rhs[b,k,j]; C/go/res[i,j]: p stride Nn, q stride 1
    BwdArgs a;
    a.Eown = sh.El, a.Eoth = sh.Er;
    a.own = lhs.p, a.osb = lhs.sb, a.osp = (int)lhs.s1, a.osk = (int)lhs.s2;
    a.oth = rhs.p, a.tsb = rhs.sb, a.tsq = (int)rhs.s2, a.tsk = (int)rhs.s1;
    a.own_max = sh.lmax, a.oth_max = sh.rmax;
    a.C = C, a.go = go, a.res = res, a.gsb = (long)M * Nn, a.gp = Nn, a.gq = 1;
    a.csb = (long)M * logmm_pair_row(Nn), a.cgp = logmm_pair_row(Nn), a.cgq = 1;
    a.flags = flags, a.flags_follow_p = 1;
    a.grad = grad.p, a.dsb = grad.sb, a.dsp = (int)grad.s1, a.dsk = (int)grad.s2;
    a.P = M, a.Q = Nn, a.K = K, a.Kp = logmm_padded_reduction(K);
    a.p_len = row_len, a.p_extra = 0, a.q_len = col_len, a.q_extra = 1;
    a.batch_scale = batch_scale;
    return launch_bwd(a, B, stream);
}

hipError_t launch_logmm_bwd_rhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const LogmmShifted &sh, const float *go, const float *res,
                                const float *C, const int *flags, const LogmmPairPlanes &planes,
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
    a.Eown = sh.Er, a.Eoth = sh.El;
    a.own = rhs.p, a.osb = rhs.sb, a.osp = (int)rhs.s2, a.osk = (int)rhs.s1;
    a.oth = lhs.p, a.tsb = lhs.sb, a.tsq = (int)lhs.s1, a.tsk = (int)lhs.s2;
    a.own_max = sh.rmax, a.oth_max = sh.lmax;
    a.C = C, a.go = go, a.res = res, a.gsb = (long)M * Nn, a.gp = 1, a.gq = Nn;
    a.csb = (long)M * logmm_pair_row(Nn), a.cgp = 1, a.cgq = logmm_pair_row(Nn);
    a.flags = flags, a.flags_follow_p = 0;
    a.grad = grad.p, a.dsb = grad.sb, a.dsp = (int)grad.s2, a.dsk = (int)grad.s1;
    a.P = Nn, a.Q = M, a.K = K, a.Kp = logmm_padded_reduction(K);
    a.p_len = col_len, a.p_extra = 1, a.q_len = row_len, a.q_extra = 0;
    a.batch_scale = batch_scale;
    if (planes.planes && planes.shifts && pair_planes_apply(M, Nn)) {
        a.ct = planes.planes, a.ct_shift = planes.shifts;
        a.ct_rows = logmm_pair_row(Nn), a.ct_frames = logmm_pair_frames(M);
    }
    return launch_bwd(a, B, stream);
}

}  // namespace wctct
