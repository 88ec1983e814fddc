// Internal launch interface between the C-ABI layer (api.hip) and the kernel
// translation units.  Plain structs of device pointers and sizes; each
// launcher enqueues on the given stream and returns hipGetLastError().
#pragma once

#include <hip/hip_runtime.h>

#include "profile.h"

namespace wctct {

// Work buffers (units, alphas, betas) hold P = padded_contexts(U) contexts per
// frame, a multiple of the wavefront size, so that the lattice sweep loads and
// stores without lane masks.
inline int padded_contexts(int U) { return ((U + 1 + 63) / 64) * 64; }

// Element type of the joint tensor / its dense gradient (values of the C ABI).
enum IoType { kIoF32 = 0, kIoF16 = 1, kIoBF16 = 2 };
inline size_t io_size(int t) { return t == kIoF32 ? 4 : 2; }
inline bool io_valid(int t) { return t == kIoF32 || t == kIoF16 || t == kIoBF16; }

// Bits of the device's sticky status word (WARPCTCT_STATUS_* of the C ABI).
constexpr unsigned kStatusLabelRange = 1u;     // a label outside [0, V) was clamped
constexpr unsigned kStatusNanInput = 2u;       // a gathered log-probability was NaN
constexpr unsigned kStatusLostHandOver = 4u;   // a chain of workgroups gave up waiting
constexpr unsigned kStatusLinearFellBack = 8u; // the joiner's linear lattices were computed again in the log domain
// The current device's status word, for kernels to set bits in (atomic OR), or
// null when it cannot be found (kernels then report nothing).
unsigned *device_status_word();

// Per-sample weight of the upstream gradient: grad_out[n * stride] (stride 0
// broadcasts a scalar), times `scale` (1/N for reduction='mean'), divided by
// lx[n] when the loss was averaged over frames (warp_ctct/__init__.py:138-147
// of the reference, differentiated).
struct Weight {
    const float *grad_out;   // null = ones
    int stride;
    float scale;
    int average_frames;
};

// Reduction over the batch folded into the lattice kernel: the workgroup that
// finishes last (counted in *counter, which must be 0 at launch) adds up the N
// costs in a fixed order.  mode 0 = none, 1 = sum, 2 = mean.
struct CostReduce {
    float *reduced;       // 1 float, or null
    unsigned *counter;
    int mode;
    int average_frames;   // costs[n] /= lx[n] before anything else
};

// Memory to clear inside another kernel's launch: n4 vectors of 16 bytes at p
// (16-byte aligned).  Workgroups appended to that launch each store 256 vectors
// and retire, while the kernel's own workgroups, which are bound by latency and
// leave the memory system idle, do their work.
struct FillTail {
    void *p = nullptr;
    size_t n4 = 0;
};

struct LatticeArgs {
    const double *units;  // (N,T,P,3) log2 units, neutral values in the padding
    const int *ys;        // (N,U)
    const int *lx;        // (N)
    const int *ly;        // (N)
    double *alphas;       // (N,T+1,P,2) log2 units, or null if beta_only
    double *betas;        // (N,T+1,P,2) log2 units
    float *costs;         // (N)
    void *relay;          // lattice_relay_slots(N,T,U) 64-bit words, or null if there are none
    bool relay_is_clear;  // every slot already holds kRelayEmpty (see RelaySlots)
    int N, T, U;
    bool beta_only;
    CostReduce reduce;    // zero-initialise for plain per-sample costs
    FillTail fill;        // cleared beside the sweeps (default: nothing)
};

// A lattice of more than 64 contexts is swept by a chain of workgroups that
// hand one value per frame and 64-context boundary through device memory:
// the number of 64-bit slots that takes (0 for U + 1 <= 64).
size_t lattice_relay_slots(int N, int T, int U);
// What a slot holds before its value has been stored: a NaN with a payload that
// no arithmetic produces.
constexpr unsigned long long kRelayEmpty = 0x7ff8dead5107e117ULL;
// The slots of a lattice launch, for the kernel that runs before it on the same
// stream to clear on the side (a launch of its own for a few hundred KB costs
// more than the stores): every thread of that kernel's grid calls
// relay_clear_share first thing, before it may return.
struct RelaySlots {
    unsigned long long *p = nullptr;
    size_t n = 0;
};
inline RelaySlots relay_slots_of(void *relay, int N, int T, int U) {
    RelaySlots r;
    r.n = relay ? lattice_relay_slots(N, T, U) : 0;
    r.p = r.n ? static_cast<unsigned long long *>(relay) : nullptr;
    return r;
}
__device__ __forceinline__ void relay_clear_share(const RelaySlots &r) {
    if (r.n == 0) return;
    const size_t block = (size_t)blockIdx.z * gridDim.y * gridDim.x + (size_t)blockIdx.y * gridDim.x + blockIdx.x;
    const size_t threads = (size_t)blockDim.x * blockDim.y * blockDim.z;
    const size_t me = block * threads + (size_t)threadIdx.z * blockDim.y * blockDim.x +
                      (size_t)threadIdx.y * blockDim.x + threadIdx.x;
    const size_t all = threads * gridDim.x * gridDim.y * gridDim.z;
    for (size_t i = me; i < r.n; i += all) r.p[i] = kRelayEmpty;
}
// How often a consumer asks again for a hand-over that has not arrived before
// it declares its input lost (0: the first look decides; negative: the
// default, about a second).  Applies to launches made afterwards; returns the
// previous limit.
int lattice_wait_limit(int spins);
int lattice_wait_limit_now();   // the limit in force
// only_if (may be null): the kernel returns at once while *only_if is 0 (see
// launch_lattice_lin: the log-domain lattices as the fall-back of the linear ones)
hipError_t launch_lattice(const LatticeArgs &a, hipStream_t stream, const unsigned *only_if = nullptr);

// ---- the joiner's lattices in the linear domain (lattice_lin.hip) -------------
// Sweeps on path masses relative to a power of two per wavefront and chunk of
// kLinChunk frames.  A wavefront holds kLinReal contexts in its lanes 1..62;
// lane 0 / lane 63 stand for the context below / above, whose wavefront hands
// its boundary value over THROUGH THE UNITS: context u lives in column
// lin_column(u) of the lin_padded(U) columns that units, alphas and betas have
// here, and the columns in between belong to those two lanes.
//   units  (N,T,Pl,kLinUnit): {blank, label, next label} as linear factors
//          ({0,0,0} in padding and outside the band of complete alignments: mass
//          that gets there is gone, instead of sitting there undiminished and
//          dictating the wavefront's scale); written by
//          launch_simple_gather_units_lin, which also sets up the columns in
//          between; the sweeps write what they hand over into them
//   alphas, betas (N,T+1,Pl,2): pairs {o, e} of masses
//   scales: lattice_lin_scales(N,T,U) exponents, entry
//          ((n*2 + d)*W + w)*(lin_chunks(T) + 1) + i,   d = 0: beta, 1: alpha,
//          W = lin_waves(U), i = 0 for the initial row (alpha: frame 0, beta:
//          frame Tn) and i = 1 + step / kLinChunk for the row stored by that
//          step (alpha: step = frame - 1, beta: step = Tn - 1 - frame)
// *flag is raised where a hand-over was lost.  The results are only meaningful
// together with the check of the kernel that reads them (launch_simple_grads_lin).
constexpr int kLinChunk = 12;
constexpr int kLinReal = 62;
constexpr int kLinUnit = 3;
__host__ __device__ inline int lin_chunks(int T) { return (T + kLinChunk - 1) / kLinChunk; }
__host__ __device__ inline int lin_waves(int U) { return (U + kLinReal) / kLinReal; }   // U + 1 contexts
__host__ __device__ inline int lin_padded(int U) { return 64 * lin_waves(U); }
__host__ __device__ inline int lin_column(int u) { return u + 2 * (u / kLinReal) + 1; }
size_t lattice_lin_scales(int N, int T, int U);
// a.units, a.alphas, a.betas: the buffers described above; a.relay is not used
hipError_t launch_lattice_lin(const LatticeArgs &a, int *scales, unsigned *flag, hipStream_t stream);

// Element strides of a joint tensor (N,T,U+1,V); dense row-major is
// {T*(U+1)*V, (U+1)*V, V, 1}.
struct JointStrides {
    long n, t, u, v;
};
inline JointStrides dense_joint_strides(int T, int U, int V) {
    return JointStrides{(long)T * (U + 1) * V, (long)(U + 1) * V, (long)V, 1L};
}

// band_only: cells outside the band of complete alignments get neutral units
// (same costs and gradients; alpha / beta of dead cells are not the oracle's)
// counter (may be null): set to 0 by the kernel, for a CostReduce that follows;
// relay: slots cleared by the kernel, for the lattice launch that follows
hipError_t launch_gather_units(const void *joint, const JointStrides &strides, int io_type,
                               const int *ys, const int *lx, const int *ly, double *units, int N,
                               int T, int U, int V, bool band_only, unsigned *counter,
                               const RelaySlots &relay, hipStream_t stream);
hipError_t launch_clear_counter(unsigned *counter, hipStream_t stream);
hipError_t launch_scale_units(const float *units_nat, const int *lx, const int *ly, double *units,
                              int N, int T, int U, hipStream_t stream);
hipError_t launch_simple_units(const float *f_g, const float *g_g, const float *den,
                               const int *lx, const int *ly, double *units, int N, int T, int U,
                               hipStream_t stream);
hipError_t launch_unit_grads(const double *units, const int *ys, const int *lx, const int *ly,
                             const double *alphas, const double *betas, float *unit_grads, int N,
                             int T, int U, hipStream_t stream);
// dense = zeros, then the patch (two launches on the same stream)
hipError_t launch_dense_grad(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                             const float *grad_out, float *dense, int N, int T, int U, int V,
                             hipStream_t stream);
// only the <= 3 non-zero entries per live row, into a tensor that holds zeros
hipError_t launch_dense_patch(const float *unit_grads, const int *ys, const int *lx,
                              const int *ly, const float *grad_out, float *dense, int N, int T,
                              int U, int V, hipStream_t stream);

// the same with the unit gradients computed on the fly from the work buffers
// and the upstream gradient given as grad_out[n*stride] * scale (/ lx[n])
hipError_t launch_dense_patch_lattice(const double *units, const double *alphas,
                                      const double *betas, const int *ys, const int *lx,
                                      const int *ly, const float *grad_out, int grad_out_stride,
                                      float scale, int average_frames, void *dense, int io_type,
                                      int N, int T, int U, int V, hipStream_t stream);

// ---- ctct_loss on logits (log_softmax inside) --------------------------------
// units + lse (N,T,U+1) from the logits; counter as in launch_gather_units
hipError_t launch_logits_units(const void *logits, int io_type, const int *ys, const int *lx,
                               const int *ly, double *units, float *lse, int N, int T, int U,
                               int V, unsigned *counter, hipStream_t stream);
// dense gradient wrt the logits, every element written
hipError_t launch_logits_grad(const void *logits, int io_type, const float *lse,
                              const double *units, const double *alphas, const double *betas,
                              const int *ys, const int *lx, const int *ly, const float *grad_out,
                              int grad_out_stride, float scale, int average_frames, void *grad,
                              int N, int T, int U, int V, hipStream_t stream);

// ---- log-add joiner path -------------------------------------------------
// The last pass of a log-matmul forward left to the kernel that reads the
// product first: where launch_logmm_fwd fills this in (partial != null), res and
// the row maxima of lhs have NOT been written yet; that kernel computes each
// res[b,i,j] with logmm_finish_cell (logmm_finish.h), and writes res and the
// maxima.
struct LogmmDeferred {
    const float *partial;    // (splits, B, pM, pN): the slabs' sums; null: nothing deferred
    const float *slab_max;   // (splits, B, pM): maxima of the rows of lhs inside the slabs
    const float *rmax;       // (B, Nn)
    int splits, B, pM, pN, Nn;
};
// den (N,T,U+1): read, or, with `deferred.partial`, computed from the deferred
// pass and written, together with fmax (N,T) (-inf for frames beyond lx).
// only_if (may be null): the kernel returns at once while *only_if is 0.
hipError_t launch_simple_gather_units(const float *f, const float *g, float *den, const int *ys,
                                      const int *lx, const int *ly, double *units, int N, int T,
                                      int U, int V, const RelaySlots &relay,
                                      const LogmmDeferred &deferred, float *fmax,
                                      unsigned *counter, hipStream_t stream,
                                      const unsigned *only_if = nullptr);
// The same for the sweeps in the linear domain: units as launch_lattice_lin
// wants them (see there); *flag is lowered.
hipError_t launch_simple_gather_units_lin(const float *f, const float *g, float *den, const int *ys,
                                          const int *lx, const int *ly, double *units, int N, int T,
                                          int U, int V, const LogmmDeferred &deferred, float *fmax,
                                          unsigned *counter, unsigned *flag, hipStream_t stream);
// compact gradients of the joiner path straight from the lattices: grad_f
// (N,T,U+1), grad_g (N,U+1,3), grad_den (N,T,U+1) or null; `partial` is scratch
// of N * T * (U+1) * 3 floats (partial sums over blocks of 8 frames, or, for
// lattices of more than 512 contexts, the unit gradients themselves)
hipError_t launch_simple_grads(const double *units, const int *ys, const int *lx, const int *ly,
                               const double *alphas, const double *betas, float *partial,
                               float *grad_f, float *grad_g, float *grad_den, int N, int T, int U,
                               hipStream_t stream, const unsigned *only_if = nullptr);
// The same from lattices in the linear domain, without the last sum over the
// blocks of frames (launch_simple_grads with only_if behind it does that sum
// whether it recomputes or not); raises *flag where the linear lattices cannot
// be trusted (posteriors of a frame not adding up to 1, a unit out of range,
// anything not finite).  units, alphas, betas, scales: as launch_lattice_lin
// describes them.  Needs simple_grads_lin_applies(T, U).
bool simple_grads_lin_applies(int T, int U);
hipError_t launch_simple_grads_lin(const double *units, const int *ys, const int *lx, const int *ly,
                                   const double *alphas, const double *betas, const int *scales,
                                   float *partial, float *grad_f, float *grad_den, int N, int T,
                                   int U, unsigned *flag, hipStream_t stream);
hipError_t launch_simple_reduce(const float *unit_grads, float *grad_f, float *grad_g,
                                float *grad_den, int N, int T, int U, hipStream_t stream);
// dense_f and dense_g of the unnormalised path in one pass (zeros + scattered
// compact gradients, whole rows); only for rows that fit into LDS
bool simple_dense_rows_fit(int V);
hipError_t launch_simple_dense_rows(const float *grad_f, const float *grad_g, const int *ys,
                                    const int *lx, const int *ly, const Weight &weight,
                                    float *dense_f, float *dense_g, int N, int T, int U, int V,
                                    hipStream_t stream);
// weights[n] = grad_out[n * stride] * scale (/ lx[n] with average_frames), see Weight
hipError_t launch_sample_weights(const Weight &weight, const int *lx, float *weights, int N,
                                 hipStream_t stream);
hipError_t launch_simple_scatter(const float *grad_f, const float *grad_g, const int *ys,
                                 const int *lx, const int *ly, const float *grad_out,
                                 float *dense_f, float *dense_g, int N, int T, int U, int V,
                                 hipStream_t stream);
hipError_t launch_zero_fill(float *p, size_t n, hipStream_t stream);
hipError_t launch_zero_fill_bytes(void *p, size_t bytes, hipStream_t stream);

// ---- log-semiring matmul -------------------------------------------------
// A strided 3-d operand: element [b, i1, i2] lives at p[b*sb + i1*s1 + i2*s2].
// lhs is (B,M,K), rhs is (B,K,Nn); a gradient uses the layout of its operand.
struct LogmmOperand {
    const float *p;
    long sb, s1, s2;
};
struct LogmmGrad {
    float *p;
    long sb, s1, s2;
};

// The reduction index of the shifted exponentials is padded to a multiple of
// the GEMM chunk (32) with zeros.
inline int logmm_padded_reduction(int K) { return (K + 31) / 32 * 32; }

// Shifted exponentials of both operands and the shifts:
//   lmax (B,M) = max_k lhs, El (B,M,Kp) = exp(lhs - lmax);
//   rmax (B,Nn) = max_k rhs, Er (B,Nn,Kp) = exp(rhs - rmax) with k contiguous.
struct LogmmShifted {
    float *lmax, *rmax, *El, *Er;
};
// El may be null where logmm_reads_lhs_itself(...) holds: launch_logmm_shift_exp
// then writes the maxima only, and the forward (with `partial`) and both gradients
// read lhs itself and exponentiate it on the way (one pass over lhs less per
// forward, and no (B,M,Kp) buffer).
bool logmm_reads_lhs_itself(const LogmmOperand &lhs, int M, int K, int Nn);

// row_len / col_len (may be null): per-batch number of valid rows of lhs and
// index of the last valid column of rhs; outputs outside are not computed.
hipError_t launch_logmm_shift_exp(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                  const LogmmShifted &sh, int B, int M, int K, int Nn,
                                  const int *row_len, const int *col_len, hipStream_t stream);
// partial (may be null): logmm_fwd_partial_floats(B,M,Nn) floats of scratch; with it the
// reduction of a small output is split over several workgroups per tile
int logmm_fwd_splits(int B, int M, int K, int Nn);
// Row length, in floats, of the pair-factor buffer C of the backward: Nn rounded
// up to the reduction chunk (32), zeros in the padding.
__host__ __device__ inline int logmm_pair_row(int Nn) { return (Nn + 31) / 32 * 32; }
// floats of `partial` that launch_logmm_fwd may use, whatever K is
size_t logmm_fwd_partial_floats(int B, int M, int Nn);
// `defer` (null unless lhs is read itself, sh.El == nullptr, which requires it):
// the forward's last pass is not launched and *defer describes it
// (LogmmDeferred above); for a stored El, defer->partial is null afterwards.
hipError_t launch_logmm_fwd(const LogmmOperand &lhs, const LogmmOperand &rhs,
                            const LogmmShifted &sh, float *res, float *partial, int B, int M,
                            int K, int Nn, const int *row_len, const int *col_len,
                            LogmmDeferred *defer, hipStream_t stream);
// The pair factors once more, laid out for the gradient of the operand with few
// rows (see logmm_bwd_rhs_planes_kernel): transposed and split into three
// bfloat16 planes (3, B, logmm_pair_row(Nn), logmm_pair_frames(M)), frames
// contiguous, zeros beyond M; and per frame the shift of its row of lhs
// (B, logmm_pair_frames(M)): the finite row maximum, +inf for padding.
// Both null: not wanted.
struct LogmmPairPlanes {
    unsigned short *planes;
    float *shifts;
};
inline int logmm_pair_frames(int M) { return (M + 31) / 32 * 32; }
// bytes of the two buffers (each a multiple of 256), 0 where the planes have no use
size_t logmm_pair_planes_bytes(int B, int M, int Nn);
size_t logmm_pair_shifts_bytes(int B, int M, int Nn);
// C (B,M,logmm_pair_row(Nn)) and flags (B,M): the pair factors go * exp(lmax + rmax - res) that
// both gradients share, and per row whether a pair was left to the exact pass;
// `weight` (with row_len as the frame counts) multiplies grad_out per batch
// entry, and is left in weights_out[b] (may be null) for the kernels that follow.
hipError_t launch_logmm_pair_factor(const float *go, const float *res, const float *lmax,
                                    const float *rmax, const Weight &weight, float *weights_out,
                                    const int *row_len, const int *col_len, float *C, int *flags,
                                    const LogmmPairPlanes &planes, int B, int M, int Nn,
                                    hipStream_t stream);
hipError_t launch_logmm_bwd_lhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const LogmmShifted &sh, const float *go, const float *res,
                                const float *C, const int *flags, const LogmmGrad &grad, int B,
                                int M, int K, int Nn, const int *row_len, const int *col_len,
                                const float *batch_scale, hipStream_t stream);
hipError_t launch_logmm_bwd_rhs(const LogmmOperand &lhs, const LogmmOperand &rhs,
                                const LogmmShifted &sh, const float *go, const float *res,
                                const float *C, const int *flags, const LogmmPairPlanes &planes,
                                const LogmmGrad &grad, int B, int M, int K, int Nn,
                                const int *row_len, const int *col_len, const float *batch_scale,
                                hipStream_t stream);

}  // namespace wctct
