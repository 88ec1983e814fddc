/* C ABI of libwarpctct_hip.so — the MI355X (gfx950) CTC-Transducer loss kernels.
 *
 * Every entry point takes plain device pointers, sizes and a HIP stream
 * (passed as void*; NULL = the null stream), launches asynchronously on that
 * stream, never synchronises with the host, never allocates, and returns 0
 * or a WARPCTCT_E* code (never exits the process, unlike CHECK_KERNEL_STAT
 * at csrc/core.h:5-12 of the reference).  The caller owns every buffer.
 *
 * Shapes use the reference's names: N lattices, T = max frames, U = max
 * labels (the joint has U+1 contexts), V = vocabulary, blank = 0.  Tensors
 * are dense row-major.  "units" are the three entries per cell (t,u) that
 * the lattice uses: k=0 blank, k=1 label y[u-1], k=2 label y[u]
 * (csrc/gather.cu:16-21 of the reference).
 *
 * Internally the lattice works on log2 values held in double ("units",
 * alphas, betas below), in work buffers whose context dimension is padded to
 * P = warpctct_padded_contexts(U), a multiple of the 64-lane wavefront.  These
 * intermediates are private to the library (the reference's alphas/betas are
 * private too); unit gradients and costs are returned as fp32 in natural-log
 * units exactly like the reference.
 */
#ifndef WARP_CTCT_HIP_H
#define WARP_CTCT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* The library is built with hidden symbol visibility; the entry points declared
 * here are its whole exported surface. */
#if defined(__GNUC__)
#pragma GCC visibility push(default)
#endif

enum {
    WARPCTCT_OK = 0,
    WARPCTCT_EINVAL = 1,     /* null pointer, negative size, or beyond N <= 65535,
                                T * (U+1 rounded up to 64) < 2^31 */
    WARPCTCT_ELAUNCH = 2,    /* hipGetLastError() reported a failed launch */
    WARPCTCT_EWORKSPACE = 3, /* workspace smaller than warpctct_workspace_bytes() */
    WARPCTCT_ENODEVICE = 4,  /* no usable HIP device */
    WARPCTCT_ETOOLARGE = 5   /* needs more than WARPCTCT_STATIC_SCRATCH_BYTES of work buffers */
};

/* Human-readable text for a return code (static storage). */
const char *warpctct_error_string(int code);

/* Version of this C ABI, "major.minor.patch"; independent of the Python
 * distribution's version, which follows the reference distribution. */
const char *warpctct_version(void);

/* Contexts per frame in the work buffers: the smallest multiple of 64 that is
 * >= U+1. */
int warpctct_padded_contexts(int U);

/* Bytes of device workspace the two *_forward orchestrators need
 * (units, alpha and beta lattices, all double, and the relay slots of
 * lattices wider than 64 contexts).  Replaces the
 * allocations of csrc/binding.cpp:70-77 (alphas, betas, counts); needs no
 * host sync because it does not depend on max(lx-ly) (binding.cpp:68). */
size_t warpctct_workspace_bytes(int N, int T, int U);

/* ---- stage entry points (each replaces one reference stage) ------------ */

/* Gather of the three units per live cell out of the joint tensor, scaled
 * to log2 units.  Replaces warp_ctct/__init__.py:124-131 (index build +
 * torch.gather).  joint (N,T,U+1,V) f32, ys (N,U) i32, lx/ly (N) i32,
 * units_out (N,T,P,3) f64.  Cells with t>=lx[n] or u>ly[n] are not read;
 * for t<lx[n] the contexts u>ly[n] (up to P-1) receive the neutral units
 * {0,0,-inf}; frames t>=lx[n] are not written. */
int warpctct_gather_units_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              double *units_out, int N, int T, int U, int V, void *stream);

/* Same for an already gathered (N,T,U+1,3) natural-log tensor, i.e. the
 * `log_probs` argument of _C.ctct_loss_fwd (csrc/binding.cpp:31-35). */
int warpctct_scale_units_f32(const float *units_nat, const int *lx, const int *ly,
                             double *units_out, int N, int T, int U, void *stream);

/* Units of the log-add joiner, LP = f + g - den (den may be NULL for the
 * unnormalised variant).  Replaces the LOGPROBY/LOGPROBB macros of
 * csrc/simple.cu:20-26 and csrc/simple_unnorm.cu:20-25.
 * f_g (N,T,U+1), g_g (N,U+1,3), den (N,T,U+1) or NULL. */
int warpctct_simple_units_f32(const float *f_g, const float *g_g, const float *den,
                              const int *lx, const int *ly, double *units_out,
                              int N, int T, int U, void *stream);

/* Alpha and beta lattices of all N samples, concurrently, one wavefront per
 * (sample, direction, 64 contexts).  Replaces run_warp_ctct (csrc/core.h:14-16,
 * csrc/gather.cu:293-309: k_warp_alphas + k_warp_betas).
 * units (N,T,P,3) f64 log2 domain; alphas, betas (N,T+1,P,2) f64 =
 * {state 2u-1, state 2u} (only t<=lx[n], and only the 64-context blocks that
 * hold a context u<=ly[n], are written); costs (N) f32
 * = -beta(0,0) in natural-log units (csrc/binding.cpp:86).
 * beta_only != 0 skips alpha (alphas may be NULL), as binding.cpp:84.
 * relay: warpctct_lattice_relay_bytes(N,T,U) bytes of scratch, 8-byte aligned,
 * through which the wavefronts of a lattice of more than 64 contexts hand
 * over their boundary values (0 bytes, relay may be NULL, for U+1 <= 64; it
 * replaces the `counts` spin-lock array of csrc/binding.cpp:77).  Should a
 * hand-over ever not arrive within its bounded wait, the workgroup that waited
 * stops, writes NaN into the rows of alpha / beta that it has not swept and
 * tells the workgroups behind it in the chain, which do the same: every
 * gradient computed from those rows is NaN, and so is the cost when the beta
 * chain is affected.  No plausible number comes out of a lattice that was not
 * swept to the end.
 * warpctct_lattice_wait_limit(spins): how often a waiting workgroup asks again
 * before it gives up (0: the first look decides; negative: back to the default,
 * about a second of polling); applies to launches made afterwards, returns the
 * previous limit.  The limit is one value for the whole process (every thread's
 * later launches see it) and exists for tests; production code leaves it alone.
 * It has no counterpart in the reference, whose spin lock
 * (csrc/gather.cu:88, :106, :171) is unbounded; tests use it to exercise the give-up
 * path with kernels that still run to their end. */
size_t warpctct_lattice_relay_bytes(int N, int T, int U);
int warpctct_lattice_wait_limit(int spins);
int warpctct_lattice_f32(const double *units, const int *ys, const int *lx, const int *ly,
                         double *alphas, double *betas, float *costs, int N, int T, int U,
                         int beta_only, void *relay, size_t relay_bytes, void *stream);

/* d(cost)/d(unit) for every cell, natural-log units, zero outside
 * t<lx[n], u<=ly[n].  Replaces run_fill_grad + the zeros_like before it
 * (csrc/core.h:18-20, csrc/gather.cu:311-387, csrc/binding.cpp:89).
 * unit_grads (N,T,U+1,3). */
int warpctct_unit_grads_f32(const double *units, const int *ys, const int *lx, const int *ly,
                            const double *alphas, const double *betas, float *unit_grads, int N,
                            int T, int U, void *stream);

/* Dense gradient wrt the joint: dense (N,T,U+1,V) = zeros, except
 * grad_out[n] * unit gradient at columns 0, y[u-1], y[u] of every live row
 * (coincident columns add).  Replaces CTCTLoss.backward
 * (warp_ctct/__init__.py:30-33) and autograd's gather backward (zeros +
 * scatter_add).  grad_out (N) f32 or NULL (= ones).  Two launches: a pure
 * zero-fill at full HBM write bandwidth, then the sparse patch. */
int warpctct_dense_grad_f32(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                            const float *grad_out, float *dense, int N, int T, int U, int V,
                            void *stream);

/* The sparse half of warpctct_dense_grad_f32 alone: dense must already hold
 * zeros (e.g. from warpctct_zero_fill_f32 run earlier on another stream, since
 * the fill does not depend on the lattice).  The non-zero elements are written,
 * not added, and when rows are a whole number of 128-byte lines the zeros of
 * the line around each of them are written again with it. */
int warpctct_dense_patch_f32(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                             const float *grad_out, float *dense, int N, int T, int U, int V,
                             void *stream);

/* ---- orchestrators ----------------------------------------------------- */

/* ctct_loss forward on the un-gathered joint: gather, lattice, unit grads.
 * Replaces warp_ctct/__init__.py:124-136 + _C.ctct_loss_fwd
 * (csrc/binding.cpp:31-100).  unit_grads may be NULL (no-grad mode). */
int warpctct_loss_forward_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              int N, int T, int U, int V, void *workspace,
                              size_t workspace_bytes, float *costs, float *unit_grads,
                              void *stream);

/* Element types of the joint tensor and of its dense gradient. */
#define WARPCTCT_F32 0
#define WARPCTCT_F16 1
#define WARPCTCT_BF16 2

/* ctct_loss forward as the Python function uses it: gather + lattices on a
 * joint of type `dtype` (the reference converts to float after its gather,
 * warp_ctct/__init__.py:124-136; here the conversion happens in the gather's
 * loads), with the reduction of warp_ctct/__init__.py:138-147 folded in:
 * costs[n] is divided by lx[n] if average_frames, and for reduction 1 (sum)
 * or 2 (mean) *reduced receives the sum or mean over the batch, added in a
 * fixed order (reduction 0: reduced is ignored).  The workspace holds what
 * warpctct_dense_grad_lattice needs and must be kept until it has run.
 * want_alpha == 0 is the no-grad mode (beta only). */
int warpctct_loss_lattice(const void *joint, int dtype, const int *ys, const int *lx,
                          const int *ly, int N, int T, int U, int V, void *workspace,
                          size_t workspace_bytes, float *costs, int want_alpha, int reduction,
                          int average_frames, float *reduced, void *stream);

/* The same for a joint that is a strided view: element [n,t,u,v] lives at
 * joint[n*strides[0] + t*strides[1] + u*strides[2] + v*strides[3]] (in
 * elements; strides may be zero or negative as long as every address stays
 * inside the caller's buffer).  The reference's torch.gather works on such
 * views directly (warp_ctct/__init__.py:131); this avoids a copy of the joint. */
int warpctct_loss_lattice_strided(const void *joint, int dtype, const long *strides,
                                  const int *ys, const int *lx, const int *ly, int N, int T, int U,
                                  int V, void *workspace, size_t workspace_bytes, float *costs,
                                  int want_alpha, int reduction, int average_frames,
                                  float *reduced, void *stream);

/* warpctct_loss_lattice_strided that also clears the buffer of the dense
 * gradient, dense_bytes bytes at `dense`, for warpctct_dense_patch_lattice to
 * write into later (the reference forms its dense gradient inside autograd:
 * the backward of torch.gather, warp_ctct/__init__.py:131, zero-fills the
 * joint's shape and scatters into it).  The clear rides in the launch of the
 * lattice kernel, as extra workgroups behind the sweeps: those wait on chains
 * of dependent arithmetic and leave the memory system idle, the clear is pure
 * write traffic, so the sweeps cost no time of their own.  Everything runs on
 * `stream`.  dense == NULL or dense_bytes == 0: nothing to clear. */
int warpctct_loss_lattice_clearing(const void *joint, int dtype, const long *strides,
                                   const int *ys, const int *lx, const int *ly, int N, int T,
                                   int U, int V, void *workspace, size_t workspace_bytes,
                                   float *costs, int want_alpha, int reduction, int average_frames,
                                   float *reduced, void *dense, size_t dense_bytes, void *stream);

/* Dense gradient of type `dtype` from that workspace (see
 * warpctct_dense_grad_lattice_f32 below for the weights); values are summed in
 * fp32 and rounded once to nearest even. */
int warpctct_dense_grad_lattice(const void *workspace, size_t workspace_bytes, const int *ys,
                                const int *lx, const int *ly, const float *grad_out,
                                int grad_out_stride, float scale, int average_frames, void *dense,
                                int dtype, int N, int T, int U, int V, void *stream);
int warpctct_dense_patch_lattice(const void *workspace, size_t workspace_bytes, const int *ys,
                                 const int *lx, const int *ly, const float *grad_out,
                                 int grad_out_stride, float scale, int average_frames, void *dense,
                                 int dtype, int N, int T, int U, int V, void *stream);

/* p[0..bytes) = 0 with a kernel (one 16-byte store per thread; safe to capture
 * in a HIP graph). */
int warpctct_zero_fill(void *p, size_t bytes, void *stream);

/* warpctct_loss_forward_f32 (below) for a joint of type `dtype`: costs and the
 * compact unit gradients (N,T,U+1,3) fp32, i.e. what _C.ctct_loss_fwd of the
 * reference returns (csrc/binding.cpp:31-100), computed from the un-gathered
 * joint.  For callers that own the joiner and apply the gradient themselves
 * instead of receiving the dense (N,T,U+1,V) tensor. */
int warpctct_loss_forward(const void *joint, int dtype, const int *ys, const int *lx,
                          const int *ly, int N, int T, int U, int V, void *workspace,
                          size_t workspace_bytes, float *costs, float *unit_grads, void *stream);

/* warpctct_loss_forward without a workspace argument, for callers that cannot
 * allocate device memory (code under HIP graph capture, tight serving loops,
 * harnesses that forbid hipMalloc).  It has no counterpart in the reference.
 * The work buffers (units, alpha, beta) live in a device array of
 * WARPCTCT_STATIC_SCRATCH_BYTES that is part of the library's code object, one
 * copy per GPU, held until the process ends; the call allocates and frees
 * nothing.  A problem whose warpctct_workspace_bytes(N,T,U) exceeds that size
 * is refused with WARPCTCT_ETOOLARGE before anything is launched.  All calls
 * on one GPU share that GPU's array: calls that overlap on one GPU (two
 * streams, two host threads) race and must be serialised by the caller.  The
 * array's address is looked up on the first call on each device
 * (hipGetSymbolAddress); make that call outside a graph capture. */
#define WARPCTCT_STATIC_SCRATCH_BYTES (32u << 20)
int warpctct_loss_forward_static(const void *joint, int dtype, const int *ys, const int *lx,
                                 const int *ly, int N, int T, int U, int V, float *costs,
                                 float *unit_grads, void *stream);

/* ---- ctct_loss on logits --------------------------------------------------
 * The step before the reference's path fused into it: a caller of the
 * reference computes log_probs = logits.log_softmax(-1) and passes it to
 * warp_ctct.ctct_loss (warp_ctct/__init__.py:88-147); here the row-wise
 * logsumexp is taken inside the gather and the backward of log_softmax inside
 * the kernel that writes the dense gradient, so the log-probability tensor and
 * its gradient never exist.  Same arguments and results as
 * warpctct_loss_lattice / warpctct_dense_grad_lattice, with logits (N,T,U+1,V)
 * in place of the joint and d(loss)/d(logits) in place of the dense gradient;
 * the workspace is larger (it also holds the logsumexp of every live row). */
size_t warpctct_logits_workspace_bytes(int N, int T, int U);
int warpctct_logits_loss_lattice(const void *logits, int dtype, const int *ys, const int *lx,
                                 const int *ly, int N, int T, int U, int V, void *workspace,
                                 size_t workspace_bytes, float *costs, int want_alpha,
                                 int reduction, int average_frames, float *reduced, void *stream);
int warpctct_logits_grad_lattice(const void *workspace, size_t workspace_bytes,
                                 const void *logits, int dtype, const int *ys, const int *lx,
                                 const int *ly, const float *grad_out, int grad_out_stride,
                                 float scale, int average_frames, void *grad_logits, int N, int T,
                                 int U, int V, void *stream);

/* The same without unit gradients: gather + lattices only.  The workspace then
 * holds everything the dense gradient needs (units, alpha, beta) and must be
 * kept until warpctct_dense_grad_lattice_f32 has run.  want_alpha == 0 is the
 * no-grad mode (beta only). */
int warpctct_loss_lattice_f32(const float *joint, const int *ys, const int *lx, const int *ly,
                              int N, int T, int U, int V, void *workspace, size_t workspace_bytes,
                              float *costs, int want_alpha, void *stream);

/* Dense gradient straight from that workspace: zero-fill, then per live cell
 * the unit gradients are computed on the fly and written to columns 0, y[u-1],
 * y[u].  Sample n is weighted by grad_out[n*grad_out_stride] * scale
 * (/ lx[n] if average_frames): stride 0 with scale 1/N is the backward of
 * reduction='mean', stride 1 with scale 1 of reduction='none'
 * (warp_ctct/__init__.py:138-147 differentiated; CTCTLoss.backward :30-33;
 * gather backward).  grad_out NULL = ones. */
int warpctct_dense_grad_lattice_f32(const void *workspace, size_t workspace_bytes, const int *ys,
                                    const int *lx, const int *ly, const float *grad_out,
                                    int grad_out_stride, float scale, int average_frames,
                                    float *dense, int N, int T, int U, int V, void *stream);

/* Its sparse half alone, into a tensor that already holds zeros. */
int warpctct_dense_patch_lattice_f32(const void *workspace, size_t workspace_bytes, const int *ys,
                                     const int *lx, const int *ly, const float *grad_out,
                                     int grad_out_stride, float scale, int average_frames,
                                     float *dense, int N, int T, int U, int V, void *stream);

/* _C.ctct_loss_fwd proper: the input is already gathered (N,T,U+1,3). */
int warpctct_loss_forward_units_f32(const float *units_nat, const int *ys, const int *lx,
                                    const int *ly, int N, int T, int U, void *workspace,
                                    size_t workspace_bytes, float *costs, float *unit_grads,
                                    void *stream);

/* ---- log-add joiner path (ctct_simple_loss) ------------------------------ */

/* Units straight from the un-gathered operands: f (N,T,V), g (N,U+1,V),
 * den (N,T,U+1) or NULL.  Replaces the two torch.gather calls of
 * warp_ctct/__init__.py:204-215 plus the LOGPROB macros of csrc/simple.cu:20-26. */
int warpctct_simple_gather_units_f32(const float *f, const float *g, const float *den,
                                     const int *ys, const int *lx, const int *ly,
                                     double *units_out, int N, int T, int U, int V, void *stream);

/* Reductions of unit gradients (N,T,U+1,3) that csrc/binding.cpp:198-219 does
 * with ATen: grad_f (N,T,U+1), grad_g (N,U+1,3), grad_den (N,T,U+1) or NULL. */
int warpctct_simple_reduce_f32(const float *unit_grads, float *grad_f, float *grad_g,
                               float *grad_den, int N, int T, int U, void *stream);

/* Backward of the two gathers: dense_f (N,T,V) += grad_out[n]*grad_f at columns
 * [0, y0..y_{U-1}], dense_g (N,U+1,V) += grad_out[n]*grad_g at [0, y[u-1], y[u]]
 * (atomic adds into buffers the caller has initialised).  Either dense pointer
 * may be NULL.  Replaces SimpleCTCTLoss.backward (warp_ctct/__init__.py:76-85)
 * and autograd's gather backward. */
int warpctct_simple_scatter_f32(const float *grad_f, const float *grad_g, const int *ys,
                                const int *lx, const int *ly, const float *grad_out,
                                float *dense_f, float *dense_g, int N, int T, int U, int V,
                                void *stream);

/* p[0..n) = 0 with a kernel (one 16-byte store per thread; safe to capture in
 * a HIP graph). */
int warpctct_zero_fill_f32(float *p, size_t n, void *stream);

/* Bytes of workspace for the two simple_forward orchestrators. */
size_t warpctct_simple_workspace_bytes(int N, int T, int U);

/* ctct_simple_loss forward on f (N,T,V), g (N,U+1,V): den (if normalized),
 * units, lattice, unit gradients and their reductions.  Replaces
 * warp_ctct/__init__.py:195-225 + _C.ctct_loss_simple_fwd
 * (csrc/binding.cpp:103-222).  When normalized != 0, these are outputs that
 * the backward needs (otherwise they are ignored): den (N,T,U+1; only
 * t<lx[n], u<=ly[n] is written), fmax (N,T) = max_v f, gmax (N,U+1) = max_v g,
 * fexp (N,T,Vp) = exp(f - fmax) (see warpctct_simple_needs_fexp) and
 * gexp (N,U+1,Vp) = exp(g - gmax) with
 * Vp = warpctct_logmm_padded_reduction(V), zero in the padding.
 * grad_f/grad_g/grad_den may all be NULL (no-grad mode); without frames
 * (T = 0) grad_f and grad_den have no elements and may be NULL beside a
 * grad_g, which is then cleared. */
/* 0 where the log-matmul kernels of the normalised path read f itself and form
 * exp(f - fmax) on the way (U+1 <= 96 contexts, 512 <= V <= 2048 in whole
 * multiples of 32, T >= 128, f aligned to 16 bytes): fexp is then neither
 * written by the forward nor read by the backward and may be NULL in both,
 * and fmax is written by the kernel that gathers the lattice's inputs (which
 * also finishes den) instead of a pass of its own over f.  1 otherwise.  No counterpart in the reference
 * (which recomputes every exponential in every kernel,
 * csrc/logmatmul.cu:44-146). */
int warpctct_simple_needs_fexp(const float *f, int T, int U, int V);

int warpctct_simple_forward_f32(const float *f, const float *g, const int *ys, const int *lx,
                                const int *ly, int N, int T, int U, int V, int normalized,
                                void *workspace, size_t workspace_bytes, float *den, float *fmax,
                                float *gmax, float *fexp, float *gexp, float *costs,
                                float *grad_f, float *grad_g, float *grad_den, void *stream);

/* The same with the reduction over the batch that ctct_simple_loss applies to
 * the costs (warp_ctct/__init__.py:138-147) folded into the lattice kernel, as
 * in warpctct_loss_lattice: costs[n] is divided by lx[n] if average_frames, and
 * for reduction 1 (sum) or 2 (mean) *reduced receives the sum or mean of the N
 * costs, added in a fixed order (reduction 0: reduced may be NULL). */
int warpctct_simple_forward_reduced_f32(const float *f, const float *g, const int *ys,
                                        const int *lx, const int *ly, int N, int T, int U, int V,
                                        int normalized, void *workspace, size_t workspace_bytes,
                                        float *den, float *fmax, float *gmax, float *fexp,
                                        float *gexp, float *costs, float *grad_f, float *grad_g,
                                        float *grad_den, int reduction, int average_frames,
                                        float *reduced, void *stream);

/* _C.ctct_loss_simple_fwd proper: f_g (N,T,U+1), g_g (N,U+1,3) already
 * gathered, den (N,T,U+1) or NULL (unnormalised, csrc/simple_unnorm.cu). */
int warpctct_simple_forward_units_f32(const float *f_g, const float *g_g, const float *den,
                                      const int *ys, const int *lx, const int *ly, int N, int T,
                                      int U, void *workspace, size_t workspace_bytes, float *costs,
                                      float *grad_f, float *grad_g, float *grad_den, void *stream);

/* Bytes of workspace for warpctct_simple_backward_f32: the factors
 * w*grad_den*exp(fmax+gmax-den) shared by both gradients of the den-path, and,
 * for U+1 <= 96 and T >= 128, the same factors once more as transposed
 * bfloat16 planes for the gradient wrt g. */
size_t warpctct_simple_backward_workspace_bytes(int N, int T, int U);

/* Dense gradients of ctct_simple_loss: dense_f (N,T,V), dense_g (N,U+1,V),
 * every element written.  With den != NULL the den-path
 * (LogMMExp.backward, warp_ctct/__init__.py:45-52) is included:
 * dense_f[t,v] = sum_u w*grad_den[t,u]*exp(f[t,v]+g[u,v]-den[t,u]) + scatter,
 * dense_g likewise summed over t; fmax/gmax/fexp/gexp are the forward's.
 * Either dense pointer may be NULL; workspace is only used with den. */
int warpctct_simple_backward_f32(const float *f, const float *g, const float *den,
                                 const float *fmax, const float *gmax, const float *fexp,
                                 const float *gexp, const float *grad_f,
                                 const float *grad_g, const float *grad_den,
                                 const int *ys, const int *lx, const int *ly,
                                 const float *grad_out, int N, int T, int U, int V,
                                 void *workspace, size_t workspace_bytes, float *dense_f,
                                 float *dense_g, void *stream);

/* The same for a loss that went through warpctct_simple_forward_reduced_f32:
 * sample n is weighted by grad_out[n * grad_out_stride] * scale (/ lx[n] if
 * average_frames); stride 0 with scale 1/N is the backward of reduction 'mean'
 * (warp_ctct/__init__.py:138-147, differentiated; grad_out NULL = ones).
 * weights: N floats of scratch for the kernels that read a plain array of
 * per-sample weights (may be NULL if grad_out already is one: stride 1,
 * scale 1, no average_frames). */
int warpctct_simple_backward_weighted_f32(const float *f, const float *g, const float *den,
                                          const float *fmax, const float *gmax, const float *fexp,
                                          const float *gexp, const float *grad_f,
                                          const float *grad_g, const float *grad_den,
                                          const int *ys, const int *lx, const int *ly,
                                          const float *grad_out, int grad_out_stride, float scale,
                                          int average_frames, float *weights, int N, int T, int U,
                                          int V, void *workspace, size_t workspace_bytes,
                                          float *dense_f, float *dense_g, void *stream);

/* ---- log-semiring matmul -------------------------------------------------- */

/* Row length of the shifted exponentials: K rounded up to the chunk (32) of
 * the matrix-core GEMMs. */
int warpctct_logmm_padded_reduction(int K);

/* Bytes of workspace for warpctct_logmm_fwd_f32 / _bwd_f32: row and column
 * maxima, the operands shifted by them and exponentiated ((B,M,Kp) and
 * (B,Nn,Kp) floats), and the per-pair factors go*exp(lmax+rmax-res) that both
 * gradients share.  Offsets inside one batch of an operand must fit 31 bits
 * (else EINVAL). */
size_t warpctct_logmm_workspace_bytes(int B, int M, int K, int Nn);

/* res[b,i,j] = log sum_k exp(lhs[b,i,k] + rhs[b,k,j]); operands strided in
 * elements (lhs[b,i,k] at lhs[b*lsb + i*lsm + k*lsk], rhs[b,k,j] at
 * rhs[b*rsb + k*rsk + j*rsn]), res contiguous (B,M,Nn).  Replaces
 * log_matmul_cuda (csrc/binding.cpp:224-245, csrc/logmatmul.cu:148-181). */
int warpctct_logmm_fwd_f32(const float *lhs, long lsb, long lsm, long lsk, const float *rhs,
                           long rsb, long rsk, long rsn, int B, int M, int K, int Nn,
                           void *workspace, size_t workspace_bytes, float *res, void *stream);

/* grad_lhs[b,i,k] = sum_j go*exp(lhs+rhs-res), grad_rhs[b,k,j] = sum_i (same);
 * grad_out and res contiguous (B,M,Nn); the gradients use the given element
 * strides; either may be NULL.  Replaces log_matmul_backward
 * (csrc/binding.cpp:247-324). */
int warpctct_logmm_bwd_f32(const float *grad_out, const float *lhs, long lsb, long lsm, long lsk,
                           const float *rhs, long rsb, long rsk, long rsn, const float *res, int B,
                           int M, int K, int Nn, void *workspace, size_t workspace_bytes,
                           float *grad_lhs, long glsb, long glsm, long glsk, float *grad_rhs,
                           long grsb, long grsk, long grsn, void *stream);

/* ---- status word ----------------------------------------------------------
 * Kernels never synchronise with the host, so what the reference reports by
 * raising (torch.gather on a label outside [0, V): warp_ctct/__init__.py:131)
 * is recorded instead in a sticky word on the device, one per GPU:
 *   WARPCTCT_STATUS_LABEL_RANGE    a label outside [0, V) was clamped into it
 *                                  before it was used as a column index;
 *   WARPCTCT_STATUS_NAN_INPUT      a gathered log-probability was NaN; it
 *                                  entered the lattice as log 0 (-inf), so the
 *                                  cost is that of the joint with that entry
 *                                  masked, not NaN as in the reference, whose
 *                                  logaddexpf_ (csrc/gather.cu:23-34) lets a
 *                                  NaN through;
 *   WARPCTCT_STATUS_LOST_HAND_OVER a chain of workgroups gave up waiting for a
 *                                  hand-over (see warpctct_lattice_f32): the NaN
 *                                  costs / gradients of that call do not come
 *                                  from the inputs.
 *   WARPCTCT_STATUS_LINEAR_FELL_BACK  the fused joiner forward swept a batch's
 *                                  lattices in the linear domain, its check
 *                                  refused the result, and the log-domain
 *                                  kernels computed the batch again (the
 *                                  results are those; see
 *                                  warpctct_joiner_linear_lattice).
 * warpctct_status waits for the work queued on the current device
 * (hipDeviceSynchronize: the one entry point that does), copies the word to
 * *bits and, with clear != 0, sets it back to 0.  Bits set by launches that
 * overlap the call may land before or after it. */
enum {
    WARPCTCT_STATUS_LABEL_RANGE = 1,
    WARPCTCT_STATUS_NAN_INPUT = 2,
    WARPCTCT_STATUS_LOST_HAND_OVER = 4,
    WARPCTCT_STATUS_LINEAR_FELL_BACK = 8
};
int warpctct_status(unsigned *bits, int clear);

/* The fused joiner forward (warpctct_simple_forward_f32 / _reduced_f32 with
 * gradients, U + 1 <= 512, long inputs) sweeps its lattices in the LINEAR domain
 * first: path masses relative to one power of two per wavefront (62 contexts)
 * and 12 frames, three multiplications and three additions per frame where the
 * log domain needs two semiring sums per state (half the time per frame; the
 * frames of a lattice are strictly serial, so that is the latency of the whole
 * call).  The linear form drops states that lie ~2^-1000 below the largest of
 * their wavefront.  The kernel that forms the gradients therefore checks that
 * the posteriors of every frame add up to 1 within 2e-5 (lost mass shows there,
 * and so does anything not finite) and that no gathered unit exceeds 2^80; if not,
 * the log-domain kernels, launched behind it in the same stream, compute the
 * batch again (they return at once otherwise), and
 * WARPCTCT_STATUS_LINEAR_FELL_BACK is set.  No counterpart in the reference
 * (csrc/simple.cu sweeps in the log domain).  The linear sweeps save 35-45 ns
 * per frame and cost ~10 us per call (the launches that return at once, a
 * slower gather), so they are used from T = 768 frames on, with normalisation
 * from T = 384 on, and only for batches of up to 768 wavefronts of sweeps
 * (2 N ceil((U+1)/62); up to 256 where a lattice needs one per direction):
 * larger batches are bound by the memory system, where the linear form has
 * nothing to gain.  The rows of these lattices hold the states' high words
 * (20 bits of mantissa): the posteriors formed from them carry a relative error
 * of ~1e-6, the costs none (they come from the sweeps' registers).
 * warpctct_joiner_linear_lattice(n) sets one limit in frames for later calls of
 * the process, which then holds for batches of any size (0: never; 1: always;
 * negative: back to those defaults), and returns the previous setting (negative:
 * the defaults). */
int warpctct_joiner_linear_lattice(int from_frames);

/* ---- measurement aid ------------------------------------------------------
 * No counterpart in the reference.  warpctct_profile(1) clears earlier records
 * and starts bracketing every kernel launch of the library with two HIP events
 * on the launch's own stream; warpctct_profile(0) stops.  After the caller has
 * synchronised, record `index` (0 <= index < warpctct_profile_count(), in
 * launch order) gives the kernel's name (static storage) and its duration.
 * warpctct_profile_filter(text) limits the bracketing to kernels whose name
 * contains `text` (at most 63 characters; NULL or "": every kernel), so that
 * one kernel can be timed inside a timed region at the cost of two events.
 * Creating events allocates: keep it off in production.  Launches into a stream
 * that is under graph capture are not bracketed and leave no record. */
int warpctct_profile(int enable);
int warpctct_profile_filter(const char *text);
int warpctct_profile_count(void);
int warpctct_profile_read(int index, const char **kernel, float *microseconds);

#if defined(__GNUC__)
#pragma GCC visibility pop
#endif

#ifdef __cplusplus
}
#endif
#endif /* WARP_CTCT_HIP_H */
