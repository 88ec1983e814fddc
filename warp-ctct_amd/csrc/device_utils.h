// Device-side helpers shared by the gfx950 kernels: log2-domain semiring
// arithmetic (double state, native fp32 transcendentals) and 64-lane
// wavefront data movement through DPP.
#pragma once

#include <hip/hip_bf16.h>
#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>

namespace wctct {

// Element types of the joint tensor and of its dense gradient: the lattice
// always computes in fp32 / fp64, only the loads and stores at the two ends
// differ.  Stores round to nearest even.
__device__ __forceinline__ float load_as_float(const float *p) { return *p; }
__device__ __forceinline__ float load_as_float(const __half *p) { return __half2float(*p); }
__device__ __forceinline__ float load_as_float(const __hip_bfloat16 *p) {
    return __bfloat162float(*p);
}
__device__ __forceinline__ void store_from_float(float *p, float v) { *p = v; }
__device__ __forceinline__ void store_from_float(__half *p, float v) { *p = __float2half(v); }
__device__ __forceinline__ void store_from_float(__hip_bfloat16 *p, float v) {
    *p = __float2bfloat16(v);
}

// A label as a column index: clamped into [0, V) so that a corrupt label cannot
// make a kernel read outside its tensors.  `status` (may be null) is the
// device's status word: a label that had to be clamped sets its label-range bit
// there (the reference's torch.gather raises instead, warp_ctct/__init__.py:131).
__device__ __forceinline__ int label_column(int y, int V, unsigned *status) {
    const int c = min(max(y, 0), V - 1);
    if (c != y && status) atomicOr(status, 1u);
    return c;
}
// A gathered log-probability that is NaN becomes log 0 (-inf) before it enters
// the lattice, whose maximum would otherwise drop it in one place and let it
// erase a state in another, and is reported in the same word (bit 2).
__device__ __forceinline__ float unit_or_log_zero(float x, unsigned *status) {
    if (x == x) return x;
    if (status) atomicOr(status, 2u);
    return -__builtin_huge_valf();
}

constexpr int kWave = 64;
constexpr double kLog2e = 1.4426950408889634074;
constexpr double kLn2 = 0.6931471805599453094;
// Finite stand-in used only to form differences against a maximum that may be
// -inf:  (-inf) - max(-inf, kFloor) = -inf  instead of NaN.
constexpr double kFloor = -1.0e300;

__device__ __forceinline__ double neg_inf() { return -__builtin_huge_val(); }

// 2^x and log2(x) straight on the transcendental unit (v_exp_f32, v_log_f32;
// no denormal fix-up: a result below 2^-126 flushes to 0, which is what a
// log-semiring sum wants).
__device__ __forceinline__ float exp2_hw(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float log2_hw(float x) { return __builtin_amdgcn_logf(x); }

// The lattice keeps its log2 values in double (gfx950 issues v_add_f64 /
// v_max_f64 at the fp32 rate), so sums of hundreds of log-probabilities lose
// nothing; only the bounded correction term log2(1 + 2^d), d <= 0, goes
// through the fp32 transcendental unit.  The absolute error of one (+) is
// ~1e-7 whatever the magnitude of the operands, where plain fp32 arithmetic
// on values near -2000 would lose ~1e-4 per operation.

// log2(2^x + 2^y); -inf (+) -inf = -inf, never NaN for non-NaN inputs.
// Same value as logaddexpf_ of the reference (csrc/gather.cu:23-34) up to the
// change of base: larger + log(1 + exp(smaller - larger)).
__device__ __forceinline__ double lse2(double x, double y) {
    const double mx = __builtin_fmax(x, y);
    const double mn = __builtin_fmin(x, y);
    const float d = (float)(mn - __builtin_fmax(mx, kFloor));
    return mx + (double)log2_hw(1.0f + exp2_hw(d));
}

// log2((1 + 2^-|d|) / 2), in [-1, 0]: the correction term of a semiring sum
// whose operands are d apart, less one.  log2(2^x + 2^y) is then
// (max(x, y) + 1) + this, where the first sum does not wait for the
// transcendental unit.  d = NaN (the difference of two -inf) gives -inf: the
// clamp of the multiply-add turns NaN into 0 (kernels run with DX10 clamping).
// Three instructions between the difference and the result.
__device__ __forceinline__ float half_sum_log2(float d) {
    const float e = exp2_hw(-__builtin_fabsf(d));
    // median of (x, 0, 1) on a multiply-add: folded into the instruction's clamp
    const float t = __builtin_amdgcn_fmed3f(__builtin_fmaf(e, 0.5f, 0.5f), 0.0f, 1.0f);
    return log2_hw(t);
}

// Lane l receives x of lane l-1; lane 0 receives `fill`.  Two DPP moves
// (wave_shr:1), no LDS traffic.
__device__ __forceinline__ double wave_shift_up(double x, double fill) {
    const int lo = __builtin_amdgcn_update_dpp(__double2loint(fill), __double2loint(x),
                                               0x138 /* wave_shr:1 */, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(__double2hiint(fill), __double2hiint(x), 0x138,
                                               0xf, 0xf, false);
    return __hiloint2double(hi, lo);
}

// Lane l receives x of lane l+1; lane 63 receives `fill` (wave_shl:1).
__device__ __forceinline__ double wave_shift_down(double x, double fill) {
    const int lo = __builtin_amdgcn_update_dpp(__double2loint(fill), __double2loint(x),
                                               0x130 /* wave_shl:1 */, 0xf, 0xf, false);
    const int hi = __builtin_amdgcn_update_dpp(__double2hiint(fill), __double2hiint(x), 0x130,
                                               0xf, 0xf, false);
    return __hiloint2double(hi, lo);
}

}  // namespace wctct
