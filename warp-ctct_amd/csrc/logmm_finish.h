// The last pass of the log-matmul's slab forward, as a device function: the
// kernel that reads the product first can do it on the way instead of a launch
// of its own (see LogmmDeferred in launch.h).
#pragma once
#include <hip/hip_runtime.h>

#include "device_utils.h"
#include "launch.h"

namespace wctct {

// res[b,i,j] from the slabs' partial sums, each taken against the slab's own
// maximum of row i; row_max receives the row's maximum.  lrow / rcol are row i
// of lhs and column j of rhs (element strides lsk, rsk, K entries) for the
// exact evaluation of a sum that fell below 2^-60 (or overflowed).  At most 8
// slabs; all loads are requested before the first is used.
__device__ __forceinline__ float logmm_finish_cell(const LogmmDeferred &d, int b, int i, int j,
                                                   const float *lrow, long lsk, const float *rcol,
                                                   long rsk, int K, float &row_max) {
    const float kLog2eF = 1.4426950408889634f, kLn2F = 0.6931471805599453f;
    const float kTiny = 8.6736174e-19f;   // 2^-60
    const float ninf = -__builtin_huge_valf();
    const size_t per = (size_t)d.pM * d.pN;
    const float *p = d.partial + (size_t)b * per + (size_t)i * d.pN + j;
    const float *sm = d.slab_max + (size_t)b * d.pM + i;
    float pv[8], mv[8];
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) {
        const int spc = min(sp, d.splits - 1);
        pv[sp] = p[(size_t)spc * d.B * per];
        mv[sp] = sp < d.splits ? sm[(size_t)spc * d.B * d.pM] : ninf;
    }
    const float mr = d.rmax[(size_t)b * d.Nn + j];
    float m = ninf;
#pragma unroll
    for (int sp = 0; sp < 8; ++sp) m = fmaxf(m, mv[sp]);
    row_max = m;
    float s = 0.0f;
#pragma unroll
    for (int sp = 0; sp < 8; ++sp)
        if (mv[sp] != ninf) s += pv[sp] * exp2_hw((mv[sp] - m) * kLog2eF);
    if (s >= kTiny && s < __builtin_huge_valf()) return m + mr + log2_hw(s) * kLn2F;
    float mx = ninf;
    for (int k = 0; k < K; ++k) mx = fmaxf(mx, lrow[(size_t)k * lsk] + rcol[(size_t)k * rsk]);
    if (mx == ninf) return mx;
    float e = 0.0f;
    for (int k = 0; k < K; ++k)
        e += exp2_hw((lrow[(size_t)k * lsk] + rcol[(size_t)k * rsk] - mx) * kLog2eF);
    return mx + log2_hw(e) * kLn2F;
}

}  // namespace wctct
