// The end of a lattice's beta sweep that holds context 0: costs[n] is final,
// and the reduction over the batch (warp_ctct/__init__.py:138-147 of the
// reference) is taken by the workgroup that finishes last.  Shared by the
// lattice kernels.
#pragma once
#include <hip/hip_runtime.h>

#include "launch.h"

namespace wctct {

// Called by the whole wavefront (lane = its lane index) after lane 0 has written
// costs[n].
__device__ __forceinline__ void cost_reduce_tail(const CostReduce &red, float *costs, const int *lx,
                                                 int n, int N, int lane) {
    if (red.average_frames && lane == 0) costs[n] /= (float)lx[n];
    if (red.reduced == nullptr) return;
    // every workgroup publishes its cost (release fence), then counts itself;
    // the one that sees N-1 earlier arrivals reads all N costs (acquire fence)
    // and adds them in a fixed order, so the result does not depend on the
    // order of arrival
    int last = 0;
    if (lane == 0) {
        __threadfence();
        last = (atomicAdd(red.counter, 1u) == (unsigned)(N - 1)) ? 1 : 0;
    }
    last = __shfl(last, 0, 64);
    if (!last) return;
    __threadfence();
    float s = 0.0f;
    for (int i = lane; i < N; i += 64)
        s += __hip_atomic_load(costs + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if (lane == 0) *red.reduced = (red.mode == 2) ? s / (float)N : s;
}

}  // namespace wctct
