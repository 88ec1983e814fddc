// Optional per-kernel timing for measurement runs: while switched on, every
// kernel launch of the library is bracketed by two HIP events recorded on the
// stream the kernel is launched on, and the pairs are kept (up to kMaxRecords)
// until they are read.  Switched off (the default) a launch pays one relaxed
// atomic load.  Not for use under graph capture.
#pragma once

#include <hip/hip_runtime.h>

namespace wctct {

bool profile_enabled();
// slot: index of the record that was opened (-1: none); generation: which run of
// records it belongs to (warpctct_profile(1) starts a new one and drops the
// old records: an end that arrives for an earlier generation is ignored)
void profile_begin(const char *kernel, hipStream_t stream, int *slot, unsigned *generation);
void profile_end(hipStream_t stream, int slot, unsigned generation);

struct KernelTimer {
    hipStream_t stream;
    int slot;
    unsigned generation;
    KernelTimer(const char *kernel, hipStream_t s) : stream(s), slot(-1), generation(0) {
        if (profile_enabled()) profile_begin(kernel, s, &slot, &generation);
    }
    ~KernelTimer() {
        if (slot >= 0) profile_end(stream, slot, generation);
    }
    KernelTimer(const KernelTimer &) = delete;
    KernelTimer &operator=(const KernelTimer &) = delete;
};

}  // namespace wctct

// hipLaunchKernelGGL with the timing bracket; the record is named after the
// kernel expression as written at the launch site.
#define TIMED_LAUNCH(kernel, grid, block, shmem, stream, ...)                  \
    do {                                                                       \
        ::wctct::KernelTimer kernel_timer_(#kernel, stream);                   \
        hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);   \
    } while (0)
