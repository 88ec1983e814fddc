// Optional per-kernel timing for measurement runs: while switched on, every
// kernel launch of the library is bracketed by two HIP events recorded on the
// stream the kernel is launched on, and the pairs are kept (up to kMaxRecords)
// until they are read.  Switched off (the default) a launch pays one relaxed
// atomic load.  Not for use under graph capture.
#pragma once

#include <hip/hip_runtime.h>

namespace wctct {

bool profile_enabled();
void profile_begin(const char *kernel, hipStream_t stream, int *slot);
void profile_end(hipStream_t stream, int slot);

struct KernelTimer {
    hipStream_t stream;
    int slot;
    KernelTimer(const char *kernel, hipStream_t s) : stream(s), slot(-1) {
        if (profile_enabled()) profile_begin(kernel, s, &slot);
    }
    ~KernelTimer() {
        if (slot >= 0) profile_end(stream, slot);
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
