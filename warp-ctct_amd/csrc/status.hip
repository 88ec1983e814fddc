// Sticky status word of a device: bits that kernels set when they meet input
// they had to repair (a label outside [0, V) clamped into it, a NaN among the
// gathered log-probabilities) or when a lattice could not be swept to its end
// (a hand-over between the workgroups of a chain that did not arrive).  The
// word lives in the library's code object, one copy per GPU; kernels reach it
// through the pointer device_status_word() returns for the current device, the
// host reads it with warpctct_status.  No counterpart in the reference, whose
// torch.gather raises on a bad index (warp_ctct/__init__.py:131) after a
// device-to-host synchronisation; here nothing synchronises unless asked.
#include <hip/hip_runtime.h>

#include <atomic>

#include "launch.h"
#include "warp_ctct_hip.h"

// In host code this name is only a handle for hipGetSymbolAddress.
static __device__ __align__(16) unsigned status_word[4];

namespace wctct {

namespace {
constexpr int kMaxDevices = 64;
std::atomic<unsigned *> g_status_ptr[kMaxDevices];
}  // namespace

unsigned *device_status_word() {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        (void)hipGetLastError();
        return nullptr;
    }
    unsigned *p = g_status_ptr[device].load(std::memory_order_acquire);
    if (p) return p;
    void *found = nullptr;
    if (hipGetSymbolAddress(&found, HIP_SYMBOL(status_word)) != hipSuccess || !found) {
        (void)hipGetLastError();
        return nullptr;
    }
    // (two threads may look it up at once: both find the same address)
    g_status_ptr[device].store(static_cast<unsigned *>(found), std::memory_order_release);
    return static_cast<unsigned *>(found);
}

}  // namespace wctct

extern "C" {

int warpctct_status(unsigned *bits, int clear) {
    if (!bits) return WARPCTCT_EINVAL;
    unsigned *word = wctct::device_status_word();
    if (!word) return WARPCTCT_ENODEVICE;
    // waits for the work queued on the device so far: the bits of every launch
    // made before this call are in
    if (hipDeviceSynchronize() != hipSuccess) return WARPCTCT_ELAUNCH;
    if (hipMemcpy(bits, word, sizeof(unsigned), hipMemcpyDeviceToHost) != hipSuccess)
        return WARPCTCT_ELAUNCH;
    if (clear && *bits != 0u && hipMemset(word, 0, sizeof(unsigned)) != hipSuccess)
        return WARPCTCT_ELAUNCH;
    return WARPCTCT_OK;
}

}  // extern "C"
