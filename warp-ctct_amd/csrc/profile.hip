// Per-kernel HIP-event timing behind warpctct_profile* (see profile.h).
#include "profile.h"

#include <atomic>
#include <cstring>
#include <mutex>
#include <vector>

#include "warp_ctct_hip.h"

namespace wctct {

namespace {

constexpr int kMaxRecords = 8192;

struct Record {
    const char *kernel;
    hipEvent_t begin, end;
    bool complete;
};

std::atomic<bool> g_enabled{false};
std::mutex g_mutex;
std::vector<Record> g_records;
unsigned g_generation = 0;   // bumped whenever the records are dropped
char g_filter[64] = "";   // bracket only kernels whose name contains this

void drop_records() {
    ++g_generation;
    for (Record &r : g_records) {
        (void)hipEventDestroy(r.begin);
        (void)hipEventDestroy(r.end);
    }
    g_records.clear();
}

}  // namespace

bool profile_enabled() { return g_enabled.load(std::memory_order_relaxed); }

void profile_begin(const char *kernel, hipStream_t stream, int *slot, unsigned *generation) {
    std::lock_guard<std::mutex> lock(g_mutex);
    if ((int)g_records.size() >= kMaxRecords) return;
    if (g_filter[0] && !std::strstr(kernel, g_filter)) return;
    // A stream under graph capture takes no timing events (recording one would
    // become a node of the graph, or fail and leave its error for the caller's
    // own check of the launch): launches into a capture are not bracketed.
    hipStreamCaptureStatus capture = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &capture) != hipSuccess) {
        (void)hipGetLastError();
        return;
    }
    if (capture != hipStreamCaptureStatusNone) return;
    Record r = {kernel, nullptr, nullptr, false};
    if (hipEventCreate(&r.begin) != hipSuccess) return;
    if (hipEventCreate(&r.end) != hipSuccess) {
        (void)hipEventDestroy(r.begin);
        return;
    }
    if (hipEventRecord(r.begin, stream) != hipSuccess) {
        (void)hipEventDestroy(r.begin);
        (void)hipEventDestroy(r.end);
        return;
    }
    g_records.push_back(r);
    *slot = (int)g_records.size() - 1;
    *generation = g_generation;
}

void profile_end(hipStream_t stream, int slot, unsigned generation) {
    std::lock_guard<std::mutex> lock(g_mutex);
    // (the records this launch belongs to were dropped by another thread in between)
    if (generation != g_generation) return;
    if (slot < 0 || slot >= (int)g_records.size()) return;
    g_records[slot].complete = hipEventRecord(g_records[slot].end, stream) == hipSuccess;
}

}  // namespace wctct

extern "C" {

int warpctct_profile(int enable) {
    using namespace wctct;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (enable) drop_records();
    g_enabled.store(enable != 0, std::memory_order_relaxed);
    return WARPCTCT_OK;
}

int warpctct_profile_filter(const char *text) {
    using namespace wctct;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (text && std::strlen(text) >= sizeof(g_filter)) return WARPCTCT_EINVAL;
    std::strcpy(g_filter, text ? text : "");
    return WARPCTCT_OK;
}

int warpctct_profile_count(void) {
    using namespace wctct;
    std::lock_guard<std::mutex> lock(g_mutex);
    return (int)g_records.size();
}

int warpctct_profile_read(int index, const char **kernel, float *microseconds) {
    using namespace wctct;
    std::lock_guard<std::mutex> lock(g_mutex);
    if (index < 0 || index >= (int)g_records.size() || !kernel || !microseconds)
        return WARPCTCT_EINVAL;
    const Record &r = g_records[index];
    if (!r.complete) return WARPCTCT_ELAUNCH;
    if (hipEventSynchronize(r.end) != hipSuccess) return WARPCTCT_ELAUNCH;
    float ms = 0.0f;
    if (hipEventElapsedTime(&ms, r.begin, r.end) != hipSuccess) return WARPCTCT_ELAUNCH;
    *kernel = r.kernel;
    *microseconds = ms * 1000.0f;
    return WARPCTCT_OK;
}

}  // extern "C"
