// Torch-free parity harness for the C ABI of libwarpctct_hip.so: every buffer
// is hipMalloc'ed here, the library is called exactly as a non-Python host
// (the reference's own C++ binding, a serving loop) would call it, and the
// results are compared with the float64 C oracle on the same seeded inputs.
// Test infrastructure: built by tests/abi_harness/Makefile, run by
// tests/test_abi_harness_gpu.py.  Prints one line per case and exits non-zero
// on the first mismatch.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "warp_ctct_hip.h"

extern "C" int oracle_ctct_loss_dense_f64(const double *joint, const int *ys, const int *lx,
                                          const int *ly, int N, int T, int U, int V,
                                          const double *grad_out, double *costs, double *dense);

#define HIP_OK(x)                                                                     \
    do {                                                                              \
        hipError_t e_ = (x);                                                          \
        if (e_ != hipSuccess) {                                                       \
            std::fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_));              \
            std::exit(2);                                                             \
        }                                                                             \
    } while (0)
#define ABI_OK(x)                                                                     \
    do {                                                                              \
        int rc_ = (x);                                                                \
        if (rc_ != WARPCTCT_OK) {                                                     \
            std::fprintf(stderr, "%s: %s\n", #x, warpctct_error_string(rc_));         \
            std::exit(3);                                                             \
        }                                                                             \
    } while (0)

namespace {

struct Rng {   // splitmix64: the same inputs on every run and every host
    uint64_t s;
    uint64_t next() {
        uint64_t z = (s += 0x9e3779b97f4a7c15ull);
        z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
        z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
        return z ^ (z >> 31);
    }
    double uniform() { return (next() >> 11) * (1.0 / 9007199254740992.0); }
    int range(int lo, int hi) { return lo + (int)(next() % (uint64_t)(hi - lo + 1)); }
};

template <typename T>
T *to_device(const std::vector<T> &h) {
    T *d = nullptr;
    HIP_OK(hipMalloc(&d, h.size() * sizeof(T) + 16));
    HIP_OK(hipMemcpy(d, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

bool run_case(const char *name, uint64_t seed, int N, int T, int U, int V, int reduction) {
    Rng rng{seed};
    const int U1 = U + 1;
    const size_t elems = (size_t)N * T * U1 * V;
    // joint = log_softmax of random logits, as float (what the library reads)
    std::vector<float> joint(elems);
    for (size_t r = 0; r < elems / V; ++r) {
        double mx = -1e30, sum = 0.0;
        std::vector<double> x(V);
        for (int v = 0; v < V; ++v) {
            x[v] = 3.0 * (rng.uniform() - 0.5);
            mx = std::fmax(mx, x[v]);
        }
        for (int v = 0; v < V; ++v) sum += std::exp(x[v] - mx);
        for (int v = 0; v < V; ++v) joint[r * V + v] = (float)(x[v] - mx - std::log(sum));
    }
    std::vector<int> ys((size_t)N * U), lx(N), ly(N);
    for (auto &y : ys) y = rng.range(1, V - 1);
    for (int n = 0; n < N; ++n) {
        ly[n] = rng.range(U > 0 ? 1 : 0, U);
        if (ly[n] >= 2) ys[(size_t)n * U + 1] = ys[(size_t)n * U];   // one adjacent repeat
        lx[n] = rng.range(std::min(T, ly[n] + 2), T);
    }
    std::vector<float> grad_out(N);
    for (auto &g : grad_out) g = (float)(0.5 + rng.uniform());

    // oracle, float64, on the same float inputs
    std::vector<double> jd(joint.begin(), joint.end()), god(grad_out.begin(), grad_out.end());
    std::vector<double> ref_costs(N), ref_dense(elems);
    const double scale = reduction == 2 ? 1.0 / N : 1.0;
    if (reduction != 0) for (auto &g : god) g = scale;
    if (oracle_ctct_loss_dense_f64(jd.data(), ys.data(), lx.data(), ly.data(), N, T, U, V,
                                   god.data(), ref_costs.data(), ref_dense.data()) != 0) {
        std::fprintf(stderr, "%s: oracle rejected the case\n", name);
        return false;
    }
    double ref_reduced = 0.0;
    for (double c : ref_costs) ref_reduced += c * scale;

    // the library, through its C ABI only
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    float *d_joint = to_device(joint), *d_go = to_device(grad_out);
    int *d_ys = to_device(ys), *d_lx = to_device(lx), *d_ly = to_device(ly);
    const size_t ws_bytes = warpctct_workspace_bytes(N, T, U);
    void *d_ws = nullptr;
    float *d_costs = nullptr, *d_reduced = nullptr, *d_dense = nullptr;
    HIP_OK(hipMalloc(&d_ws, ws_bytes));
    HIP_OK(hipMalloc(&d_costs, N * sizeof(float)));
    HIP_OK(hipMalloc(&d_reduced, sizeof(float)));
    HIP_OK(hipMalloc(&d_dense, elems * sizeof(float)));
    HIP_OK(hipMemset(d_dense, 0xff, elems * sizeof(float)));   // every element must be overwritten
    ABI_OK(warpctct_loss_lattice(d_joint, WARPCTCT_F32, d_ys, d_lx, d_ly, N, T, U, V, d_ws,
                                 ws_bytes, d_costs, 1, reduction, 0, d_reduced, stream));
    if (reduction == 0) {
        ABI_OK(warpctct_dense_grad_lattice(d_ws, ws_bytes, d_ys, d_lx, d_ly, d_go, 1, 1.0f, 0,
                                           d_dense, WARPCTCT_F32, N, T, U, V, stream));
    } else {   // upstream gradient 1 of the reduced scalar: broadcast, scaled by 1/N for the mean
        ABI_OK(warpctct_dense_grad_lattice(d_ws, ws_bytes, d_ys, d_lx, d_ly, nullptr, 0,
                                           (float)scale, 0, d_dense, WARPCTCT_F32, N, T, U, V,
                                           stream));
    }
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<float> costs(N), dense(elems);
    float reduced = 0.0f;
    HIP_OK(hipMemcpy(costs.data(), d_costs, N * sizeof(float), hipMemcpyDeviceToHost));
    HIP_OK(hipMemcpy(dense.data(), d_dense, elems * sizeof(float), hipMemcpyDeviceToHost));
    if (reduction != 0)
        HIP_OK(hipMemcpy(&reduced, d_reduced, sizeof(float), hipMemcpyDeviceToHost));

    double cost_err = 0.0, grad_err = 0.0;
    for (int n = 0; n < N; ++n)
        cost_err = std::fmax(cost_err, std::fabs(costs[n] - ref_costs[n]) / std::fabs(ref_costs[n]));
    if (reduction != 0)
        cost_err = std::fmax(cost_err, std::fabs(reduced - ref_reduced) / std::fabs(ref_reduced));
    size_t wrong_zero = 0;
    for (size_t i = 0; i < elems; ++i) {
        grad_err = std::fmax(grad_err, std::fabs((double)dense[i] - ref_dense[i]));
        if (ref_dense[i] == 0.0 && dense[i] != 0.0f) ++wrong_zero;
    }
    const bool ok = cost_err <= 1e-5 && grad_err <= 1e-4 && wrong_zero == 0;   // the build's bar
    std::printf("%-28s N=%d T=%d U=%d V=%d reduction=%d  cost rel-err %.2e  grad abs-err %.2e  "
                "non-zero structural zeros %zu  %s\n",
                name, N, T, U, V, reduction, cost_err, grad_err, wrong_zero, ok ? "ok" : "FAIL");
    for (void *p : {(void *)d_joint, (void *)d_go, (void *)d_ys, (void *)d_lx, (void *)d_ly, d_ws,
                    (void *)d_costs, (void *)d_reduced, (void *)d_dense})
        HIP_OK(hipFree(p));
    HIP_OK(hipStreamDestroy(stream));
    return ok;
}

}  // namespace

int main() {
    std::printf("libwarpctct_hip %s\n", warpctct_version());
    bool ok = true;
    ok &= run_case("reference_config", 1, 2, 40, 10, 32, 0);
    ok &= run_case("ragged_mean", 2, 5, 23, 7, 16, 2);
    ok &= run_case("two_wavefronts_sum", 3, 3, 150, 100, 12, 1);
    ok &= run_case("odd_vocabulary", 4, 3, 17, 5, 37, 0);
    ok &= run_case("no_labels", 5, 2, 9, 0, 6, 0);
    return ok ? 0 : 1;
}
