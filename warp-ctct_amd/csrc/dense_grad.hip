// Dense gradient of ctct_loss wrt the (N,T,U+1,V) joint tensor.
//
// The reference obtains it in two steps: CTCTLoss.backward scales the saved
// unit gradients by grad_output (warp_ctct/__init__.py:30-33) and autograd's
// gather backward zero-fills an (N,T,U+1,V) tensor and scatter-adds into it.
// Here one streaming pass writes every element exactly once: a row (n,t,u) of
// V floats is all zeros except columns 0, y[u-1], y[u], which receive
// grad_out[n] * g0 / g1 / g2 (coincident columns add, as scatter_add does).
// The pass is pure HBM write traffic (4*N*T*(U+1)*V bytes) and decides the
// throughput of the whole loss: stores are 16 bytes per lane, 1 KiB contiguous
// per wavefront instruction, non-temporal (the data is not read again by this
// library), and a 256-column chunk that holds none of the three columns takes
// a branch-free all-zero path.
#include "device_utils.h"
#include "launch.h"

namespace wctct {

namespace {

typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int kRowsPerBlock = 16;
constexpr int kWavesPerBlock = 4;

template <bool VEC4>
__global__ __launch_bounds__(kWavesPerBlock * 64) void dense_grad_kernel(
    const float *__restrict__ unit_grads, const int *__restrict__ ys,
    const int *__restrict__ lx, const int *__restrict__ ly, const float *__restrict__ grad_out,
    float *__restrict__ dense, int T, int U, int V) {
    const int n = blockIdx.z;
    const int t = blockIdx.y;
    const int U1 = U + 1;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    const int Tn = min(max(lx[n], 0), T);
    const int Un = min(max(ly[n], 0), U);
    const float w = grad_out ? grad_out[n] : 1.0f;
    const int *y = ys + (size_t)n * U;

    for (int r = wave; r < kRowsPerBlock; r += kWavesPerBlock) {
        const int u = blockIdx.x * kRowsPerBlock + r;
        if (u > U) break;
        const size_t row = ((size_t)n * T + t) * U1 + u;
        float *out = dense + row * (size_t)V;
        const bool live = (t < Tn) && (u <= Un);
        float g0 = 0.0f, g1 = 0.0f, g2 = 0.0f;
        int c1 = 0, c2 = 0;
        if (live) {
            const float *g = unit_grads + row * 3;
            g0 = g[0] * w;
            if (u >= 1) {
                g1 = g[1] * w;
                c1 = min(max(y[u - 1], 0), V - 1);
            }
            if (u < Un) {
                g2 = g[2] * w;
                c2 = min(max(y[u], 0), V - 1);
            }
        }
        if (VEC4) {
            v4f *out4 = reinterpret_cast<v4f *>(out);
            const int nvec = V >> 2;
            for (int base = 0; base < nvec; base += 64) {
                const int fi = base + lane;
                // does this 256-column chunk hold any of the three columns?
                const int chunk = base >> 6;
                const bool hit = live && (chunk == 0 || (c1 >> 8) == chunk || (c2 >> 8) == chunk);
                v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
                if (hit) {
                    const int col = fi << 2;
                    const int d1 = c1 - col;
                    const int d2 = c2 - col;
                    v.x = (col == 0 ? g0 : 0.0f) + (d1 == 0 ? g1 : 0.0f) + (d2 == 0 ? g2 : 0.0f);
                    v.y = (d1 == 1 ? g1 : 0.0f) + (d2 == 1 ? g2 : 0.0f);
                    v.z = (d1 == 2 ? g1 : 0.0f) + (d2 == 2 ? g2 : 0.0f);
                    v.w = (d1 == 3 ? g1 : 0.0f) + (d2 == 3 ? g2 : 0.0f);
                }
                if (fi < nvec) __builtin_nontemporal_store(v, out4 + fi);
            }
        } else {
            for (int col = lane; col < V; col += 64) {
                float v = 0.0f;
                if (live)
                    v = (col == 0 ? g0 : 0.0f) + (col == c1 ? g1 : 0.0f) + (col == c2 ? g2 : 0.0f);
                out[col] = v;
            }
        }
    }
}

}  // namespace

hipError_t launch_dense_grad(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                             const float *grad_out, float *dense, int N, int T, int U, int V,
                             hipStream_t stream) {
    dim3 grid((unsigned)((U + 1 + kRowsPerBlock - 1) / kRowsPerBlock), (unsigned)T, (unsigned)N);
    dim3 block(kWavesPerBlock * 64);
    const bool vec4 = (V % 4 == 0) && ((reinterpret_cast<uintptr_t>(dense) & 15u) == 0);
    if (vec4)
        hipLaunchKernelGGL(dense_grad_kernel<true>, grid, block, 0, stream, unit_grads, ys, lx, ly,
                           grad_out, dense, T, U, V);
    else
        hipLaunchKernelGGL(dense_grad_kernel<false>, grid, block, 0, stream, unit_grads, ys, lx,
                           ly, grad_out, dense, T, U, V);
    return hipGetLastError();
}

}  // namespace wctct
