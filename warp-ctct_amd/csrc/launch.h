// Internal launch interface between the C-ABI layer (api.hip) and the kernel
// translation units.  Plain structs of device pointers and sizes; each
// launcher enqueues on the given stream and returns hipGetLastError().
#pragma once

#include <hip/hip_runtime.h>

namespace wctct {

struct LatticeArgs {
    const double *units;  // (N,T,U+1,3) log2 units
    const int *ys;        // (N,U)
    const int *lx;        // (N)
    const int *ly;        // (N)
    double *alphas;       // (N,T+1,U+1,2) log2 units, or null if beta_only
    double *betas;        // (N,T+1,U+1,2) log2 units
    float *costs;         // (N)
    int N, T, U;
    bool beta_only;
};

int lattice_max_contexts();
hipError_t launch_lattice(const LatticeArgs &a, hipStream_t stream);

hipError_t launch_gather_units(const float *joint, const int *ys, const int *lx, const int *ly,
                               double *units, int N, int T, int U, int V, hipStream_t stream);
hipError_t launch_scale_units(const float *units_nat, const int *lx, const int *ly, double *units,
                              int N, int T, int U, hipStream_t stream);
hipError_t launch_simple_units(const float *f_g, const float *g_g, const float *den,
                               const int *lx, const int *ly, double *units, int N, int T, int U,
                               hipStream_t stream);
hipError_t launch_unit_grads(const double *units, const int *ys, const int *lx, const int *ly,
                             const double *alphas, const double *betas, float *unit_grads, int N,
                             int T, int U, hipStream_t stream);
hipError_t launch_dense_grad(const float *unit_grads, const int *ys, const int *lx, const int *ly,
                             const float *grad_out, float *dense, int N, int T, int U, int V,
                             hipStream_t stream);

}  // namespace wctct
