// d(cost)/d(unit) of one live cell from the stored lattices; shared by the
// kernel that writes the (N,T,U+1,3) unit-gradient tensor and by the kernel
// that writes the non-zero entries of the dense gradient directly.
#pragma once

#include "device_utils.h"
#include "launch.h"

namespace wctct {

// Every frame consumes exactly one unit and a label needs at least one frame,
// so a complete alignment of Tn frames and Un labels can only use cell (t,u)
// if u labels fit into the t frames before it (t >= u) and the Un - u labels
// still missing fit into the Tn - t frames from t on.  Outside this band alpha
// is -inf, or every successor's beta is, whatever the units are, and the
// gradient is exactly zero (the reference skips the same cells through its
// shifted storage, csrc/gather.cu:333-336, :354-357).
__device__ __forceinline__ bool outside_band(int t, int u, int Tn, int Un) {
    return t < u || Tn - t < Un - u;
}

// The weight of sample n (see Weight in launch.h); lxn = lx[n].
__device__ __forceinline__ float sample_weight(const Weight &w, int n, int lxn) {
    float v = w.grad_out ? w.grad_out[(size_t)n * w.stride] : 1.0f;
    v *= w.scale;
    if (w.average_frames) v /= (float)lxn;
    return v;
}

struct UnitGrad {
    float g0, g1, g2;   // blank, current label (u >= 1), next label (u < Un)
};

// g0 = -[2^(a_e+LP0+b_e-ll) + 2^(a_o+LP0+b_e-ll)]
// g1 = - 2^(a_o+LP1+b_o-ll)
// g2 = -[2^(a_e+LP2+b_o'-ll) + [y[u-1]!=y[u]] 2^(a_o+LP2+b_o'-ll)]       (u < Un)
// with a_* = alpha(t,.) of context u, b_* = beta(t+1,.) of context u,
// b_o' = beta(t+1, 2u+1) (context u+1), ll = beta(0,0), all in log2 units
// (csrc/gather.cu:311-374 of the reference in natural coordinates).
// alpha(t, 2u-1) of context 0 is stored as -inf, which zeroes the u >= 1 terms.
// The exponent is summed in double and rounded once.
// units_n / alpha_n / beta_n point at sample n; P contexts per frame.
__device__ __forceinline__ UnitGrad unit_grad_cell(const double *units_n, const double *alpha_n,
                                                   const double *beta_n, const int *y, int t,
                                                   int u, int Un, int P) {
    const double ll = beta_n[1];   // beta(0, state 0): pair {o,e} of context 0 at t = 0
    const double2 a = *reinterpret_cast<const double2 *>(alpha_n + ((size_t)t * P + u) * 2);
    const double2 b = *reinterpret_cast<const double2 *>(beta_n + ((size_t)(t + 1) * P + u) * 2);
    const double *lp = units_n + ((size_t)t * P + u) * 3;
    const double lp0 = lp[0] - ll, lp1 = lp[1] - ll;
    UnitGrad r;
    r.g0 = -(exp2_hw((float)(a.y + lp0 + b.y)) + exp2_hw((float)(a.x + lp0 + b.y)));
    r.g1 = (u >= 1) ? -exp2_hw((float)(a.x + lp1 + b.x)) : 0.0f;
    r.g2 = 0.0f;
    if (u < Un) {
        const double lp2 = lp[2] - ll;
        const double bo_next = beta_n[((size_t)(t + 1) * P + u + 1) * 2];
        r.g2 = -exp2_hw((float)(a.y + lp2 + bo_next));
        if (u >= 1 && y[u - 1] != y[u]) r.g2 -= exp2_hw((float)(a.x + lp2 + bo_next));
    }
    return r;
}

// The same from lattices in the linear domain (lattice_lin.hip): alpha / beta
// rows are masses relative to 2^scale, one scale per (direction, wavefront of
// kLinReal contexts, chunk of frames), of which a row holds the high words
// (20 bits of mantissa); units are linear; Pl columns per row,
// context u in column lin_column(u).  sa / sb / sb_next: the scales of row t of
// alpha, and of row t+1 of beta for context u and for context u+1; inv_ll and
// s_ll: 1 / mantissa and exponent of the lattice's total mass beta(0, state 0).
// A state from the high word that its row holds: the low word was cut off, so
// the middle of what it can have been is taken (the error of a posterior is
// then 2.4e-7 at most and has no sign of its own; with 0 for the low word every
// posterior came out low, and a gradient that sums 1500 of them 1e-6 low).  A
// state of exactly 0 becomes 1e-314, which no product notices.
__device__ __forceinline__ double lin_state(unsigned high) {
    return __hiloint2double((int)high, (int)0x80000000u);
}

__device__ __forceinline__ UnitGrad unit_grad_cell_lin(const double *units_n, const unsigned *alpha_n,
                                                       const unsigned *beta_n, const int *y, int t,
                                                       int u, int Un, int Pl, int sa, int sb,
                                                       int sb_next, double inv_ll, int s_ll,
                                                       bool &out_of_range) {
    const int col = lin_column(u);
    const uint2 aw = *reinterpret_cast<const uint2 *>(alpha_n + ((size_t)t * Pl + col) * 2);
    const uint2 bw = *reinterpret_cast<const uint2 *>(beta_n + ((size_t)(t + 1) * Pl + col) * 2);
    const double2 a = make_double2(lin_state(aw.x), lin_state(aw.y));
    const double2 b = make_double2(lin_state(bw.x), lin_state(bw.y));
    const double *lp = units_n + ((size_t)t * Pl + col) * kLinUnit;
    const double lp0 = lp[0], lp1 = lp[1];
    // a unit above 2^80 may overflow a chunk of frames (small ones can only lose
    // mass, which the sums of the posteriors show): such a batch is not for this form
    out_of_range = lp0 > 0x1p80 || (u >= 1 && lp1 > 0x1p80);
    // posterior = (alpha * unit) * beta * 2^(sa + sb - s_ll) / mantissa of the total;
    // half of the power of two goes to each factor first, so that a product of two
    // small numbers does not leave the range on its way to a posterior that is in it
    const int k = sa + sb - s_ll, ka = k / 2;
    const double2 as = make_double2(__builtin_amdgcn_ldexp(a.x, ka), __builtin_amdgcn_ldexp(a.y, ka));
    const double bo = __builtin_amdgcn_ldexp(b.x, k - ka) * inv_ll, be = __builtin_amdgcn_ldexp(b.y, k - ka) * inv_ll;
    UnitGrad r;
    r.g0 = -(float)(((as.y + as.x) * lp0) * be);
    r.g1 = (u >= 1) ? -(float)((as.x * lp1) * bo) : 0.0f;
    r.g2 = 0.0f;
    if (u < Un) {
        const double lp2 = lp[2];
        out_of_range = out_of_range || lp2 > 0x1p80;
        const int k2 = sa + sb_next - s_ll;
        const double bo_next = __builtin_amdgcn_ldexp(lin_state(beta_n[((size_t)(t + 1) * Pl + lin_column(u + 1)) * 2]), k2 - ka) * inv_ll;
        const double from = (u >= 1 && y[u - 1] != y[u]) ? as.y + as.x : as.y;
        r.g2 = -(float)((from * lp2) * bo_next);
    }
    return r;
}

}  // namespace wctct
