// ctct_loss on un-normalised joiner outputs ("logits"): log_softmax over the
// vocabulary is taken inside the gather, and its backward inside the kernel
// that writes the dense gradient, so the (N,T,U+1,V) log-probability tensor
// that a caller of the reference has to materialise before
// warp_ctct.ctct_loss (and whose gradient autograd has to push back through
// log_softmax) never exists:
//   forward   lse[n,t,u] = logsumexp_v logits[n,t,u,v]          (live rows only)
//             units      = logits[n,t,u,{0, y[u-1], y[u]}] - lse
//   backward  d/dlogits[v] = w_n * (G[v] - softmax[v] * (g0 + g1 + g2))
// where G is the gather backward of the unit gradients g (non-zero in at most
// three columns, csrc/gather.cu:311-374 of the reference) and w_n the upstream
// weight of sample n.  Rows of padding and rows outside the band of complete
// alignments are not read at all; their gradient is zero.
// One wavefront per row; a row is read once in each direction.
#include "device_utils.h"
#include "launch.h"
#include "unit_grad.h"

namespace wctct {

namespace {

constexpr int kRowsPerBlock = 4;       // wavefronts per workgroup, forward
constexpr int kGradWaves = 1;          // ... and backward: 4 KiB per workgroup, like the plain zero-fill
constexpr float kLog2eF = 1.4426950408889634f;
constexpr float kLn2F = 0.6931471805599453f;

// one 16-byte vector of floats (these loads serve the backward, which is the
// last to read a row: non-temporal, 503 -> 475 us for the typical batch; the
// forward's loads stay ordinary, the backward finds part of its rows in the
// memory-side cache because of them)
__device__ __forceinline__ void load4(const float *p, float (&x)[4]) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    const v4f v = __builtin_nontemporal_load(reinterpret_cast<const v4f *>(p));
    x[0] = v.x;
    x[1] = v.y;
    x[2] = v.z;
    x[3] = v.w;
}
// (the stores of the gradient are non-temporal: it is not read again by this
// path, and written the ordinary way 2 GB of it linger in the caches and are
// written back while the next forward runs: 231 us instead of 188 us there)
__device__ __forceinline__ void store4(float *p, const float (&x)[4]) {
    typedef float v4f __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(v4f{x[0], x[1], x[2], x[3]}, reinterpret_cast<v4f *>(p));
}

// 16-byte vectors of 2-byte elements
__device__ __forceinline__ void load8(const __half *p, float (&x)[8]) {
    typedef _Float16 v8h __attribute__((ext_vector_type(8)));
    const v8h v = __builtin_nontemporal_load(reinterpret_cast<const v8h *>(p));
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = (float)v[i];
}
__device__ __forceinline__ void load8(const __hip_bfloat16 *p, float (&x)[8]) {
    typedef unsigned short v8u __attribute__((ext_vector_type(8)));
    const v8u v = __builtin_nontemporal_load(reinterpret_cast<const v8u *>(p));
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = __uint_as_float((unsigned)v[i] << 16);
}
// two floats rounded to nearest even into one 32-bit word of 2-byte elements
__device__ __forceinline__ unsigned pack2(const __half *, float a, float b) {
    const __half2 h = __floats2half2_rn(a, b);
    return *reinterpret_cast<const unsigned *>(&h);
}
__device__ __forceinline__ unsigned pack2(const __hip_bfloat16 *, float a, float b) {
    const __hip_bfloat162 h = __float22bfloat162_rn(make_float2(a, b));
    return *reinterpret_cast<const unsigned *>(&h);
}
template <typename IO>
__device__ __forceinline__ void store8(IO *p, const float (&x)[8]) {
    uint4 v;
    v.x = pack2(p, x[0], x[1]);
    v.y = pack2(p, x[2], x[3]);
    v.z = pack2(p, x[4], x[5]);
    v.w = pack2(p, x[6], x[7]);
    typedef unsigned int u4 __attribute__((ext_vector_type(4)));
    __builtin_nontemporal_store(u4{v.x, v.y, v.z, v.w}, reinterpret_cast<u4 *>(p));
}
// EV elements = one 16-byte vector of the element type
__device__ __forceinline__ void load_vec(const float *p, float (&x)[4]) { load4(p, x); }
__device__ __forceinline__ void load_vec(const __half *p, float (&x)[8]) { load8(p, x); }
__device__ __forceinline__ void load_vec(const __hip_bfloat16 *p, float (&x)[8]) { load8(p, x); }
__device__ __forceinline__ void store_vec(float *p, const float (&x)[4]) { store4(p, x); }
__device__ __forceinline__ void store_vec(__half *p, const float (&x)[8]) { store8(p, x); }
__device__ __forceinline__ void store_vec(__hip_bfloat16 *p, const float (&x)[8]) { store8(p, x); }

// Maximum / sum over a group of LANES consecutive lanes (64 or 32).
template <int LANES>
__device__ __forceinline__ float group_max(float v) {
#pragma unroll
    for (int off = LANES / 2; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
#pragma unroll
    for (int off = LANES / 2; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Rows are addressable by 16-byte vectors when every row starts on a 16-byte
// boundary and holds a whole number of them.
template <typename IO>
__device__ __forceinline__ bool rows_vectorised(const IO *base, int V) {
    return (V % (16 / (int)sizeof(IO))) == 0 && (reinterpret_cast<uintptr_t>(base) & 15u) == 0;
}

// A 16-byte vector as loaded, and its EV elements as floats: a vector that is
// still in flight costs 4 registers in this form, whatever the element type.
typedef unsigned int raw16 __attribute__((ext_vector_type(4)));
template <typename IO>
__device__ __forceinline__ raw16 load_raw(const IO *p) {
    return *reinterpret_cast<const raw16 *>(p);
}
__device__ __forceinline__ void unpack(const float *, const raw16 &v, float (&x)[4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) x[i] = __uint_as_float(v[i]);
}
// (each half taken out of its word with integer operations: a cast of the word
// to a vector of two halves read word 0 for every i once compiled)
__device__ __forceinline__ void unpack(const __half *, const raw16 &v, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const unsigned word = v[i];
        x[2 * i] = (float)__builtin_bit_cast(_Float16, (unsigned short)(word & 0xffffu));
        x[2 * i + 1] = (float)__builtin_bit_cast(_Float16, (unsigned short)(word >> 16));
    }
}
__device__ __forceinline__ void unpack(const __hip_bfloat16 *, const raw16 &v, float (&x)[8]) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        x[2 * i] = __uint_as_float(v[i] << 16);
        x[2 * i + 1] = __uint_as_float(v[i] & 0xffff0000u);
    }
}

// The element at byte offset `at` (0 or 2 for the 2-byte types) of a 32-bit word.
__device__ __forceinline__ float word_element(const float *, unsigned word, unsigned) {
    return __uint_as_float(word);
}
__device__ __forceinline__ float word_element(const __half *, unsigned word, unsigned at) {
    const unsigned short bits = (unsigned short)(word >> (at * 8));
    return (float)__builtin_bit_cast(_Float16, bits);
}
__device__ __forceinline__ float word_element(const __hip_bfloat16 *, unsigned word, unsigned at) {
    return __uint_as_float((word >> (at * 8)) << 16);
}

// One workgroup of 4 wavefronts per frame (n, t) = (blockIdx.y, blockIdx.x).
// Frames of padding cost one workgroup that retires at once.  The cells of a
// live frame outside the band of complete alignments get neutral units, as in
// gather_units_kernel, written by the whole workgroup in one sweep.  The rows
// inside the band, u in [max(0, Un - (Tn - t)), min(Un, t)], are dealt to the
// wavefronts round-robin; a wavefront walks over its rows in rounds of 1024
// elements (NV 16-byte vectors per lane) and requests the next round before it
// works on the present one, so that it always has a round in flight: logsumexp
// of the row in one pass (running maximum and rescaled sum per lane, combined
// over the wavefront at the end of the row), then the three units.
template <typename IO, bool STAGED>
__global__ __launch_bounds__(64 * kRowsPerBlock)
    __attribute__((amdgpu_waves_per_eu(sizeof(IO) == 4 ? 6 : 8, 8))) void
    logits_units_kernel(const IO *__restrict__ logits, const int *__restrict__ ys,
                    const int *__restrict__ lx, const int *__restrict__ ly,
                    double *__restrict__ units, float *__restrict__ lse, int T, int U, int V, int P,
                    unsigned *__restrict__ counter, unsigned *__restrict__ status) {
    constexpr int EV = 16 / (int)sizeof(IO);    // elements per 16-byte vector
    constexpr int NV = 1024 / (64 * EV);        // vectors per lane and round of 1024 elements
    if (counter && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0) *counter = 0u;
    const int n = blockIdx.y, t = blockIdx.x;
    const int Tn = min(max(lx[n], 0), T), Un = min(max(ly[n], 0), U);
    if (t >= Tn) return;
    // the wavefront's index as a scalar: rows, labels and the three logits that
    // become units are then addressed (and the latter two loaded) by the scalar
    // unit, whose loads do not queue behind the row's vector loads
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ulo = max(0, Un - (Tn - t)), uhi = min(Un, t);
    double *frame = units + ((size_t)n * T + t) * P * 3;
    // STAGED: the frame's units (P x 3 doubles, neutral outside the band) and
    // logsumexps (P floats) are put together in LDS and written out in one
    // sweep at the end.  A global store inside the loop over the rows would
    // make every re-use of its data registers wait for the store, and with it
    // for the loads of the next round, which must stay in flight.
    extern __shared__ double staged[];
    double *frame_out = STAGED ? staged : frame;
    float *lse_out = STAGED ? reinterpret_cast<float *>(staged + (size_t)P * 3)
                            : lse + ((size_t)n * T + t) * (U + 1);
    for (int i = threadIdx.x; i < P * 3; i += 64 * kRowsPerBlock) {
        const int u = i / 3;
        if (STAGED || u < ulo || u > uhi) frame_out[i] = (i - u * 3 == 2) ? neg_inf() : 0.0;
    }
    if (STAGED) __syncthreads();
    const int *y = ys + (size_t)n * U;
    const size_t r0 = ((size_t)n * T + t) * (U + 1);
    const bool vec = rows_vectorised(logits, V);

    // the end of a row: every lane holds m (maximum of its raw values) and s
    // (sum of e^(x - m)); xb, x1, x2 are the logits that become units
    auto finish_row = [&](int u, float m, float s, float xb, float x1, float x2) {
        const float M = group_max<64>(m);
        const float Mf = fmaxf(M, -2.0e38f);
        const float S = group_sum<64>(s * exp2_hw((m - Mf) * kLog2eF));
        if (lane != 0) return;
        const float l = M + log2_hw(S) * kLn2F;   // natural-log logsumexp of the row
        lse_out[u] = l;
        // what the status word reports: a label that had to be clamped into [0, V)
        // on its way to a column index, a NaN among the values that become units
        if (status) {
            const bool bad = (u >= 1 && (unsigned)y[u - 1] >= (unsigned)V) ||
                             (u < Un && (unsigned)y[u] >= (unsigned)V);
            if (bad) atomicOr(status, 1u);
        }
        double *o = frame_out + (size_t)u * 3;
        const double b = (double)xb - (double)l;
        double cur = b, nxt = neg_inf();
        if (u >= 1) cur = (double)x1 - (double)l;
        if (u < Un) nxt = ((double)x2 - (double)l) * kLog2e;
        // a NaN unit (a NaN anywhere in the row makes its logsumexp NaN) enters the
        // lattice as log 0 and is reported
        if (b != b || cur != cur || nxt != nxt) {
            if (status) atomicOr(status, kStatusNanInput);
            o[0] = (b != b) ? neg_inf() : b * kLog2e;
            o[1] = (cur != cur) ? neg_inf() : cur * kLog2e;
            o[2] = (nxt != nxt) ? neg_inf() : nxt;
            return;
        }
        o[0] = b * kLog2e;
        o[1] = cur * kLog2e;
        o[2] = nxt;
    };
    if (!vec) {   // rows that cannot be read as 16-byte vectors: element by element
        for (int u = ulo + wave; u <= uhi; u += kRowsPerBlock) {
            const IO *row = logits + (r0 + u) * (size_t)V;
            const int c1 = (u >= 1) ? min(max(y[u - 1], 0), V - 1) : 0;
            const int c2 = (u < Un) ? min(max(y[u], 0), V - 1) : 0;
            const float xb = load_as_float(row), x1 = load_as_float(row + c1),
                        x2 = load_as_float(row + c2);
            float m = -__builtin_huge_valf(), s = 0.0f;
            for (int k = lane; k < V; k += 64) {
                const float x = load_as_float(row + k);
                const float mn = fmaxf(m, x);
                const float mf = fmaxf(mn, -2.0e38f);
                s = s * exp2_hw((m - mf) * kLog2eF) + exp2_hw((x - mf) * kLog2eF);
                m = mn;
            }
            finish_row(u, m, s, xb, x1, x2);
        }
    }
    // One step = one round of one row.  Two register sets hold the step being
    // worked on and the one in flight.
    struct Step {
        int u, k0;
    };
    auto next_step = [&](Step at) {
        Step nx = {at.u, at.k0 + 1024};
        if (nx.k0 >= V) nx = Step{at.u + kRowsPerBlock, 0};
        return nx;
    };
    // One element at a wavefront-uniform index: the aligned 32-bit word that
    // holds it (a scalar load; the tensor starts on a 16-byte boundary here),
    // then the element out of the word.
    const unsigned *words = reinterpret_cast<const unsigned *>(logits);
    auto uniform_element = [&](size_t index) {
        const size_t byte = index * sizeof(IO);
        return word_element(logits, words[byte >> 2], (unsigned)(byte & 3u));
    };
    // A step past the last row asks for the last row again (and is dropped):
    // every step issues the same vector loads, so that the wait for a step's
    // vectors can leave exactly the next step's in flight.  The three logits
    // that become units come through the scalar unit (every lane would ask for
    // the same address), which keeps them out of that count.
    auto request = [&](Step at, raw16 (&raw)[NV], float (&side)[3]) {
        const int u = min(at.u, uhi);
        const size_t first = (r0 + u) * (size_t)V;
        const IO *row = logits + first;
#pragma unroll
        for (int j = 0; j < NV; ++j)
            raw[j] = load_raw(row + min(at.k0 + (j * 64 + lane) * EV, V - EV));
        if (at.k0 == 0) {
            const int c1 = (u >= 1) ? min(max(y[u - 1], 0), V - 1) : 0;
            const int c2 = (u < Un) ? min(max(y[u], 0), V - 1) : 0;
            side[0] = uniform_element(first);
            side[1] = uniform_element(first + c1);
            side[2] = uniform_element(first + c2);
        }
    };
    float m = -__builtin_huge_valf(), s = 0.0f;
    float xb = 0.0f, x1 = 0.0f, x2 = 0.0f;
    auto work = [&](Step at, const raw16 (&raw)[NV], const float (&side)[3]) {
        if (at.k0 == 0) xb = side[0], x1 = side[1], x2 = side[2];
        float x[NV][EV];
#pragma unroll
        for (int j = 0; j < NV; ++j) unpack(logits, raw[j], x[j]);
        if (at.k0 + 1024 > V) {   // the last, partial round: drop what lies past the row
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const bool in = (at.k0 + (j * 64 + lane) * EV) < V;
#pragma unroll
                for (int i = 0; i < EV; ++i) x[j][i] = in ? x[j][i] : -__builtin_huge_valf();
            }
        }
        float mn = m;
#pragma unroll
        for (int j = 0; j < NV; ++j)
#pragma unroll
            for (int i = 0; i < EV; ++i) mn = fmaxf(mn, x[j][i]);
        // mn = -inf only while everything seen is -inf: keep s = 0 (the floor
        // times log2(e) must stay finite)
        const float mf = fmaxf(mn, -2.0e38f);
        const float shift = -mf * kLog2eF;
        float acc = s * exp2_hw((m - mf) * kLog2eF);
#pragma unroll
        for (int j = 0; j < NV; ++j)
#pragma unroll
            for (int i = 0; i < EV; ++i) acc += exp2_hw(fmaf(x[j][i], kLog2eF, shift));
        s = acc;
        m = mn;
        if (at.k0 + 1024 >= V) {
            finish_row(at.u, m, s, xb, x1, x2);
            m = -__builtin_huge_valf(), s = 0.0f;
        }
    };
    raw16 raw_a[NV], raw_b[NV];
    float side_a[3] = {0.0f, 0.0f, 0.0f}, side_b[3] = {0.0f, 0.0f, 0.0f};
    Step sa = {ulo + wave, 0};
    if (vec && sa.u <= uhi) {
        // Both register sets are kept in flight: a set is asked for again as soon
        // as its step has been worked on.  The steps of this wavefront are
        // counted beforehand and walked in pairs without a branch in between
        // (with one, the compiler's count of outstanding loads turns cautious
        // and it waits for both sets at once).
        const int rounds = (V + 1023) / 1024;
        const int steps = ((uhi - sa.u) / kRowsPerBlock + 1) * rounds;
        Step sb = next_step(sa);
        request(sa, raw_a, side_a);
        request(sb, raw_b, side_b);
        int i = 0;
        for (; i + 2 <= steps; i += 2) {
            work(sa, raw_a, side_a);
            sa = next_step(sb);
            request(sa, raw_a, side_a);
            work(sb, raw_b, side_b);
            sb = next_step(sa);
            request(sb, raw_b, side_b);
        }
        if (i < steps) work(sa, raw_a, side_a);
    }
    if (!STAGED) return;
    __syncthreads();
    for (int i = threadIdx.x; i < P * 3; i += 64 * kRowsPerBlock) frame[i] = staged[i];
    float *lse_row = lse + ((size_t)n * T + t) * (U + 1);
    for (int u = ulo + threadIdx.x; u <= uhi; u += 64 * kRowsPerBlock) lse_row[u] = lse_out[u];
}

// ROWS rows (n,t,u) of the gradient per wavefront, 64 / ROWS lanes each (see
// logits_units_kernel); blockIdx.y = n.
template <typename IO, int ROWS>
__global__ __launch_bounds__(64 * kGradWaves) __attribute__((amdgpu_waves_per_eu(8, 8))) void
logits_grad_kernel(
    const IO *__restrict__ logits, const float *__restrict__ lse, const double *__restrict__ units,
    const double *__restrict__ alphas, const double *__restrict__ betas,
    const int *__restrict__ ys, const int *__restrict__ lx, const int *__restrict__ ly,
    Weight weight, IO *__restrict__ grad, int T, int U, int V, int P) {
    constexpr int LANES = 64 / ROWS;
    constexpr int EV = 16 / (int)sizeof(IO);    // elements per 16-byte vector
    constexpr int ROUND = 1024;                 // elements of a row per round
    constexpr int NV = ROUND / (LANES * EV);    // vectors per lane and round
    const int U1 = U + 1;
    const int n = blockIdx.y;
    const int lane = threadIdx.x & 63, hl = lane % LANES;
    const int cell = (blockIdx.x * kGradWaves + (threadIdx.x >> 6)) * ROWS + lane / LANES;
    if (cell >= T * U1) return;
    const int t = cell / U1, u = cell - t * U1;
    const int lxn = lx[n];
    const int Tn = min(max(lxn, 0), T), Un = min(max(ly[n], 0), U);
    const size_t r = ((size_t)n * T + t) * U1 + u;
    IO *out = grad + r * (size_t)V;
    const bool vec = rows_vectorised(logits, V) && rows_vectorised(grad, V);
    if (t >= Tn || u > Un || outside_band(t, u, Tn, Un)) {
        if (vec) {
            // zeros in 16-byte pieces whatever the element type
            constexpr int E16 = 16 / (int)sizeof(IO);
            typedef unsigned int u4 __attribute__((ext_vector_type(4)));
            for (int k = hl * E16; k < V; k += LANES * E16)
                __builtin_nontemporal_store(u4{0u, 0u, 0u, 0u}, reinterpret_cast<u4 *>(out + k));
        } else {
            for (int k = hl; k < V; k += LANES) store_from_float(out + k, 0.0f);
        }
        return;
    }
    // the first round of the row is requested before the (dependent) loads of
    // the unit gradients, not after them
    const IO *row = logits + r * (size_t)V;
    float x[NV][EV];
    if (vec) {
#pragma unroll
        for (int j = 0; j < NV; ++j) load_vec(row + min((j * LANES + hl) * EV, V - EV), x[j]);
    }
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * P * 2;
    const UnitGrad g = unit_grad_cell(units + (size_t)n * T * P * 3, alphas + (size_t)n * lat,
                                      betas + (size_t)n * lat, y, t, u, Un, P);
    const float w = sample_weight(weight, n, lxn);
    const float g0 = g.g0 * w, g1 = g.g1 * w, g2 = g.g2 * w;   // g1 = 0 at u = 0, g2 = 0 at u = Un
    const float total = g0 + g1 + g2;
    const int c1 = (u >= 1) ? min(max(y[u - 1], 0), V - 1) : -1;
    const int c2 = (u < Un) ? min(max(y[u], 0), V - 1) : -1;
    const float shift = lse[r] * kLog2eF;
    const float neg_shift = -shift, neg_total = -total;
    if (vec) {
        for (int k0 = 0; k0 < V; k0 += ROUND) {
            if (k0 > 0) {
#pragma unroll
                for (int j = 0; j < NV; ++j)
                    load_vec(row + min(k0 + (j * LANES + hl) * EV, V - EV), x[j]);
            }
#pragma unroll
            for (int j = 0; j < NV; ++j) {
                const int k = k0 + (j * LANES + hl) * EV;
                if (k >= V) continue;
#pragma unroll
                for (int i = 0; i < EV; ++i)
                    x[j][i] = neg_total * exp2_hw(fmaf(x[j][i], kLog2eF, neg_shift));
                // the <= 3 columns that also receive a unit gradient: looked for
                // per vector, not per element (few lanes ever find one)
                if ((unsigned)(0 - k) < (unsigned)EV || (unsigned)(c1 - k) < (unsigned)EV ||
                    (unsigned)(c2 - k) < (unsigned)EV) {
#pragma unroll
                    for (int i = 0; i < EV; ++i) {
                        const int col = k + i;
                        float add = 0.0f;
                        if (col == 0) add += g0;
                        if (col == c1) add += g1;
                        if (col == c2) add += g2;
                        x[j][i] += add;
                    }
                }
                store_vec(out + k, x[j]);
            }
        }
    } else {
        for (int k = hl; k < V; k += LANES) {
            float v = -total * exp2_hw(load_as_float(row + k) * kLog2eF - shift);
            if (k == 0) v += g0;
            if (k == c1) v += g1;
            if (k == c2) v += g2;
            store_from_float(out + k, v);
        }
    }
}

// Rows per wavefront by element size: 4 KiB of a row per 64 lanes either way.
template <typename IO> struct RowsPerWave { static constexpr int value = sizeof(IO) == 4 ? 1 : 2; };

template <typename IO>
void launch_units_typed(const void *logits, const int *ys, const int *lx, const int *ly,
                        double *units, float *lse, int N, int T, int U, int V, unsigned *counter,
                        hipStream_t stream) {
    const int P = padded_contexts(U);
    const size_t staged = (size_t)P * (3 * sizeof(double) + sizeof(float));
    if (staged <= 64 * 1024) {
        TIMED_LAUNCH((logits_units_kernel<IO, true>), dim3((unsigned)T, (unsigned)N),
                     dim3(64 * kRowsPerBlock), staged, stream, static_cast<const IO *>(logits), ys,
                     lx, ly, units, lse, T, U, V, P, counter, device_status_word());
    } else {   // a frame too wide for LDS: results stored row by row
        TIMED_LAUNCH((logits_units_kernel<IO, false>), dim3((unsigned)T, (unsigned)N),
                     dim3(64 * kRowsPerBlock), 0, stream, static_cast<const IO *>(logits), ys, lx,
                     ly, units, lse, T, U, V, P, counter, device_status_word());
    }
}

template <typename IO>
void launch_grad_typed(const void *logits, const float *lse, const double *units,
                       const double *alphas, const double *betas, const int *ys, const int *lx,
                       const int *ly, const Weight &w, void *grad, int N, int T, int U, int V,
                       hipStream_t stream) {
    const long cells = (long)T * (U + 1);
    constexpr int ROWS = RowsPerWave<IO>::value, PER_BLOCK = kGradWaves * ROWS;
    dim3 grid((unsigned)((cells + PER_BLOCK - 1) / PER_BLOCK), (unsigned)N);
    TIMED_LAUNCH((logits_grad_kernel<IO, ROWS>), grid, dim3(64 * kGradWaves), 0, stream,
                       static_cast<const IO *>(logits), lse, units, alphas, betas, ys, lx, ly, w,
                       static_cast<IO *>(grad), T, U, V, padded_contexts(U));
}

}  // namespace

hipError_t launch_logits_units(const void *logits, int io_type, const int *ys, const int *lx,
                               const int *ly, double *units, float *lse, int N, int T, int U,
                               int V, unsigned *counter, hipStream_t stream) {
    if (N == 0 || T == 0) return hipSuccess;
    switch (io_type) {
        case kIoF32:
            launch_units_typed<float>(logits, ys, lx, ly, units, lse, N, T, U, V, counter, stream);
            break;
        case kIoF16:
            launch_units_typed<__half>(logits, ys, lx, ly, units, lse, N, T, U, V, counter,
                                       stream);
            break;
        case kIoBF16:
            launch_units_typed<__hip_bfloat16>(logits, ys, lx, ly, units, lse, N, T, U, V, counter,
                                               stream);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

hipError_t launch_logits_grad(const void *logits, int io_type, const float *lse,
                              const double *units, const double *alphas, const double *betas,
                              const int *ys, const int *lx, const int *ly, const float *grad_out,
                              int grad_out_stride, float scale, int average_frames, void *grad,
                              int N, int T, int U, int V, hipStream_t stream) {
    if (N == 0 || T == 0) return hipSuccess;
    const Weight w = {grad_out, grad_out_stride, scale, average_frames};
    switch (io_type) {
        case kIoF32:
            launch_grad_typed<float>(logits, lse, units, alphas, betas, ys, lx, ly, w, grad, N, T,
                                     U, V, stream);
            break;
        case kIoF16:
            launch_grad_typed<__half>(logits, lse, units, alphas, betas, ys, lx, ly, w, grad, N, T,
                                      U, V, stream);
            break;
        case kIoBF16:
            launch_grad_typed<__hip_bfloat16>(logits, lse, units, alphas, betas, ys, lx, ly, w,
                                              grad, N, T, U, V, stream);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace wctct
