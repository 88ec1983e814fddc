// Alpha / beta lattices of the log-add joiner in the LINEAR domain: the fast
// form of lattice.hip's sweeps, used where its result is verified afterwards.
//
// States are path masses (not their logarithms), held in double relative to a
// power of two that the 64 contexts of a wavefront share: mass = value * 2^S.
// A frame is then two multiplications, three multiply-adds or additions and the
// two DPP moves of the neighbouring context's value, against two semiring sums
// (exponential, logarithm, conversions) per state in the log form: a lone
// wavefront pays for every instruction, and a frame costs less than half.
// Every R frames the largest state of the wavefront is brought back to [0.5, 1)
// and S moves by its exponent; the rows a chunk stores are relative to the S of
// that chunk, which is recorded per (sample, direction, wavefront, chunk) for
// the kernel that reads the lattices.
//
// What the linear form cannot do is keep a state that lies more than ~2^-1000
// below the largest state of its 64 contexts: it becomes 0.  That is harmless
// unless the alignments that carry the posterior mass pass through such a
// state.  The kernel that forms the gradients from these lattices therefore
// checks, per frame, that the posteriors it hands out add up to 1 (every
// alignment consumes exactly one unit per frame), and that no unit lies outside
// the range in which R frames can neither overflow nor lose a state on their
// own; if any check fails (or a value is not finite, or a hand-over was lost)
// it raises a flag, and the log-domain kernels of lattice.hip, which follow
// in the same stream and return at once while the flag is down, compute the
// batch again.
//
// Chains of workgroups hand the boundary value over as in lattice.hip (one
// 64-bit slot per boundary and frame, empty / lost patterns, bounded polls);
// the producer's S of a chunk travels in a slot of its own, and the consumer
// rescales what comes in by 2^(S_producer - S_own).  A wavefront that holds no
// mass yet takes over the producer's S, so that the first mass to arrive is not
// rounded against a scale that means nothing.
//
// Math restated from ref_ctct.py:6-74 of the reference, as in lattice.hip.
#include <algorithm>

#include "cost_reduce.h"
#include "device_utils.h"
#include "launch.h"

namespace wctct {

namespace {

constexpr int R = kLinChunk;
constexpr int kRelayPad = 16;   // slots behind a boundary's T, as in lattice.hip
constexpr unsigned long long kEmptyBits = kRelayEmpty;
constexpr unsigned long long kLostBits = kEmptyBits ^ (1ULL << 32);
constexpr int kNoMass = -(1 << 30);   // "exponent" of a wavefront whose states are all 0

struct ChunkL {
    double lp[R][3];
};

typedef unsigned v4u_lin __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void pair_store(double *dst, double o, double e) {
    *reinterpret_cast<double2 *>(dst) = make_double2(o, e);
}

__device__ __forceinline__ void slot_put_lin(unsigned long long *slot, double v) {
    __hip_atomic_store(slot, (unsigned long long)__double_as_longlong(v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// The largest of v over the wavefront, in every lane: four rotations inside the
// rows of 16 lanes (DPP row_ror), then the four rows through scalar registers.
__device__ __forceinline__ int wave_max_int(int v) {
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x128 /* row_ror:8 */, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x124 /* row_ror:4 */, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x122 /* row_ror:2 */, 0xf, 0xf, false));
    v = max(v, __builtin_amdgcn_update_dpp(v, v, 0x121 /* row_ror:1 */, 0xf, 0xf, false));
    const int a = __builtin_amdgcn_readlane(v, 0), b = __builtin_amdgcn_readlane(v, 16);
    const int c = __builtin_amdgcn_readlane(v, 32), d = __builtin_amdgcn_readlane(v, 48);
    return max(max(a, b), max(c, d));
}

static __device__ __forceinline__ void chunk_load_lin(ChunkL &c, const double *units_lane, size_t row,
                                                      int Tn, int t_first, int dir) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = min(max(t_first + dir * r, 0), Tn - 1);
        const double *p = units_lane + (size_t)t * row;
        c.lp[r][0] = p[0];
        c.lp[r][1] = p[1];
        c.lp[r][2] = p[2];
    }
}

// The units of R frames that all exist, through a pointer that walks from row to
// row (two scalar additions per frame instead of a clamp and a 64-bit product):
// `frame` points at the row of the chunk's first frame, the same for all lanes.
template <bool DOWN>
static __device__ __forceinline__ void chunk_load_walk_lin(ChunkL &c, const char *&frame,
                                                           unsigned lane_bytes, unsigned step) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const double *p = reinterpret_cast<const double *>(frame + lane_bytes);
        c.lp[r][0] = p[0];
        c.lp[r][1] = p[1];
        c.lp[r][2] = p[2];
        frame = DOWN ? frame - step : frame + step;
    }
}

// Lane l receives x of lane l-1 / l+1; the lane at the end receives 0 (no value
// flows in from outside the wavefront): DPP with the out-of-range lanes reading 0.
__device__ __forceinline__ double wave_shift_up_zero(double x) {
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(x), 0x138, 0xf, 0xf, true);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(x), 0x138, 0xf, 0xf, true);
    return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double wave_shift_down_zero(double x) {
    const int lo = __builtin_amdgcn_update_dpp(0, __double2loint(x), 0x130, 0xf, 0xf, true);
    const int hi = __builtin_amdgcn_update_dpp(0, __double2hiint(x), 0x130, 0xf, 0xf, true);
    return __hiloint2double(hi, lo);
}

static __device__ __forceinline__ void slots_request_lin(const unsigned long long *slots, int s0,
                                                         unsigned long long (&bits)[R]) {
    const unsigned long long *p = slots + s0;
#pragma unroll
    for (int r = 0; r < R; ++r)
        bits[r] = __hip_atomic_load(p + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// 0: a slot is still empty; 1: none is empty and one says "lost"; else values.
static __device__ __forceinline__ unsigned slots_state_lin(const unsigned long long (&bits)[R], int cnt,
                                                           unsigned long long scale_bits) {
    constexpr unsigned kEmptyHigh = (unsigned)(kEmptyBits >> 32);
    unsigned least = (unsigned)(scale_bits >> 32) ^ kEmptyHigh;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const unsigned d = (unsigned)(bits[r] >> 32) ^ kEmptyHigh;
        least = min(least, r < cnt ? d : 0xffffffffu);
    }
    return (unsigned)__builtin_amdgcn_readfirstlane((int)least);
}

// One direction of the 64 contexts [64*wave, 64*wave + 64) of one lattice.
// Step s handles frame t = s (alpha) or Tn-1-s (beta) and stores the front of
// frame t+1 (alpha) or t (beta), as in lattice.hip.  scales[0] belongs to the
// initial row, scales[1 + k] to the rows that chunk k stores.
// slots_in / scale_in, slots_out / scale_out: the boundary this wavefront reads
// and the one it writes (values per step, the producer's S per chunk), or null.
template <bool BETA, bool HAS_IN>
static __device__ void sweep_lin(const double *units_n, const int *y, int Tn, int Un, int T, int P, int wave,
                                 double *lat_n, int *scales, float *cost_n,
                                 const unsigned long long *slots_in, const unsigned long long *scale_in,
                                 unsigned long long *slots_out, unsigned long long *scale_out,
                                 int max_spins, unsigned *flag, unsigned *status) {
    const int lane = threadIdx.x & 63;
    const int u = wave * 64 + lane;
    double omask = 1.0, skipf, e, o;
    if (BETA) {
        skipf = ((u >= 1) && (u < Un) && (y[u - 1] != y[u])) ? 1.0 : 0.0;
        omask = ((u >= 1) && (u <= Un)) ? 1.0 : 0.0;
        e = (u == Un) ? 1.0 : 0.0;
        o = (u == Un && Un >= 1) ? 1.0 : 0.0;
    } else {
        skipf = ((u >= 1) && (u < Un) && (y[u] != y[u - 1])) ? 1.0 : 0.0;
        e = (u == 0) ? 1.0 : 0.0;
        o = 0.0;
    }
    const size_t srow = (size_t)P * 2, urow = (size_t)P * 3;
    double *out = lat_n + (size_t)u * 2;
    const double *in = units_n + (size_t)u * 3;
    pair_store(out + (size_t)(BETA ? Tn : 0) * srow, o, e);
    if (lane == 0) scales[0] = 0;
    const unsigned out_lane = (unsigned)u * 2u * (unsigned)sizeof(double);
    const unsigned out_step = (unsigned)(srow * sizeof(double));
    char *out_row = reinterpret_cast<char *>(lat_n) + (size_t)(BETA ? Tn - 1 : 1) * srow * sizeof(double);
    const int edge_lane = BETA ? 0 : 63;
    int S = 0;   // the states are mass / 2^S

    if (Tn > 0) {
        ChunkL a, b;
        const int dir = BETA ? -1 : 1;
        const int t_start = BETA ? Tn - 1 : 0;
        chunk_load_lin(a, in, urow, Tn, t_start, dir);
        // The relay slots of a chunk are requested kAhead chunks before they are
        // used: a chunk of this sweep takes ~0.6 us, a slot's way from the
        // producer through the L2 and back longer than that, and a wavefront that
        // looks too early pays a whole round trip for asking again.  Four register
        // sets in rotation (set index = chunk index mod 4): the one chunk k reads
        // was requested at the start of chunk k-3, and the set that chunk k-1 has
        // read takes the request for chunk k+3.
        unsigned long long q0[R], q1[R], q2[R], q3[R];
        unsigned long long sq0 = kEmptyBits, sq1 = kEmptyBits, sq2 = kEmptyBits, sq3 = kEmptyBits;
#pragma unroll
        for (int r = 0; r < R; ++r) q0[r] = q1[r] = q2[r] = q3[r] = kEmptyBits;
        auto request = [&](int k, unsigned long long (&set)[R], unsigned long long &sc) {
            slots_request_lin(slots_in, min(k * R, T), set);
            sc = __hip_atomic_load(scale_in + min(k, lin_chunks(T)), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
        };
        if (HAS_IN) {
            request(0, q0, sq0);
            request(1, q1, sq1);
            request(2, q2, sq2);
        }
        bool lost = false;
        auto run_chunk = [&](const ChunkL &c, unsigned long long (&have)[R], unsigned long long &sc_have,
                             unsigned long long (&next)[R], unsigned long long &sc_next, int s0,
                             int cnt, bool full) {
            const int k = s0 / R;
            double mail[R], mine[R];
#pragma unroll
            for (int r = 0; r < R; ++r) mail[r] = 0.0;
            if (HAS_IN) {
                request(k + 3, next, sc_next);
                unsigned state = slots_state_lin(have, cnt, sc_have);
                if (state == 0 && max_spins > 0 && !lost) {
                    int spins = 0;
                    do {
                        __builtin_amdgcn_s_sleep(2);
                        slots_request_lin(slots_in, s0, have);
                        sc_have = __hip_atomic_load(scale_in + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        state = slots_state_lin(have, cnt, sc_have);
                    } while (state == 0 && ++spins < max_spins);
                }
                if (state <= 1) lost = true;
                if (!lost) {
                    const int S_in = (int)__longlong_as_double((long long)sc_have);
                    // no mass here yet: what flows in sets the scale
                    const bool any = __ballot(e != 0.0 || o != 0.0) != 0ULL;
                    if (!any) S = S_in;
                    // the value belongs to the lane at the boundary; all other lanes
                    // scale theirs down to 0 (every lane has loaded the same slot), so
                    // that it can simply be added to what the DPP move brings
                    const int shift = (lane == (BETA ? 63 : 0)) ? S_in - S : -5000;
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        if (full || r < cnt)
                            mail[r] = __builtin_amdgcn_ldexp(__longlong_as_double((long long)have[r]), shift);
                }
            }
            if (scale_out && !lost && lane == edge_lane) slot_put_lin(scale_out + k, (double)S);
            const int rows_here = full ? R : cnt;
            const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(
                BETA ? out_row - (size_t)(rows_here - 1) * out_step : out_row, 0, 0xffffffffu, 0x00020000);
            unsigned at = BETA ? (unsigned)(rows_here - 1) * out_step : 0u;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                mine[r] = 0.0;
                if (full || r < cnt) {
                    if (BETA) {
                        // beta(t,2u)   = beta(t+1,2u) lp0 + beta(t+1,2u+1) lp2
                        // beta(t,2u-1) = beta(t+1,2u-1) lp1 + beta(t+1,2u) lp0 + [skip] beta(t+1,2u+1) lp2
                        mine[r] = o;
                        const double nb = HAS_IN ? wave_shift_down_zero(o) + mail[r] : wave_shift_down_zero(o);
                        const double nxt = nb * c.lp[r][2];
                        const double stay_e = e * c.lp[r][0];
                        const double sel = __builtin_fma(skipf, nxt, stay_e);
                        o = __builtin_fma(o, c.lp[r][1], sel) * omask;
                        e = stay_e + nxt;
                    } else {
                        // alpha(t+1,2u)   = [alpha(t,2u) + alpha(t,2u-1)] lp0
                        // alpha(t+1,2u-1) = alpha(t,2u-1) lp1 + (what context u-1 sends)
                        // sends: ([skip] alpha(t,2u-1) + alpha(t,2u)) lp2
                        const double sum = e + o;
                        mine[r] = __builtin_fma(o, skipf, e) * c.lp[r][2];
                        const double recv = HAS_IN ? wave_shift_up_zero(mine[r]) + mail[r] : wave_shift_up_zero(mine[r]);
                        o = __builtin_fma(o, c.lp[r][1], recv);
                        e = sum * c.lp[r][0];
                    }
                    v4u_lin w;
                    w[0] = __double2loint(o), w[1] = __double2hiint(o);
                    w[2] = __double2loint(e), w[3] = __double2hiint(e);
                    __builtin_amdgcn_raw_buffer_store_b128(w, rows, out_lane, at, 0);
                    at = BETA ? at - out_step : at + out_step;
                }
            }
            out_row = BETA ? out_row - (size_t)rows_here * out_step : out_row + (size_t)rows_here * out_step;
            if (slots_out && !lost && lane == edge_lane) {
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (full || r < cnt) slot_put_lin(slots_out + s0 + r, mine[r]);
            }
            if (lane == 0) scales[1 + k] = S;
            // the largest state back into [0.5, 1) (not after the last chunk: the
            // cost below is taken from the rows as they were stored)
            if (s0 + cnt < Tn) {
                const double m = __builtin_fmax(e, o);
                int ex = (m > 0.0 && m < __builtin_huge_val()) ? __builtin_amdgcn_frexp_exp(m) : kNoMass;
                ex = wave_max_int(ex);
                if (ex != kNoMass) {
                    e = __builtin_amdgcn_ldexp(e, -ex);
                    o = __builtin_amdgcn_ldexp(o, -ex);
                    S += ex;
                }
            }
        };
        int s0 = 0;
        const unsigned in_lane = (unsigned)u * 3u * (unsigned)sizeof(double);
        const unsigned in_step = (unsigned)(urow * sizeof(double));
        // four chunks per turn (the slot sets come round); while the chunk after
        // the turn lies inside the sample, the rows of units need no clamp
        if (5 * R <= Tn) {
            const char *frame = reinterpret_cast<const char *>(units_n) +
                                (size_t)(t_start + dir * R) * urow * sizeof(double);
            do {
                chunk_load_walk_lin<BETA>(b, frame, in_lane, in_step);
                run_chunk(a, q0, sq0, q3, sq3, s0, R, true);
                chunk_load_walk_lin<BETA>(a, frame, in_lane, in_step);
                run_chunk(b, q1, sq1, q0, sq0, s0 + R, R, true);
                chunk_load_walk_lin<BETA>(b, frame, in_lane, in_step);
                run_chunk(a, q2, sq2, q1, sq1, s0 + 2 * R, R, true);
                chunk_load_walk_lin<BETA>(a, frame, in_lane, in_step);
                run_chunk(b, q3, sq3, q2, sq2, s0 + 3 * R, R, true);
                s0 += 4 * R;
            } while (s0 + 5 * R <= Tn);
        }
        // the rest (fewer than five chunks), one chunk per turn: the sets move up
        // by copies instead
        while (s0 < Tn) {
            chunk_load_lin(b, in, urow, Tn, t_start + dir * (s0 + R), dir);
            run_chunk(a, q0, sq0, q3, sq3, s0, min(Tn - s0, R), false);
            a = b;
#pragma unroll
            for (int r = 0; r < R; ++r) q0[r] = q1[r], q1[r] = q2[r], q2[r] = q3[r];
            sq0 = sq1, sq1 = sq2, sq2 = sq3;
            s0 += R;
        }
        if (lost) {
            // the log-domain kernels take over; whoever waits behind is told
            if (lane == 0) {
                atomicOr(flag, 1u);
                if (status) atomicOr(status, kStatusLostHandOver);
            }
            if (slots_out && lane == edge_lane) {
                for (int s = 0; s < Tn; ++s)
                    __hip_atomic_store(slots_out + s, kLostBits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                for (int k = 0; k * R < Tn; ++k)
                    __hip_atomic_store(scale_out + k, kLostBits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    // cost = -ln(beta(0, state 0) * 2^S)
    if (BETA && u == 0) {
        float c = __builtin_huge_valf();
        if (e > 0.0) {
            const int ex = __builtin_amdgcn_frexp_exp(e);
            const float mant = (float)__builtin_amdgcn_ldexp(e, -ex);   // in [0.5, 1)
            c = (float)(-((double)log2_hw(mant) + (double)(ex + S)) * kLn2);
        }
        *cost_n = c;
    }
}

__global__ __launch_bounds__(64) void lattice_lin_kernel(
    const double *__restrict__ units, const int *__restrict__ ys, const int *__restrict__ lx,
    const int *__restrict__ ly, double *__restrict__ alphas, double *__restrict__ betas,
    int *__restrict__ scales, float *__restrict__ costs, unsigned long long *__restrict__ relay, int N,
    int T, int U, int W, int chains_pad, const CostReduce red, int max_spins,
    unsigned *__restrict__ flag, unsigned *__restrict__ status) {
    // workgroup index = link * chains_pad + chain, chain = n * 2 + d (d = 0: beta,
    // 1: alpha), first producer first, as in lattice.hip
    const int chain = blockIdx.x % chains_pad, link = blockIdx.x / chains_pad;
    if (chain >= N * 2) return;
    const int n = chain / 2;
    const bool beta = (chain % 2) == 0;
    const int wave = beta ? W - 1 - link : link;
    const int P = 64 * W;
    const int Tn = min(max(lx[n], 0), T);
    const int Un = min(max(ly[n], 0), U);
    if (wave * 64 > Un) return;
    const double *units_n = units + (size_t)n * T * P * 3;
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * P * 2;
    const int chunks = lin_chunks(T);
    int *sc = scales + (((size_t)n * 2 + (beta ? 0 : 1)) * W + wave) * (size_t)(chunks + 1);
    // slots of one boundary and direction: T + kRelayPad values, then chunks + 1 scales
    const size_t TS = (size_t)T + kRelayPad + (size_t)chunks + 1;
    unsigned long long *slots_n =
        relay ? relay + ((size_t)n * 2 + (beta ? 0 : 1)) * (size_t)(W - 1) * TS : nullptr;
    const size_t to_scales = (size_t)T + kRelayPad;
    if (!beta) {
        const unsigned long long *in = wave > 0 ? slots_n + (size_t)(wave - 1) * TS : nullptr;
        unsigned long long *out = (wave + 1) * 64 <= Un ? slots_n + (size_t)wave * TS : nullptr;
        if (in)
            sweep_lin<false, true>(units_n, y, Tn, Un, T, P, wave, alphas + (size_t)n * lat, sc, nullptr, in,
                                   in + to_scales, out, out ? out + to_scales : nullptr, max_spins, flag,
                                   status);
        else
            sweep_lin<false, false>(units_n, y, Tn, Un, T, P, wave, alphas + (size_t)n * lat, sc, nullptr,
                                    nullptr, nullptr, out, out ? out + to_scales : nullptr, max_spins, flag,
                                    status);
        return;
    }
    {
        const unsigned long long *in = (wave + 1) * 64 <= Un ? slots_n + (size_t)wave * TS : nullptr;
        unsigned long long *out = wave > 0 ? slots_n + (size_t)(wave - 1) * TS : nullptr;
        if (in)
            sweep_lin<true, true>(units_n, y, Tn, Un, T, P, wave, betas + (size_t)n * lat, sc, costs + n, in,
                                  in + to_scales, out, out ? out + to_scales : nullptr, max_spins, flag,
                                  status);
        else
            sweep_lin<true, false>(units_n, y, Tn, Un, T, P, wave, betas + (size_t)n * lat, sc, costs + n,
                                   nullptr, nullptr, out, out ? out + to_scales : nullptr, max_spins, flag,
                                   status);
    }
    if (wave != 0) return;
    cost_reduce_tail(red, costs, lx, n, N, threadIdx.x);
}

}  // namespace

size_t lattice_lin_relay_slots(int N, int T, int U) {
    const int W = (U + 1 + 63) / 64;
    return (size_t)N * 2 * (size_t)(W - 1) * ((size_t)T + kRelayPad + (size_t)lin_chunks(T) + 1);
}

size_t lattice_lin_scales(int N, int T, int U) {
    const int W = (U + 1 + 63) / 64;
    return (size_t)N * 2 * W * (size_t)(lin_chunks(T) + 1);
}

hipError_t launch_lattice_lin(const LatticeArgs &a, int *scales, unsigned *flag, hipStream_t stream) {
    if (a.N == 0) return hipSuccess;
    if (a.beta_only || !scales || !flag) return hipErrorInvalidValue;
    const int W = (a.U + 1 + 63) / 64;
    const size_t slots = lattice_lin_relay_slots(a.N, a.T, a.U);
    unsigned long long *relay = slots ? reinterpret_cast<unsigned long long *>(a.relay) : nullptr;
    if (slots > 0 && (!relay || !a.relay_is_clear)) return hipErrorInvalidValue;
    const long chains_pad = ((long)a.N * 2 + 7) / 8 * 8;
    if (chains_pad * W > 0x7fffffffL) return hipErrorInvalidValue;
    const int max_spins = lattice_wait_limit_now();
    TIMED_LAUNCH(lattice_lin_kernel, dim3((unsigned)(chains_pad * W)), dim3(64), 0, stream, a.units, a.ys,
                 a.lx, a.ly, a.alphas, a.betas, scales, a.costs, relay, a.N, a.T, a.U, W, (int)chains_pad,
                 a.reduce, max_spins, flag, device_status_word());
    return hipGetLastError();
}

}  // namespace wctct
