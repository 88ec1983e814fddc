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
// 64-bit slot per boundary and frame, empty / lost patterns, bounded polls),
// here with the slots of a chunk in one line of 128 bytes: R values, then the
// producer's S of the chunk.  The consumer fetches the line with one load (lane
// r holds step r's value) and rescales it by 2^(S_producer - S_own) at once.  A wavefront that holds no
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
constexpr int kLine = 16;       // slots of a chunk's line: R values, the scale, spare ones
constexpr int kLinesAhead = 4;  // lines behind a boundary's last chunk that a request may touch
static_assert(R < kLine, "a chunk's values and its scale share a line");
constexpr unsigned long long kEmptyBits = kRelayEmpty;
constexpr unsigned long long kLostBits = kEmptyBits ^ (1ULL << 32);

struct ChunkL {
    double lp[R][3];
};

typedef unsigned v4u_lin __attribute__((ext_vector_type(4)));
typedef unsigned v2u_lin __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void pair_store(double *dst, double o, double e) {
    *reinterpret_cast<double2 *>(dst) = make_double2(o, e);
}

__device__ __forceinline__ void slot_put_lin(unsigned long long *slot, double v) {
    __hip_atomic_store(slot, (unsigned long long)__double_as_longlong(v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// The largest of v >= 0 over the wavefront, as a scalar: four rotations inside
// the rows of 16 lanes (DPP row_ror), then the four rows through scalar registers.
__device__ __forceinline__ int wave_max_nonneg(int v) {
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x128 /* row_ror:8 */, 0xf, 0xf, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x124 /* row_ror:4 */, 0xf, 0xf, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x122 /* row_ror:2 */, 0xf, 0xf, true));
    v = max(v, __builtin_amdgcn_update_dpp(0, v, 0x121 /* row_ror:1 */, 0xf, 0xf, true));
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

// The units of R frames that all exist, through a buffer descriptor over the
// sample's units and a scalar offset that walks from row to row (one scalar
// addition per frame; the lane's part of the address is a constant register):
// `at` is the byte offset of the row of the chunk's first frame.
template <bool DOWN>
static __device__ __forceinline__ void chunk_load_walk_lin(ChunkL &c, __amdgpu_buffer_rsrc_t units,
                                                           unsigned &at, unsigned lane_bytes, unsigned step) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const v4u_lin w = __builtin_amdgcn_raw_buffer_load_b128(units, lane_bytes, at, 0);
        const v2u_lin x = __builtin_amdgcn_raw_buffer_load_b64(units, lane_bytes + 16u, at, 0);
        c.lp[r][0] = __hiloint2double((int)w[1], (int)w[0]);
        c.lp[r][1] = __hiloint2double((int)w[3], (int)w[2]);
        c.lp[r][2] = __hiloint2double((int)x[1], (int)x[0]);
        at = DOWN ? at - step : at + step;
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

// What a chunk needs from the boundary it reads, in one load: lane r < R asks
// for the value of the chunk's step r, lane R for the producer's S of the chunk
// (the lanes behind repeat lane R).  `lines` is a descriptor over the boundary's
// lines, lane_bytes = 8 * min(lane, R).
static __device__ __forceinline__ unsigned long long chunk_request_lin(__amdgpu_buffer_rsrc_t lines, int k,
                                                                       unsigned lane_bytes) {
    const v2u_lin w = __builtin_amdgcn_raw_buffer_load_b64(lines, lane_bytes, (unsigned)k * (kLine * 8u),
                                                           16 /* sc1: at agent scope */);
    return ((unsigned long long)w[1] << 32) | w[0];
}

// 0: one of the chunk's cnt values or its scale is still empty; 1: none is
// empty and one says "lost"; else all are there.
static __device__ __forceinline__ unsigned chunk_state_lin(unsigned long long bits, int cnt) {
    constexpr unsigned kEmptyHigh = (unsigned)(kEmptyBits >> 32);
    constexpr unsigned kLostHigh = (unsigned)(kLostBits >> 32);
    const unsigned hi = (unsigned)(bits >> 32);
    const unsigned long long need = ((1ULL << cnt) - 1ULL) | (1ULL << R);
    if (__ballot(hi == kEmptyHigh) & need) return 0u;
    if (__ballot(hi == kLostHigh) & need) return 1u;
    return 2u;
}

// The double that lane `from` holds, as a scalar.
template <int from>
static __device__ __forceinline__ double lane_value(double x) {
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(x), from),
                            __builtin_amdgcn_readlane(__double2loint(x), from));
}
static __device__ __forceinline__ double mail_at(double x, int r) {   // r: constant once unrolled
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(x), r),
                            __builtin_amdgcn_readlane(__double2loint(x), r));
}

// One direction of the 64 contexts [64*wave, 64*wave + 64) of one lattice.
// Step s handles frame t = s (alpha) or Tn-1-s (beta) and stores the front of
// frame t+1 (alpha) or t (beta), as in lattice.hip.  scales[0] belongs to the
// initial row, scales[1 + k] to the rows that chunk k stores.
// lines_in, lines_out: the lines (one per chunk) of the boundary this wavefront
// reads and of the one it writes, or null.
template <bool BETA, bool HAS_IN>
static __device__ void sweep_lin(const double *units_n, const int *y, int Tn, int Un, int T, int P, int wave,
                                 double *lat_n, int *scales, float *cost_n, const unsigned long long *lines_in,
                                 unsigned long long *lines_out, int max_spins, unsigned *flag,
                                 unsigned *status) {
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
        // What a chunk needs from the boundary is requested three chunks before
        // it is used: a chunk of this sweep takes ~0.6 us, a slot's way from the
        // producer through the L2 and back longer than that, and a wavefront that
        // looks too early pays a whole round trip for asking again.  Four registers
        // in rotation (index = chunk index mod 4): the one chunk k reads was
        // requested at the start of chunk k-3, and the one that chunk k-1 has read
        // takes the request for chunk k+3.
        unsigned long long q0 = kEmptyBits, q1 = kEmptyBits, q2 = kEmptyBits, q3 = kEmptyBits;
        const __amdgpu_buffer_rsrc_t lines = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<unsigned long long *>(lines_in), 0, 0xffffffffu, 0x00020000);
        const unsigned line_lane = 8u * (unsigned)min(lane, R);
        // (a request past the last chunk reads one of the kLinesAhead spare lines)
        auto request = [&](int k) { return chunk_request_lin(lines, k, line_lane); };
        if (HAS_IN) {
            q0 = request(0);
            q1 = request(1);
            q2 = request(2);
        }
        // 1 in the lane whose context borders on the producer's, 0 elsewhere
        const double in_lane = (lane == (BETA ? 63 : 0)) ? 1.0 : 0.0;
        bool lost = false;
        auto run_chunk = [&](const ChunkL &c, unsigned long long &have, unsigned long long &next, int k,
                             int cnt, bool full, bool last) {
            double mine[R];
            double mail = 0.0;   // lane r: what flows in at step r of this chunk, in this wavefront's scale
            if (HAS_IN) {
                next = request(k + 3);
                unsigned state = chunk_state_lin(have, cnt);
                if (state == 0 && max_spins > 0 && !lost) {
                    int spins = 0;
                    do {
                        __builtin_amdgcn_s_sleep(2);
                        have = request(k);
                        state = chunk_state_lin(have, cnt);
                    } while (state == 0 && ++spins < max_spins);
                }
                if (state <= 1) lost = true;
                if (!lost) {
                    const double got = __longlong_as_double((long long)have);
                    const int S_in = (int)lane_value<R>(got);
                    // no mass here yet: what flows in sets the scale
                    const bool any = __ballot(e != 0.0 || o != 0.0) != 0ULL;
                    if (!any) S = S_in;
                    mail = __builtin_amdgcn_ldexp(got, S_in - S);
                }
            }
            unsigned long long *line_out = lines_out + (size_t)k * kLine;
            if (lines_out && !lost && lane == edge_lane) slot_put_lin(line_out + R, (double)S);
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
                        const double nb = HAS_IN ? __builtin_fma(mail_at(mail, r), in_lane, wave_shift_down_zero(o))
                                                 : wave_shift_down_zero(o);
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
                        const double recv = HAS_IN ? __builtin_fma(mail_at(mail, r), in_lane, wave_shift_up_zero(mine[r]))
                                                   : wave_shift_up_zero(mine[r]);
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
            if (lines_out && !lost && lane == edge_lane) {
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (full || r < cnt) slot_put_lin(line_out + r, mine[r]);
            }
            if (lane == 0) scales[1 + k] = S;
            // the largest state back into [0.5, 1) (not after the last chunk: the
            // cost below is taken from the rows as they were stored).  The states
            // are not negative, so the largest one has the largest high word, whose
            // bits 20.. are its exponent + 1023: scalar arithmetic from there on.
            // All states 0 (or below the normal range): nothing to scale; a state
            // that is not finite: the check behind the sweeps will say so.
            if (!last) {
                const int top = wave_max_nonneg(max(__double2hiint(e), __double2hiint(o))) >> 20;
                if (top > 0 && top < 0x7ff) {
                    const int ex = top - 1022;
                    e = __builtin_amdgcn_ldexp(e, -ex);
                    o = __builtin_amdgcn_ldexp(o, -ex);
                    S += ex;
                }
            }
        };
        int s0 = 0;
        // four chunks per turn (the requests come round); while the chunk after
        // the turn lies inside the sample, the rows of units need no clamp
        if (5 * R <= Tn) {
            const __amdgpu_buffer_rsrc_t rows_in = __builtin_amdgcn_make_buffer_rsrc(
                const_cast<double *>(units_n), 0, 0xffffffffu, 0x00020000);
            const unsigned in_bytes = (unsigned)u * 3u * (unsigned)sizeof(double);
            const unsigned in_step = (unsigned)(urow * sizeof(double));
            unsigned at = (unsigned)(t_start + dir * R) * in_step;
            int k = 0;
            do {
                chunk_load_walk_lin<BETA>(b, rows_in, at, in_bytes, in_step);
                run_chunk(a, q0, q3, k, R, true, false);
                chunk_load_walk_lin<BETA>(a, rows_in, at, in_bytes, in_step);
                run_chunk(b, q1, q0, k + 1, R, true, false);
                chunk_load_walk_lin<BETA>(b, rows_in, at, in_bytes, in_step);
                run_chunk(a, q2, q1, k + 2, R, true, false);
                chunk_load_walk_lin<BETA>(a, rows_in, at, in_bytes, in_step);
                run_chunk(b, q3, q2, k + 3, R, true, false);
                k += 4;
                s0 += 4 * R;
            } while (s0 + 5 * R <= Tn);
        }
        // the rest (fewer than five chunks), one chunk per turn: the requests move
        // up by copies instead
        while (s0 < Tn) {
            chunk_load_lin(b, in, urow, Tn, t_start + dir * (s0 + R), dir);
            run_chunk(a, q0, q3, s0 / R, min(Tn - s0, R), false, s0 + R >= Tn);
            a = b;
            q0 = q1, q1 = q2, q2 = q3;
            s0 += R;
        }
        if (lost) {
            // the log-domain kernels take over; whoever waits behind is told
            if (lane == 0) {
                atomicOr(flag, 1u);
                if (status) atomicOr(status, kStatusLostHandOver);
            }
            if (lines_out && lane == edge_lane) {
                for (int k = 0; k * R < Tn; ++k)
                    for (int r = 0; r <= R; ++r)
                        __hip_atomic_store(lines_out + (size_t)k * kLine + r, kLostBits, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
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
    // one boundary and direction: a line per chunk and the spare lines behind
    const size_t TS = (size_t)(chunks + kLinesAhead) * kLine;
    unsigned long long *lines_n =
        relay ? relay + ((size_t)n * 2 + (beta ? 0 : 1)) * (size_t)(W - 1) * TS : nullptr;
    if (!beta) {
        const unsigned long long *in = wave > 0 ? lines_n + (size_t)(wave - 1) * TS : nullptr;
        unsigned long long *out = (wave + 1) * 64 <= Un ? lines_n + (size_t)wave * TS : nullptr;
        if (in)
            sweep_lin<false, true>(units_n, y, Tn, Un, T, P, wave, alphas + (size_t)n * lat, sc, nullptr, in,
                                   out, max_spins, flag, status);
        else
            sweep_lin<false, false>(units_n, y, Tn, Un, T, P, wave, alphas + (size_t)n * lat, sc, nullptr,
                                    nullptr, out, max_spins, flag, status);
        return;
    }
    {
        const unsigned long long *in = (wave + 1) * 64 <= Un ? lines_n + (size_t)wave * TS : nullptr;
        unsigned long long *out = wave > 0 ? lines_n + (size_t)(wave - 1) * TS : nullptr;
        if (in)
            sweep_lin<true, true>(units_n, y, Tn, Un, T, P, wave, betas + (size_t)n * lat, sc, costs + n, in,
                                  out, max_spins, flag, status);
        else
            sweep_lin<true, false>(units_n, y, Tn, Un, T, P, wave, betas + (size_t)n * lat, sc, costs + n,
                                   nullptr, out, max_spins, flag, status);
    }
    if (wave != 0) return;
    cost_reduce_tail(red, costs, lx, n, N, threadIdx.x);
}

}  // namespace

size_t lattice_lin_relay_slots(int N, int T, int U) {
    const int W = (U + 1 + 63) / 64;
    return (size_t)N * 2 * (size_t)(W - 1) * (size_t)(lin_chunks(T) + kLinesAhead) * kLine;
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
    // a sample's units are addressed through 32-bit byte offsets
    if ((size_t)a.T * 64 * W * 3 * sizeof(double) >= (1ULL << 31)) return hipErrorInvalidValue;
    const int max_spins = lattice_wait_limit_now();
    TIMED_LAUNCH(lattice_lin_kernel, dim3((unsigned)(chains_pad * W)), dim3(64), 0, stream, a.units, a.ys,
                 a.lx, a.ly, a.alphas, a.betas, scales, a.costs, relay, a.N, a.T, a.U, W, (int)chains_pad,
                 a.reduce, max_spins, flag, device_status_word());
    return hipGetLastError();
}

}  // namespace wctct
