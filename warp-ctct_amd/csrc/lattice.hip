// Alpha / beta lattices of the CTC-Transducer loss on gfx950.
//
// The sweep is time-synchronous: all states of frame t are updated from frame
// t-1 (alpha) or t+1 (beta); states of one frame do not depend on each other,
// so a step needs no barrier and no atomics — only one value from the
// neighbouring context.  Every lane owns one context u and its state pair
//     o = state 2u-1 (inside label y[u-1])      e = state 2u (blank after u labels)
// in registers; the value of the neighbouring context moves with single-lane
// DPP shifts.
//
// One wavefront sweeps 64 contexts and is a workgroup of its own.  A lattice
// with more contexts is a chain of W = ceil((U+1)/64) such workgroups, each on
// its own compute unit (a compute unit's vector-memory path serves ~64 bytes
// per clock: five wavefronts of one lattice sharing it ran at 178 ns per frame
// against 92 ns for one alone).  The one value that crosses a 64-context
// boundary per frame is handed from workgroup to workgroup through a slot in
// device memory, one slot per (boundary, frame): the producer stores the value
// itself, the consumer polls the slot until it no longer holds the "empty"
// pattern.  Value and "it is there" are one 64-bit word, so the hand-over needs
// no fences and no counters.  A consumer runs one chunk of R frames behind its
// producer and asks for the next chunk's slots while it sweeps the current one.
// Workgroups are ordered so that a producer always has a lower index than its
// consumer (workgroups are dispatched in index order: a waiting consumer's
// producer is running or done), and all links of a chain share `index % 8`,
// i.e. the XCD and its L2, under round-robin dispatch.
// A wait is bounded; a consumer whose wait runs out fills the rows it could not
// sweep properly with NaN and stores a "lost" pattern instead of values, which
// makes the workgroups behind it do the same: the gradients, and the cost when
// the beta chain is hit, come out as NaN instead of a plausible number.
//
// Values are log2 of the path mass, held in double; the exponentials and
// logarithms of the semiring sum run on the fp32 transcendental unit (see
// device_utils.h).  Units for the next chunk of R frames are prefetched into
// registers while the current chunk is swept.
//
// Math restated from ref_ctct.py:6-74 of the reference (alpha :6-37, beta
// :40-74); this kernel replaces k_warp_alphas / k_warp_betas
// (csrc/gather.cu:36-291) and their global-memory spin-lock row pipeline.
#include <atomic>

#include "cost_reduce.h"
#include "device_utils.h"
#include "launch.h"

namespace wctct {

namespace {

constexpr int kRelayPad = 16;   // slots behind a boundary's T: a request may start at any step <= T
constexpr int kMaxSpins = 1 << 20;   // ~1 s of polling before a hand-over is given up (default)

// What a relay slot holds before its value has been stored: a NaN with a
// payload that no arithmetic produces.
constexpr unsigned long long kEmptyBits = kRelayEmpty;
// What a workgroup that has lost its input (its wait ran out, or its producer
// lost its own) stores instead of values: another such NaN, one bit away in the
// high word, so that one comparison tells empty, lost and value apart.
constexpr unsigned long long kLostBits = kEmptyBits ^ (1ULL << 32);

struct Front {
    double e, o;
};

// Work buffers are padded to P = 64*W contexts per frame so that every lane
// loads and stores unconditionally: no exec-mask branches in the sweep, which
// lets the compiler count outstanding loads exactly and keep the prefetch of
// the next chunk in flight while the current one is consumed.
//   units  (N, T,   P, 3)  {blank, cur, next}; for u > Un: {0, 0, -inf},
//                          and next = -inf at u = Un (no label follows)
//   alpha, beta (N, T+1, P, 2) pairs {o, e}
__device__ __forceinline__ void front_store(double *dst, const Front &f) {
    *reinterpret_cast<double2 *>(dst) = make_double2(f.o, f.e);
}

// A lone wavefront issues one instruction at a time, so the address arithmetic
// of a frame costs as much as its semiring sums.  Rows are therefore walked:
// loads follow a pointer that moves by one row per frame (two scalar additions
// instead of a clamp and a 64-bit product), stores go through a buffer
// descriptor: descriptor (the chunk's row of lowest address, in scalar
// registers) + scalar byte offset of the frame + the lane's own 32-bit offset,
// all inside the store instruction.  The descriptor's range is left open
// (offsets stay inside the rows by construction).  Loads through a descriptor
// were measured too: chains of five workgroups ran 10 % slower with them.
typedef unsigned v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t rows_from(const void *lowest) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(lowest), 0, 0xffffffffu, 0x00020000);
}

__device__ __forceinline__ void front_store_at(__amdgpu_buffer_rsrc_t rows, unsigned lane_bytes,
                                               unsigned at, const Front &f) {
    v4u w;
    w[0] = __double2loint(f.o), w[1] = __double2hiint(f.o);
    w[2] = __double2loint(f.e), w[3] = __double2hiint(f.e);
    // (the sum is formed where it is used: the row offsets of a whole chunk are
    // the same for every chunk, and kept in a register each they would take the
    // kernel with the clear riding along from 164 to 170 registers per lane, from
    // three workgroups per compute unit to two, and the clear of 2 GB from 287 to
    // 295 us)
    asm volatile("" : "+s"(at));
    __builtin_amdgcn_raw_buffer_store_b128(w, rows, lane_bytes + at, 0, 0);
}

// ---- hand-over between the workgroups of one lattice -------------------------
// slots[s] belongs to step s of the sweep (s < Tn <= T); a boundary has
// T + kRelayPad of them.  Relaxed atomics at agent scope: the store goes to the L2,
// the load comes from there.
__device__ __forceinline__ void slot_put(unsigned long long *slot, double v) {
    __hip_atomic_store(slot, (unsigned long long)__double_as_longlong(v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}

// ---- alpha ---------------------------------------------------------------
// alpha(t+1, 2u)   = [alpha(t,2u) (+) alpha(t,2u-1)] + LP(t,u,0)
// alpha(t+1, 2u-1) =  alpha(t,2u-1) + LP(t,u,1)
//                 (+) alpha(t,2u-2) + LP(t,u-1,2)
//                 (+) [y[u-1] != y[u-2]] alpha(t,2u-3) + LP(t,u-1,2)
// The last two terms are what context u-1 sends to context u; with
// L = alpha(t,2u-2) (+) alpha(t,2u-3), which context u-1 needs anyway for its
// own blank state, they are  (skip arc ? L : alpha(t,2u-2)) + LP(t,u-1,2):
// one semiring sum and one value to pass instead of two of each.
// skip_next: the skip arc from this context's label state into the next
// context exists (y[u] != y[u-1]).  ext = what lane 0 receives (from the
// previous 64 contexts, or -inf); out = what this lane sends to context u+1.
__device__ __forceinline__ void alpha_step(Front &f, const double *lp, bool skip_next, double ext,
                                           double &out) {
    const double top = __builtin_fmax(f.e, f.o) + 1.0;
    const double l = (double)half_sum_log2((float)(f.e - f.o));      // both = top + l
    out = skip_next ? (top + lp[2]) + l : f.e + lp[2];
    const double recv = wave_shift_up(out, ext);
    const double stay = f.o + lp[1];
    const double l2 = (double)half_sum_log2((float)(recv - stay));
    f.e = (top + lp[0]) + l;
    f.o = (__builtin_fmax(stay, recv) + 1.0) + l2;
}

// ---- beta ----------------------------------------------------------------
// beta(t, 2u)   = beta(t+1,2u) + LP(t,u,0)  (+) [u<U] beta(t+1,2u+1) + LP(t,u,2)
// beta(t, 2u-1) = beta(t+1,2u-1) + LP(t,u,1) (+) beta(t+1,2u) + LP(t,u,0)
//              (+) [u<U, y[u-1] != y[u]] beta(t+1,2u+1) + LP(t,u,2)
// The last two terms of the second line are beta(t,2u) itself when the skip
// arc exists and its first term alone when it does not.
// skip: y[u-1] != y[u] with 1 <= u < Un.  o_mask is 0 for contexts that have a
// state 2u-1 (1 <= u <= Un), else -inf.  ext = beta(t+1, 2u+1) for lane 63
// (from the next 64 contexts, or -inf); out = this lane's beta(t+1, 2u-1),
// which context u-1 needs.
__device__ __forceinline__ void beta_step(Front &f, const double *lp, bool skip, double o_mask,
                                          double ext, double &out) {
    out = f.o;
    const double nb = wave_shift_down(f.o, ext);
    const double nxt = nb + lp[2];
    const double stay_e = f.e + lp[0];
    const double l = (double)half_sum_log2((float)(stay_e - nxt));
    const double ne = (__builtin_fmax(stay_e, nxt) + 1.0) + l;
    const double sel = skip ? ne : stay_e;
    const double stay_o = f.o + lp[1];
    const double l2 = (double)half_sum_log2((float)(stay_o - sel));
    f.e = ne;
    f.o = (__builtin_fmax(stay_o, sel) + (1.0 + o_mask)) + l2;
}

// Every relay slot = empty, before the sweeps of a launch.
__global__ __launch_bounds__(256) void relay_clear_kernel(unsigned long long *slots, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) slots[i] = kEmptyBits;
}

// Everything that depends on the chunk size R (frames per chunk: prefetch depth
// and hand-over granularity).  Two sizes are in use: 12 for the plain lattice
// launch (units asked for 1.5 us ahead: 3-7 % faster sweeps than with 8; 16 is the
// same within noise at the register limit, 24 slower), 8 for the launch that also
// clears memory, whose clearing workgroups share the kernel's register count and
// need four wavefronts per SIMD (at 16 the kernel takes 256 registers and the
// clear twice its time).
template <int R>
struct Chunked {
struct Chunk {
    double lp[R][3];
};

// Units of frames t_first + dir*r, r in [0,R); the frame index is clamped into
// [0, Tn-1] so that a prefetch past the end re-reads a valid row (its values
// are then not used).
static __device__ __forceinline__ void chunk_load(Chunk &c, const double *units_lane, size_t row, int Tn,
                                           int t_first, int dir) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = min(max(t_first + dir * r, 0), Tn - 1);
        const double *p = units_lane + (size_t)t * row;
        c.lp[r][0] = p[0];
        c.lp[r][1] = p[1];
        c.lp[r][2] = p[2];
    }
}

// The units of R frames that all exist.  `frame` points at the row of the
// chunk's first frame (the same for all lanes) and is moved on by the chunk;
// `step` = bytes per frame; DOWN: frames run towards lower addresses.
template <bool DOWN>
static __device__ __forceinline__ void chunk_load_walk(Chunk &c, const char *&frame, unsigned lane_bytes,
                                                unsigned step) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const double *p = reinterpret_cast<const double *>(frame + lane_bytes);
        c.lp[r][0] = p[0];
        c.lp[r][1] = p[1];
        c.lp[r][2] = p[2];
        frame = DOWN ? frame - step : frame + step;
    }
}

// Requests the slots of steps s0 .. s0+R-1 (a boundary has T + kRelayPad slots, so a
// request that starts at any step s0 <= T stays inside; what lies beyond the
// chunk's cnt steps is not looked at).  Nothing waits for the loads until the
// values are used.
static __device__ __forceinline__ void slots_request(const unsigned long long *slots, int s0,
                                              unsigned long long (&bits)[R]) {
    const unsigned long long *p = slots + s0;
#pragma unroll
    for (int r = 0; r < R; ++r)
        bits[r] = __hip_atomic_load(p + r, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// State of the chunk's cnt slots: the smallest of (high word xor the empty
// pattern's).  0: one is still empty; 1: none is empty and one says "lost";
// anything else: all hold values (no value has either high word: they are NaN
// payloads no arithmetic produces).  The same for all lanes.
static __device__ __forceinline__ unsigned slots_state(const unsigned long long (&bits)[R], int cnt) {
    constexpr unsigned kEmptyHigh = (unsigned)(kEmptyBits >> 32);
    unsigned least = 0xffffffffu;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const unsigned d = (unsigned)(bits[r] >> 32) ^ kEmptyHigh;
        least = min(least, r < cnt ? d : 0xffffffffu);
    }
    return (unsigned)__builtin_amdgcn_readfirstlane((int)least);
}

// One direction of the 64 contexts [64*wave, 64*wave + 64) of one lattice.
// BETA selects the direction; step s handles frame t = s (alpha) or Tn-1-s
// (beta) and stores the front of frame t+1 (alpha) or t (beta).
// slots_in / slots_out: the T relay slots of the boundary this wavefront reads
// (null: nothing flows in, the neighbour is -inf) and writes (null: no
// neighbour on that side).
// HAS_IN: boundary values flow in (slots_in is not null).  A template argument
// rather than a test of the pointer: with both cases in one body the values
// that enter lane 0 / lane 63 are copied once more per frame, and a lone
// wavefront pays for every instruction (chains of five: 199 -> 182 us).
template <bool BETA, bool HAS_IN>
static __device__ void sweep(const double *units_n, const int *y, int Tn, int Un, int T, int P, int wave,
                      double *lat_n, float *cost_n, const unsigned long long *slots_in,
                      unsigned long long *slots_out, int max_spins, unsigned *status) {
    const int lane = threadIdx.x & 63;
    const int u = wave * 64 + lane;
    double o_mask = 0.0;
    bool skip;
    Front f;
    if (BETA) {
        skip = (u >= 1) && (u < Un) && (y[u - 1] != y[u]);
        o_mask = ((u >= 1) && (u <= Un)) ? 0.0 : neg_inf();
        f.e = (u == Un) ? 0.0 : neg_inf();
        f.o = (u == Un && Un >= 1) ? 0.0 : neg_inf();
    } else {
        // the skip arc from this context into context u+1
        skip = (u >= 1) && (u < Un) && (y[u] != y[u - 1]);
        f.e = (u == 0) ? 0.0 : neg_inf();
        f.o = neg_inf();
    }
    const size_t srow = (size_t)P * 2;       // doubles per frame of alpha / beta
    const size_t urow = (size_t)P * 3;       // doubles per frame of units
    double *out = lat_n + (size_t)u * 2;
    const double *in = units_n + (size_t)u * 3;
    front_store(out + (size_t)(BETA ? Tn : 0) * srow, f);
    // the row a step stores to, the same for all lanes, walked frame by frame
    const unsigned out_lane = (unsigned)u * 2u * (unsigned)sizeof(double);
    const unsigned in_lane = (unsigned)u * 3u * (unsigned)sizeof(double);
    const unsigned out_step = (unsigned)(srow * sizeof(double));     // bytes per frame
    const unsigned in_step = (unsigned)(urow * sizeof(double));
    char *out_row = reinterpret_cast<char *>(lat_n) + (size_t)(BETA ? Tn - 1 : 1) * srow * sizeof(double);
    const int edge_lane = BETA ? 0 : 63;          // lane whose value crosses the boundary

    if (Tn > 0) {
        Chunk a, b;
        const int dir = BETA ? -1 : 1;
        const int t_start = BETA ? Tn - 1 : 0;
        chunk_load(a, in, urow, Tn, t_start, dir);
        // The relay slots of a chunk are requested one chunk before they are used,
        // into two register sets used in turn (like the units): the set a chunk
        // reads was requested while the previous chunk was swept, and is free to
        // receive the request for the chunk after next as soon as it has been read.
        unsigned long long ahead_a[R], ahead_b[R];
#pragma unroll
        for (int r = 0; r < R; ++r) ahead_a[r] = ahead_b[r] = kEmptyBits;
        if (HAS_IN) slots_request(slots_in, 0, ahead_a);
        // The input is lost: a wait has run out, or the producer says that it lost
        // its own (lost_from = the first step without input).  The sweep goes on to
        // its end without waiting again and without handing anything over (leaving
        // the loop early, or a branch around a chunk, costs the common path 15 %:
        // the compiler then waits for every load in flight where the paths join);
        // what it has computed since is overwritten afterwards.
        bool lost = false;
        int lost_from = 0;
        // one chunk: steps s0 .. s0+cnt-1 with the units in `c` and the slots in
        // `have`; the slots of the next chunk are requested into `next`
        auto run_chunk = [&](const Chunk &c, unsigned long long (&have)[R],
                             unsigned long long (&next)[R], int s0, int cnt, bool full) {
            double mail[R], mine[R];
#pragma unroll
            for (int r = 0; r < R; ++r) mail[r] = neg_inf();
            if (HAS_IN) {
                slots_request(slots_in, min(s0 + R, T), next);
                // `have` was requested a chunk ago; repeat the request until the
                // producer has got this far, max_spins times at most.  The first
                // look is kept out of the polling loop: a loop header that is also
                // reached from the re-request would make the compiler wait for
                // every load in flight here, the prefetched units included.
                unsigned state = slots_state(have, cnt);
                if (state == 0 && max_spins > 0 && !lost) {
                    int spins = 0;
                    do {
                        __builtin_amdgcn_s_sleep(2);
                        slots_request(slots_in, s0, have);
                        state = slots_state(have, cnt);
                    } while (state == 0 && ++spins < max_spins);
                }
                if (state <= 1 && !lost) lost = true, lost_from = s0;
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (full || r < cnt) mail[r] = __longlong_as_double((long long)have[r]);
            }
            // the chunk's rows of the lattice, lowest address first
            const int rows_here = full ? R : cnt;
            const __amdgpu_buffer_rsrc_t rows =
                rows_from(BETA ? out_row - (size_t)(rows_here - 1) * out_step : out_row);
            unsigned at = BETA ? (unsigned)(rows_here - 1) * out_step : 0u;
#pragma unroll
            for (int r = 0; r < R; ++r) {
                mine[r] = neg_inf();
                if (full || r < cnt) {
                    if (BETA) beta_step(f, c.lp[r], skip, o_mask, mail[r], mine[r]);
                    else alpha_step(f, c.lp[r], skip, mail[r], mine[r]);
                    front_store_at(rows, out_lane, at, f);
                    at = BETA ? at - out_step : at + out_step;
                }
            }
            out_row = BETA ? out_row - (size_t)rows_here * out_step : out_row + (size_t)rows_here * out_step;
            if (slots_out && !lost && lane == edge_lane) {
#pragma unroll
                for (int r = 0; r < R; ++r)
                    if (full || r < cnt) slot_put(slots_out + s0 + r, mine[r]);
            }
        };
        int s0 = 0;
        // while the chunk after next lies inside the sample, its rows need no clamp
        if (3 * R <= Tn) {
            const char *frame = reinterpret_cast<const char *>(units_n) +
                                (size_t)(t_start + dir * R) * urow * sizeof(double);
            do {
                chunk_load_walk<BETA>(b, frame, in_lane, in_step);
                run_chunk(a, ahead_a, ahead_b, s0, R, true);
                chunk_load_walk<BETA>(a, frame, in_lane, in_step);
                run_chunk(b, ahead_b, ahead_a, s0 + R, R, true);
                s0 += 2 * R;
            } while (s0 + 3 * R <= Tn);
        }
        while (s0 + 2 * R <= Tn) {
            chunk_load(b, in, urow, Tn, t_start + dir * (s0 + R), dir);
            run_chunk(a, ahead_a, ahead_b, s0, R, true);
            chunk_load(a, in, urow, Tn, t_start + dir * (s0 + 2 * R), dir);
            run_chunk(b, ahead_b, ahead_a, s0 + R, R, true);
            s0 += 2 * R;
        }
        // fewer than 2R frames left
        chunk_load(b, in, urow, Tn, t_start + dir * (s0 + R), dir);
        const int rest = Tn - s0;
        if (rest > 0) run_chunk(a, ahead_a, ahead_b, s0, min(rest, R), false);
        if (rest > R) run_chunk(b, ahead_b, ahead_a, s0 + R, rest - R, false);
        if (lost) {
            // Nothing plausible may come out of this lattice: the rows from the
            // first step without input on are NaN (so is every gradient computed
            // from them, and the cost if this is the end of the beta chain), and
            // the consumer, which has been waiting since, is told.
            f.e = f.o = __longlong_as_double(0x7ff8000000000000LL);
            // (the device's status word tells this NaN from one that came in with the inputs)
            if (status && lane == 0) atomicOr(status, kStatusLostHandOver);
            for (int s = lost_from; s < Tn; ++s)
                front_store(out + (size_t)(BETA ? Tn - 1 - s : s + 1) * srow, f);
            if (slots_out && lane == edge_lane)
                for (int s = lost_from; s < Tn; ++s)
                    __hip_atomic_store(slots_out + s, kLostBits, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    // cost = -beta(0, state 0) in natural-log units (csrc/binding.cpp:86)
    if (BETA && u == 0) *cost_n = (float)(-f.e * kLn2);
}

// One wavefront per workgroup.  Workgroup index = link * chains_pad + chain with
// chain = n * dirs + d (d = 0: beta, which also produces the cost; d = 1:
// alpha), chains_pad = the number of chains rounded up to a multiple of 8 (the
// surplus workgroups exit), link = position in the chain of W workgroups, first
// producer first: alpha starts at contexts 0..63, beta at the last 64.
static __device__ __forceinline__ void lattice_block(const double *__restrict__ units,
                                              const int *__restrict__ ys,
                                              const int *__restrict__ lx,
                                              const int *__restrict__ ly,
                                              double *__restrict__ alphas,
                                              double *__restrict__ betas,
                                              float *__restrict__ costs,
                                              unsigned long long *__restrict__ relay, int N, int T,
                                              int U, int W, int dirs, int chains_pad,
                                              const CostReduce &red, int max_spins,
                                              unsigned *status) {
    const int chain = blockIdx.x % chains_pad, link = blockIdx.x / chains_pad;
    if (chain >= N * dirs) return;
    const int n = chain / dirs;
    const bool beta = (chain % dirs) == 0;
    const int wave = beta ? W - 1 - link : link;
    const int P = 64 * W;
    // lengths outside the allocation are clamped: nothing is ever read or
    // written beyond (T, U), whatever the length tensors hold
    const int Tn = min(max(lx[n], 0), T);
    const int Un = min(max(ly[n], 0), U);
    // 64 contexts that lie entirely beyond this sample's last context hold no
    // state that anything reads, and pass nothing on: -inf flows in from them
    if (wave * 64 > Un) return;
    const double *units_n = units + (size_t)n * T * P * 3;
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * P * 2;
    // boundary b lies between contexts 64b+63 and 64b+64; its slots for one
    // direction of one sample: relay[((n*2 + direction)*(W-1) + b) * (T + kRelayPad) ...]
    const size_t TS = (size_t)T + kRelayPad;
    unsigned long long *slots_n =
        relay ? relay + ((size_t)n * 2 + (beta ? 0 : 1)) * (size_t)(W - 1) * TS : nullptr;
    if (!beta) {
        const unsigned long long *in = wave > 0 ? slots_n + (size_t)(wave - 1) * TS : nullptr;
        unsigned long long *out = (wave + 1) * 64 <= Un ? slots_n + (size_t)wave * TS : nullptr;
        if (in) sweep<false, true>(units_n, y, Tn, Un, T, P, wave, alphas + (size_t)n * lat, nullptr, in, out, max_spins, status);
        else sweep<false, false>(units_n, y, Tn, Un, T, P, wave, alphas + (size_t)n * lat, nullptr, in, out, max_spins, status);
        return;
    }
    {
        const unsigned long long *in = (wave + 1) * 64 <= Un ? slots_n + (size_t)wave * TS : nullptr;
        unsigned long long *out = wave > 0 ? slots_n + (size_t)(wave - 1) * TS : nullptr;
        if (in) sweep<true, true>(units_n, y, Tn, Un, T, P, wave, betas + (size_t)n * lat, costs + n, in, out, max_spins, status);
        else sweep<true, false>(units_n, y, Tn, Un, T, P, wave, betas + (size_t)n * lat, costs + n, in, out, max_spins, status);
    }
    if (wave != 0) return;
    // thread 0 (context 0) has just written costs[n]
    cost_reduce_tail(red, costs, lx, n, N, threadIdx.x);
}

};

__global__ __launch_bounds__(64) void lattice_kernel(const double *__restrict__ units,
                                                     const int *__restrict__ ys,
                                                     const int *__restrict__ lx,
                                                     const int *__restrict__ ly,
                                                     double *__restrict__ alphas,
                                                     double *__restrict__ betas,
                                                     float *__restrict__ costs,
                                                     unsigned long long *__restrict__ relay, int N,
                                                     int T, int U, int W, int dirs, int chains_pad,
                                                     const CostReduce red, int max_spins,
                                                     unsigned *__restrict__ status,
                                                     const unsigned *__restrict__ only_if) {
    if (only_if) {
        // the fall-back of the linear lattices: nothing to do while their flag is down
        if (*only_if == 0u) return;
        if (blockIdx.x == 0 && threadIdx.x == 0 && status) atomicOr(status, kStatusLinearFellBack);
    }
    Chunked<12>::lattice_block(units, ys, lx, ly, alphas, betas, costs, relay, N, T, U, W, dirs,
                               chains_pad, red, max_spins, status);
}

// The same sweeps with a memory clear riding along: workgroups of 256 threads,
// of which the first lattice_blocks are the sweeps (their first wavefront; the
// other three retire at once) and every later one stores 256 zero vectors of
// 16 bytes and retires.  The sweeps wait on a chain of dependent arithmetic
// and leave the memory system idle; the clear is pure write traffic.
typedef float v4f_fill __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void lattice_fill_kernel(
    const double *__restrict__ units, const int *__restrict__ ys, const int *__restrict__ lx,
    const int *__restrict__ ly, double *__restrict__ alphas, double *__restrict__ betas,
    float *__restrict__ costs, unsigned long long *__restrict__ relay, int N, int T, int U, int W,
    int dirs, int chains_pad, const CostReduce red, int max_spins, unsigned *__restrict__ status,
    v4f_fill *__restrict__ fill, size_t n4, unsigned lattice_blocks) {
    if (blockIdx.x >= lattice_blocks) {
        const size_t i = (size_t)(blockIdx.x - lattice_blocks) * 256 + threadIdx.x;
        if (i < n4) fill[i] = v4f_fill{0.0f, 0.0f, 0.0f, 0.0f};
        return;
    }
    if (threadIdx.x >= 64) return;
    Chunked<8>::lattice_block(units, ys, lx, ly, alphas, betas, costs, relay, N, T, U, W, dirs,
                              chains_pad, red, max_spins, status);
}

}  // namespace

namespace {
std::atomic<int> g_wait_limit{kMaxSpins};
}

int lattice_wait_limit_now() { return g_wait_limit.load(std::memory_order_relaxed); }

int lattice_wait_limit(int spins) {
    return g_wait_limit.exchange(spins < 0 ? kMaxSpins : spins, std::memory_order_relaxed);
}

size_t lattice_relay_slots(int N, int T, int U) {
    const int W = (U + 1 + 63) / 64;
    return (size_t)N * 2 * (size_t)(W - 1) * ((size_t)T + kRelayPad);
}

hipError_t launch_lattice(const LatticeArgs &a, hipStream_t stream, const unsigned *only_if) {
    if (a.N == 0) return hipSuccess;
    const int W = (a.U + 1 + 63) / 64;
    const size_t slots = lattice_relay_slots(a.N, a.T, a.U);
    unsigned long long *relay = reinterpret_cast<unsigned long long *>(a.relay);
    if (slots > 0 && a.relay_is_clear) {
        if (!relay) return hipErrorInvalidValue;
    } else if (slots > 0) {
        if (!relay) return hipErrorInvalidValue;
        const size_t blocks = (slots + 255) / 256;
        if (blocks > 0x7fffffffUL) return hipErrorInvalidValue;
        TIMED_LAUNCH(relay_clear_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, relay,
                     slots);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    } else {
        relay = nullptr;
    }
    const int max_spins = g_wait_limit.load(std::memory_order_relaxed);
    // (only chains can lose a hand-over; a fall-back reports itself)
    unsigned *status = (W > 1 || only_if) ? device_status_word() : nullptr;
    const int dirs = a.beta_only ? 1 : 2;
    const long chains = (long)a.N * dirs;
    const long chains_pad = (chains + 7) / 8 * 8;
    if (chains_pad * W > 0x7fffffffL) return hipErrorInvalidValue;
    if (a.fill.n4 > 0) {
        if (only_if) return hipErrorInvalidValue;
        const size_t blocks = (size_t)(chains_pad * W) + (a.fill.n4 + 255) / 256;
        if (blocks > 0x7fffffffUL) return hipErrorInvalidValue;
        TIMED_LAUNCH(lattice_fill_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, a.units,
                     a.ys, a.lx, a.ly, a.alphas, a.betas, a.costs, relay, a.N, a.T, a.U, W, dirs,
                     (int)chains_pad, a.reduce, max_spins, status, static_cast<v4f_fill *>(a.fill.p), a.fill.n4,
                     (unsigned)(chains_pad * W));
        return hipGetLastError();
    }
    TIMED_LAUNCH(lattice_kernel, dim3((unsigned)(chains_pad * W)), dim3(64), 0, stream, a.units,
                 a.ys, a.lx, a.ly, a.alphas, a.betas, a.costs, relay, a.N, a.T, a.U, W, dirs,
                 (int)chains_pad, a.reduce, max_spins, status, only_if);
    return hipGetLastError();
}

}  // namespace wctct
