// Alpha / beta lattices of the CTC-Transducer loss on gfx950.
//
// The sweep is time-synchronous: all states of frame t are updated from frame
// t-1 (alpha) or t+1 (beta); states of one frame do not depend on each other,
// so a step needs no barrier and no atomics — only one value from the
// neighbouring context.  Every lane owns one context u and its state pair
//     o = state 2u-1 (inside label y[u-1])      e = state 2u (blank after u labels)
// in registers.  A lattice with up to 64 contexts is one wavefront; the value
// of the neighbouring context moves with single-lane DPP shifts.  A wider
// lattice (up to 512 contexts) is W = ceil((U+1)/64) wavefronts of one
// workgroup, each sweeping its own 64 contexts: the one value that crosses a
// wavefront boundary per step goes through a small LDS ring, published and
// consumed a chunk of R frames at a time, so the wavefronts run skewed by one
// chunk instead of meeting at a barrier every frame.
//
// Values are log2 of the path mass, held in double; the exponentials and
// logarithms of the semiring sum run on the fp32 transcendental unit (see
// device_utils.h).  Units for the next chunk of R frames are prefetched into
// registers while the current chunk is swept.
//
// Math restated from ref_ctct.py:6-74 of the reference (alpha :6-37, beta
// :40-74); this kernel replaces k_warp_alphas / k_warp_betas
// (csrc/gather.cu:36-291) and their global-memory spin-lock row pipeline.
#include "device_utils.h"
#include "launch.h"

namespace wctct {

namespace {

constexpr int R = 8;          // frames per chunk (prefetch depth and hand-over granularity)
constexpr int kRing = 4 * R;  // ring slots per wavefront boundary
constexpr int kMaxSpins = 1 << 22;

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

struct Chunk {
    double lp[R][3];
};

// Units of frames t_first + dir*r, r in [0,R); the frame index is clamped into
// [0, Tn-1] so that a prefetch past the end re-reads a valid row (its values
// are then not used).
__device__ __forceinline__ void chunk_load(Chunk &c, const double *units_lane, size_t row, int Tn,
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

// ---- hand-over between the wavefronts of one lattice -------------------------
// Boundary b sits between wavefront b and b+1.  done[b] counts the steps whose
// value the producer has put into ring[b]; taken[b] counts the steps the
// consumer has read.  Both only grow; a wavefront spins (with a bound, so that
// no input can hang the GPU) until the counter it needs has advanced.
// The fences name the LDS address space only: a plain workgroup-scope fence
// would also wait for the global-memory prefetch in flight, which is exactly
// what the chunked sweep must not do.
template <int W>
struct Relay {
    double ring[W > 1 ? W - 1 : 1][kRing];
    int done[W > 1 ? W - 1 : 1];
    int taken[W > 1 ? W - 1 : 1];
};

// Returns the value seen (>= target unless the spin bound was hit).
__device__ __forceinline__ int wait_until(int *counter, int target) {
    int seen = 0;
    for (int spins = 0; spins < kMaxSpins; ++spins) {
        seen = __builtin_amdgcn_readfirstlane(
            __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP));
        if (seen >= target) break;
        __builtin_amdgcn_s_sleep(1);
    }
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return seen;
}

// Consumer side of a hand-over: the counter and the R ring slots of a chunk
// are requested in one batch (LDS serves a wavefront's requests in order, so
// slots read after a counter that already shows the chunk are the chunk's
// values).  peek() only issues the requests and returns the counter as read;
// nothing waits for them until the values are used, so a peek at the chunk
// after the current one costs the sweep no LDS round trip when the producer is
// already that far.
__device__ __forceinline__ int peek(int *counter, const double *ring, int s0, double (&mail)[R]) {
    const int seen = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __atomic_signal_fence(__ATOMIC_SEQ_CST);   // the compiler keeps the order of the requests
#pragma unroll
    for (int r = 0; r < R; ++r)
        mail[r] = __hip_atomic_load(ring + (s0 + r) % kRing, __ATOMIC_RELAXED,
                                    __HIP_MEMORY_SCOPE_WORKGROUP);
    return seen;
}

// Repeats the batch until the counter shows the chunk (with a bound).
__device__ __forceinline__ void wait_and_take(int *counter, int target, const double *ring,
                                              int s0, double (&mail)[R]) {
    for (int spins = 0; spins < kMaxSpins; ++spins) {
        const int seen = peek(counter, ring, s0, mail);
        if (__builtin_amdgcn_readfirstlane(seen) >= target) break;
        __builtin_amdgcn_s_sleep(1);
    }
}

__device__ __forceinline__ void publish(int *counter, int value) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    if ((threadIdx.x & 63) == 0)
        __hip_atomic_store(counter, value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
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
// previous wavefront, or -inf); out = what this lane sends to context u+1.
__device__ __forceinline__ void alpha_step(Front &f, const double *lp, bool skip_next, double ext,
                                           double &out) {
    const double both = lse2(f.e, f.o);
    out = (skip_next ? both : f.e) + lp[2];
    const double recv = wave_shift_up(out, ext);
    const double no = lse2(f.o + lp[1], recv);
    f.e = both + lp[0];
    f.o = no;
}

// ---- beta ----------------------------------------------------------------
// beta(t, 2u)   = beta(t+1,2u) + LP(t,u,0)  (+) [u<U] beta(t+1,2u+1) + LP(t,u,2)
// beta(t, 2u-1) = beta(t+1,2u-1) + LP(t,u,1) (+) beta(t+1,2u) + LP(t,u,0)
//              (+) [u<U, y[u-1] != y[u]] beta(t+1,2u+1) + LP(t,u,2)
// The last two terms of the second line are beta(t,2u) itself when the skip
// arc exists and its first term alone when it does not.
// skip: y[u-1] != y[u] with 1 <= u < Un.  o_mask is 0 for contexts that have a
// state 2u-1 (1 <= u <= Un), else -inf.  ext = beta(t+1, 2u+1) for lane 63
// (from the next wavefront, or -inf); out = this lane's beta(t+1, 2u-1), which
// context u-1 needs.
__device__ __forceinline__ void beta_step(Front &f, const double *lp, bool skip, double o_mask,
                                          double ext, double &out) {
    out = f.o;
    const double nb = wave_shift_down(f.o, ext);
    const double nxt = nb + lp[2];
    const double stay_e = f.e + lp[0];
    const double ne = lse2(stay_e, nxt);
    const double no = lse2(f.o + lp[1], skip ? ne : stay_e);
    f.e = ne;
    f.o = no + o_mask;
}

// One direction of one lattice, swept by the W wavefronts of this workgroup.
// BETA selects the direction; step s handles frame t = s (alpha) or Tn-1-s
// (beta) and stores the front of frame t+1 (alpha) or t (beta).
template <int W, bool BETA>
__device__ void sweep(const double *units_n, const int *y, int Tn, int Un, double *lat_n,
                      float *cost_n, Relay<W> &relay) {
    constexpr int P = 64 * W;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
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

    // which neighbour feeds this wavefront, and which one it feeds
    const bool consumes = W > 1 && (BETA ? wave < W - 1 : wave > 0);
    const bool produces = W > 1 && (BETA ? wave > 0 : wave < W - 1);
    const int b_in = BETA ? wave : wave - 1;      // boundary this wavefront reads
    const int b_out = BETA ? wave - 1 : wave;     // boundary this wavefront writes
    const int edge_lane = BETA ? 0 : 63;          // lane whose value crosses the boundary

    if (Tn > 0) {
        Chunk a, b;
        const int dir = BETA ? -1 : 1;
        const int t_start = BETA ? Tn - 1 : 0;
        chunk_load(a, in, urow, Tn, t_start, dir);
        int taken_seen = 0;
        int ahead_seen = 0;        // counter as read by the last peek ahead
        double ahead[R];           // ... and the slots of the chunk it looked at
#pragma unroll
        for (int r = 0; r < R; ++r) ahead[r] = neg_inf();
        // one chunk: steps s0 .. s0+cnt-1 with the units in `c`
        auto run_chunk = [&](const Chunk &c, int s0, int cnt, bool full) {
            double mail[R], mine[R];
#pragma unroll
            for (int r = 0; r < R; ++r) mail[r] = neg_inf();
            if (consumes) {
                // the peek of the previous chunk looked at exactly this chunk
                if (__builtin_amdgcn_readfirstlane(ahead_seen) < s0 + cnt)
                    wait_and_take(&relay.done[b_in], s0 + cnt, relay.ring[b_in], s0, ahead);
#pragma unroll
                for (int r = 0; r < R; ++r) mail[r] = ahead[r];
                publish(&relay.taken[b_in], s0 + cnt);
                ahead_seen = peek(&relay.done[b_in], relay.ring[b_in], s0 + cnt, ahead);
            }
#pragma unroll
            for (int r = 0; r < R; ++r) {
                mine[r] = neg_inf();
                if (full || r < cnt) {
                    const int s = s0 + r;
                    if (BETA) {
                        beta_step(f, c.lp[r], skip, o_mask, mail[r], mine[r]);
                        front_store(out + (size_t)(Tn - 1 - s) * srow, f);
                    } else {
                        alpha_step(f, c.lp[r], skip, mail[r], mine[r]);
                        front_store(out + (size_t)(s + 1) * srow, f);
                    }
                }
            }
            if (produces) {
                // the ring is four chunks deep: the consumer's progress is looked
                // up again only when the last value seen no longer covers this chunk
                if (taken_seen < s0 + cnt - kRing)
                    taken_seen = wait_until(&relay.taken[b_out], s0 + cnt - kRing);
                if (lane == edge_lane) {
#pragma unroll
                    for (int r = 0; r < R; ++r)
                        if (full || r < cnt) relay.ring[b_out][(s0 + r) % kRing] = mine[r];
                }
                publish(&relay.done[b_out], s0 + cnt);
            }
        };
        int s0 = 0;
        while (s0 + 2 * R <= Tn) {
            chunk_load(b, in, urow, Tn, t_start + dir * (s0 + R), dir);
            run_chunk(a, s0, R, true);
            chunk_load(a, in, urow, Tn, t_start + dir * (s0 + 2 * R), dir);
            run_chunk(b, s0 + R, R, true);
            s0 += 2 * R;
        }
        // fewer than 2R frames left
        chunk_load(b, in, urow, Tn, t_start + dir * (s0 + R), dir);
        const int rest = Tn - s0;
        if (rest > 0) run_chunk(a, s0, min(rest, R), false);
        if (rest > R) run_chunk(b, s0 + R, rest - R, false);
    }
    // cost = -beta(0, state 0) in natural-log units (csrc/binding.cpp:86)
    if (BETA && u == 0) *cost_n = (float)(-f.e * kLn2);
}

// grid = (N, beta_only ? 1 : 2), block = 64*W.  blockIdx.y == 0 runs beta (it
// also produces the cost), blockIdx.y == 1 runs alpha.
template <int W>
__global__ __launch_bounds__(64 * W) void lattice_kernel(const double *__restrict__ units,
                                                         const int *__restrict__ ys,
                                                         const int *__restrict__ lx,
                                                         const int *__restrict__ ly,
                                                         double *__restrict__ alphas,
                                                         double *__restrict__ betas,
                                                         float *__restrict__ costs, int T, int U,
                                                         const CostReduce red) {
    __shared__ Relay<W> relay;
    const int n = blockIdx.x;
    constexpr int P = 64 * W;
    if (W > 1) {
        if (threadIdx.x < W - 1) {
            relay.done[threadIdx.x] = 0;
            relay.taken[threadIdx.x] = 0;
        }
        __syncthreads();
    }
    // lengths outside the allocation are clamped: nothing is ever read or
    // written beyond (T, U), whatever the length tensors hold
    const int Tn = min(max(lx[n], 0), T);
    const int Un = min(max(ly[n], 0), U);
    const double *units_n = units + (size_t)n * T * P * 3;
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * P * 2;
    if (blockIdx.y != 0) {
        sweep<W, false>(units_n, y, Tn, Un, alphas + (size_t)n * lat, nullptr, relay);
        return;
    }
    sweep<W, true>(units_n, y, Tn, Un, betas + (size_t)n * lat, costs + n, relay);
    if (threadIdx.x >= 64) return;
    // thread 0 (context 0) has just written costs[n]
    if (red.average_frames && threadIdx.x == 0) costs[n] /= (float)lx[n];
    if (red.reduced == nullptr) return;
    // Reduction over the batch (warp_ctct/__init__.py:142-147 of the reference)
    // by the workgroup that finishes last: every workgroup publishes its cost
    // (release fence), then counts itself; the one that sees N-1 earlier
    // arrivals reads all N costs (acquire fence) and adds them in a fixed
    // order, so the result does not depend on the order of arrival.
    const int N = gridDim.x;
    int last = 0;
    if (threadIdx.x == 0) {
        __threadfence();
        last = (atomicAdd(red.counter, 1u) == (unsigned)(N - 1)) ? 1 : 0;
    }
    last = __shfl(last, 0, 64);
    if (!last) return;
    __threadfence();
    float s = 0.0f;
    for (int i = threadIdx.x; i < N; i += 64)
        s += __hip_atomic_load(costs + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) s += __shfl_xor(s, off, 64);
    if (threadIdx.x == 0) *red.reduced = (red.mode == 2) ? s / (float)N : s;
}

template <int W>
hipError_t launch_lattice_w(const LatticeArgs &a, hipStream_t stream) {
    dim3 grid(a.N, a.beta_only ? 1 : 2);
    TIMED_LAUNCH((lattice_kernel<W>), grid, dim3(64 * W), 0, stream, a.units, a.ys, a.lx,
                       a.ly, a.alphas, a.betas, a.costs, a.T, a.U, a.reduce);
    return hipGetLastError();
}

}  // namespace

int lattice_max_contexts() { return 64 * 8; }

hipError_t launch_lattice(const LatticeArgs &a, hipStream_t stream) {
    const int W = (a.U + 1 + 63) / 64;
    switch (W) {
        case 1: return launch_lattice_w<1>(a, stream);
        case 2: return launch_lattice_w<2>(a, stream);
        case 3: return launch_lattice_w<3>(a, stream);
        case 4: return launch_lattice_w<4>(a, stream);
        case 5: return launch_lattice_w<5>(a, stream);
        case 6: return launch_lattice_w<6>(a, stream);
        case 7: return launch_lattice_w<7>(a, stream);
        case 8: return launch_lattice_w<8>(a, stream);
        default: return hipErrorInvalidValue;
    }
}

}  // namespace wctct
