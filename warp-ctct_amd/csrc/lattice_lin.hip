// Alpha / beta lattices of the log-add joiner in the LINEAR domain: the fast
// form of lattice.hip's sweeps, used where its result is verified afterwards.
//
// States are path masses (not their logarithms), held in double relative to a
// power of two that the contexts of a wavefront share: mass = value * 2^S.
// A frame is then three multiplications, three multiply-adds or additions and
// the two DPP moves of the neighbouring context's value, against two semiring
// sums (exponential, logarithm, conversions) per state in the log form: a lone
// wavefront pays for every instruction, and a frame costs less than half.
// Every R frames the largest state of the wavefront is brought back to [0.5, 1)
// and S moves by its exponent; the rows a chunk stores are relative to the S of
// that chunk, which is recorded per (sample, direction, wavefront, chunk) for
// the kernel that reads the lattices.
//
// What the linear form cannot do is keep a state that lies more than ~2^-1000
// below the largest state of its wavefront: it becomes 0.  That is harmless
// unless the alignments that carry the posterior mass pass through such a
// state.  The kernel that forms the gradients from these lattices therefore
// checks, per frame, that the posteriors it hands out add up to 1 (every
// alignment consumes exactly one unit per frame), and that no unit is so large
// that R frames could overflow; if any check fails (or a value is not finite, or a hand-over was lost)
// it raises a flag, and the log-domain kernels of lattice.hip, which follow
// in the same stream and return at once while the flag is down, compute the
// batch again.
//
// Chains of workgroups: a wavefront holds 62 contexts, in its lanes 1..62.  Lane
// 0 (alpha) or lane 63 (beta) plays the context next door, which another
// wavefront computes: its state is the constant 2^(S_sender - S_own) and its
// units come from a column of the units array that belongs to no context and
// that the sender fills, frame by frame, with the value it hands over.  The
// recursion of the real lanes then needs nothing extra: the value arrives
// through the same loads and the same DPP move as a neighbour's inside the
// wavefront.  (For that the beta sweep sends its value already multiplied by
// the receiver's unit, which every lane reads from the cell of the context
// below its own.)  The sender's S of a chunk travels in a spare field of the
// chunk's first cell.  Nothing tells the receiver in advance that a value has
// arrived: a field that has not been written holds a NaN pattern, the NaN
// reaches the receiver's first real context within the chunk, and the receiver
// looks at that context once per chunk; if it finds a NaN it waits for the
// chunk's fields (bounded, as in lattice.hip), fetches them again and repeats
// the chunk from the states it had kept.  A NaN moves one lane per frame, so
// what the wavefront itself hands over from the other end of its lanes was not
// touched by it.  The first fetch of a field is an ordinary load, with the rest
// of its row: if it finds an older copy of the line in a cache, that copy holds
// the NaN pattern, never an older value, because a field changes once per launch
// (the kernel that gathers the units writes the pattern, the sender the value);
// the repeated fetch and the sender's stores go past the caches.
//
// Math restated from ref_ctct.py:6-74 of the reference, as in lattice.hip.
#include <algorithm>

#include "cost_reduce.h"
#include "device_utils.h"
#include "launch.h"

namespace wctct {

namespace {

constexpr int R = kLinChunk;
constexpr unsigned long long kEmptyBits = kRelayEmpty;
constexpr unsigned long long kLostBits = kEmptyBits ^ (1ULL << 32);
constexpr unsigned kEmptyHigh = (unsigned)(kEmptyBits >> 32);
constexpr unsigned kLostHigh = (unsigned)(kLostBits >> 32);
// a sender's S travels as S + 2^30: never 0, which stands for "not there yet"
constexpr double kScaleBias = 1073741824.0;
constexpr unsigned kCellBytes = kLinUnit * sizeof(double);
constexpr int kAgentScope = 16;   // buffer access past the caches that other workgroups do not see (sc1)

struct ChunkL {
    double lp[R][3];   // blank, label, and what the sweep multiplies the value it sends with
};

typedef unsigned v4u_lin __attribute__((ext_vector_type(4)));
typedef unsigned v2u_lin __attribute__((ext_vector_type(2)));

__device__ __forceinline__ double as_double(v2u_lin x) { return __hiloint2double((int)x[1], (int)x[0]); }
__device__ __forceinline__ v2u_lin as_words(double x) {
    v2u_lin w;
    w[0] = (unsigned)__double2loint(x), w[1] = (unsigned)__double2hiint(x);
    return w;
}

// A row of a lattice holds, per column, the HIGH words of the pair {o, e}: sign,
// exponent and 20 bits of mantissa, 8 bytes per lane.  The kernel that reads the
// rows forms posteriors from them, which tolerate a relative error of 1e-6 (the
// gradients are float32, compared at 1e-4), and takes the middle of what the
// missing low word can have been (lin_state in unit_grad.h); the sweeps carry
// the states as doubles in registers, and the cost comes from those.  Half the
// traffic of the rows, written here and read back by that kernel: what bounds
// the sweeps of more than a few dozen lattices.
__device__ __forceinline__ void pair_store(unsigned *dst, double o, double e) {
    *reinterpret_cast<uint2 *>(dst) = make_uint2((unsigned)__double2hiint(o), (unsigned)__double2hiint(e));
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

// The double that lane `from` holds, as a scalar.
template <int from>
static __device__ __forceinline__ double lane_value(double x) {
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(x), from),
                            __builtin_amdgcn_readlane(__double2loint(x), from));
}

// Byte offset, inside a cell of units, of the next label's unit: the third
// factor of the alpha sweep, and the field of a column in between that takes
// the value handed over.  The beta sweep's third factor is the same field of the
// cell of the context BELOW the lane's own (what it sends is multiplied with the
// receiver's unit before it is sent).
constexpr unsigned kNextField = 16u;
// ... and of the field that carries the sender's S in the column it fills: one
// that the lane playing the sender multiplies with a state that is always 0.
template <bool BETA>
constexpr unsigned scale_field() { return BETA ? 0u : 8u; }

// One row of units for this lane: `at` is the row's byte offset in the sample's
// units, lane_bytes the lane's own cell in a row, third_bytes its third factor.
static __device__ __forceinline__ void row_load_lin(double (&lp)[3], __amdgpu_buffer_rsrc_t units,
                                                    unsigned lane_bytes, unsigned third_bytes, unsigned at) {
    const v4u_lin w = __builtin_amdgcn_raw_buffer_load_b128(units, lane_bytes, at, 0);
    const v2u_lin x = __builtin_amdgcn_raw_buffer_load_b64(units, third_bytes, at, 0);
    lp[0] = __hiloint2double((int)w[1], (int)w[0]);
    lp[1] = __hiloint2double((int)w[3], (int)w[2]);
    lp[2] = as_double(x);
}

// The units of R frames from t_first on in sweep direction, frames clamped to the sample.
template <bool BETA>
static __device__ __forceinline__ void chunk_load_lin(ChunkL &c, __amdgpu_buffer_rsrc_t units,
                                                      unsigned lane_bytes, unsigned third_bytes,
                                                      unsigned step, int Tn, int t_first) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = min(max(t_first + (BETA ? -r : r), 0), Tn - 1);
        row_load_lin(c.lp[r], units, lane_bytes, third_bytes, (unsigned)t * step);
    }
}

// The units of R frames that all exist: `lowest` is the address of the chunk's
// row with the lowest frame index, off[r] the byte offset of step r's row from
// it (the same for every chunk, so no address arithmetic per frame).
static __device__ __forceinline__ void chunk_load_whole_lin(ChunkL &c, const char *lowest,
                                                            const unsigned (&off)[R], unsigned lane_bytes,
                                                            unsigned third_bytes) {
    const __amdgpu_buffer_rsrc_t rows =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(lowest), 0, 0xffffffffu, 0x00020000);
#pragma unroll
    for (int r = 0; r < R; ++r) row_load_lin(c.lp[r], rows, lane_bytes, third_bytes, off[r]);
}

// Only the fields another wavefront fills (the third factor of every frame and
// the scale beside the first), fetched again past the caches.
template <bool BETA>
static __device__ __forceinline__ void chunk_reload_mail_lin(ChunkL &c, __amdgpu_buffer_rsrc_t units,
                                                             unsigned lane_bytes, unsigned third_bytes,
                                                             unsigned step, int Tn, int t_first) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const int t = min(max(t_first + (BETA ? -r : r), 0), Tn - 1);
        c.lp[r][2] = as_double(
            __builtin_amdgcn_raw_buffer_load_b64(units, third_bytes, (unsigned)t * step, kAgentScope));
    }
    const int t = min(max(t_first, 0), Tn - 1);
    c.lp[0][BETA ? 0 : 1] = as_double(__builtin_amdgcn_raw_buffer_load_b64(
        units, lane_bytes + scale_field<BETA>(), (unsigned)t * step, kAgentScope));
}

// What lane `ghost` holds of a chunk's hand-over.  0: a value of the first cnt
// frames or the scale is not there yet; 1: all are there and one says "lost";
// else all are values.
template <bool BETA, int ghost>
static __device__ __forceinline__ unsigned chunk_mail_state_lin(const ChunkL &c, int cnt) {
    bool empty = false, gone = false;
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const unsigned hi = (unsigned)__double2hiint(c.lp[r][2]);
        empty = empty || (r < cnt && hi == kEmptyHigh);
        gone = gone || (r < cnt && hi == kLostHigh);
    }
    const double s = c.lp[0][BETA ? 0 : 1];
    empty = empty || s == 0.0;
    gone = gone || (unsigned)__double2hiint(s) == kLostHigh;
    if (__ballot(empty) & (1ULL << ghost)) return 0u;
    if (__ballot(gone) & (1ULL << ghost)) return 1u;
    return 2u;
}

// Lane l receives x of lane l-1 / l+1; the lane at the end receives 0.
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

// One direction of the contexts [62*wave, 62*wave + 62) of one lattice.  Step s
// handles frame t = s (alpha) or Tn-1-s (beta) and stores the front of frame
// t+1 (alpha) or t (beta), as in lattice.hip.  scales[0] belongs to the initial
// row, scales[1 + k] to the rows that chunk k stores.
// HAS_IN: a wavefront fills this one's column of hand-overs; has_out: this one
// fills the next one's.
template <bool BETA, bool HAS_IN>
static __device__ void sweep_lin(double *units_n, const int *y, int Tn, int Un, int Pl, int wave, unsigned *lat_n,
                                 int *scales, float *cost_n, bool has_out, int max_spins, unsigned *flag,
                                 unsigned *status) {
    constexpr int kGhost = BETA ? 63 : 0;    // plays the context next door
    constexpr int kProbe = BETA ? 62 : 1;    // the context that receives from it
    constexpr int kEdge = BETA ? 1 : 62;     // the context whose value is handed on
    const int lane = threadIdx.x & 63;
    const bool real = lane >= 1 && lane <= kLinReal;
    const int real_bits = real ? -1 : 0;   // (a mask, not a condition: no branch in the renormalisation)
    const int u = wave * kLinReal + lane - 1;
    double omask = 1.0, skipf, e, o;
    skipf = (real && (u >= 1) && (u < Un) && (y[u] != y[u - 1])) ? 1.0 : 0.0;
    if (BETA) {
        omask = ((real && (u >= 1) && (u <= Un)) || lane == kGhost) ? 1.0 : 0.0;
        e = (real && u == Un) ? 1.0 : 0.0;
        o = (real && u == Un && Un >= 1) ? 1.0 : 0.0;
    } else {
        e = (real && u == 0) ? 1.0 : 0.0;
        o = 0.0;
    }
    const int col = wave * 64 + lane;
    const size_t srow = (size_t)Pl * 2;
    unsigned *out = lat_n + (size_t)col * 2;
    pair_store(out + (size_t)(BETA ? Tn : 0) * srow, o, e);
    if (lane == 0) scales[0] = 0;
    const unsigned out_lane = (unsigned)col * 2u * (unsigned)sizeof(unsigned);
    const unsigned out_step = (unsigned)(srow * sizeof(unsigned));
    char *out_row = reinterpret_cast<char *>(lat_n) + (size_t)(BETA ? Tn - 1 : 1) * srow * sizeof(unsigned);
    int S = 0;   // the states are mass / 2^S

    if (Tn > 0) {
        ChunkL a, b;
        const int dir = BETA ? -1 : 1;
        const int t_start = BETA ? Tn - 1 : 0;
        const __amdgpu_buffer_rsrc_t rows_in = __builtin_amdgcn_make_buffer_rsrc(units_n, 0, 0xffffffffu, 0x00020000);
        const unsigned in_bytes = (unsigned)col * kCellBytes;
        const unsigned in_step = (unsigned)Pl * kCellBytes;
        // Where the lane's third factor lies.  Alpha: the next label's unit of its
        // own cell (for lane kGhost, the value handed over).  Beta: that of the
        // context below, i.e. of the column before its own, or, for the first
        // context of a wavefront, of the last context of the wavefront below, three
        // columns before (the first context of all reads the 0 of the column in
        // front of it); lane kGhost reads the value handed over from its own cell;
        // lane 0, whose state is always 0, reads the 1 of its own cell.
        unsigned third_bytes = in_bytes + kNextField;
        if (BETA) {
            if (lane == 0) third_bytes = in_bytes;
            else if (lane == 1) third_bytes = in_bytes - (wave > 0 ? 3u : 1u) * kCellBytes + kNextField;
            else if (lane != kGhost) third_bytes = in_bytes - kCellBytes + kNextField;
        }
        // the column this wavefront fills for the next one: its lane kGhost's
        const unsigned send_bytes = (unsigned)((BETA ? wave - 1 : wave + 1) * 64 + kGhost) * kCellBytes;
        chunk_load_lin<BETA>(a, rows_in, in_bytes, third_bytes, in_step, Tn, t_start);
        // byte offsets of a whole chunk's rows from its lowest one, in the units
        // and in the lattice: step r's row is the r-th from the bottom (alpha) or
        // from the top (beta)
        unsigned in_off[R], out_at[R];
#pragma unroll
        for (int r = 0; r < R; ++r) {
            in_off[r] = (unsigned)(BETA ? R - 1 - r : r) * in_step;
            out_at[r] = out_lane + (unsigned)(BETA ? R - 1 - r : r) * out_step;
        }
        bool lost = false;     // the hand-over did not arrive in time, or its sender says so
        // whether a chunk has to find out that its hand-over was complete (not
        // once it is lost, or holds NaNs of the sender's own)
        bool watch = HAS_IN;
        // lowest: the address of the chunk's lowest row of units (whole chunks only)
        auto run_chunk = [&](ChunkL &c, int k, int cnt, bool full, bool last, const char *lowest) {
            const int t_first = t_start + dir * k * R;
            const double e_kept = e, o_kept = o;
            const int S_kept = S;
            double mine[R];
            // (written so that the ordinary way through a chunk is one straight run
            // of instructions: a lone wavefront pays for every taken branch.  The
            // pass through the chunk's frames therefore exists twice for a wavefront
            // that receives: once in that run, once behind the wait for a hand-over
            // that had not arrived, out of the way.)
            auto pass = [&]() {
                double coded = 1.0;
                if (HAS_IN) {
                    coded = lane_value<kGhost>(c.lp[0][BETA ? 0 : 1]);
                    const int S_in = (int)(coded - kScaleBias);
                    // no mass here yet: what flows in sets the scale
                    const bool mass = (e != 0.0) | (o != 0.0);
                    S = (__ballot(real & mass) != 0ULL) ? S : S_in;
                    const double factor = __builtin_amdgcn_ldexp(1.0, S_in - S);
                    if (BETA) o = (lane == kGhost) ? factor : o;
                    else e = (lane == kGhost) ? factor : e;
                }
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
                            // with beta(t+1,2u+1) lp2 sent by context u+1, which holds
                            // lp2 of context u as its third factor
                            mine[r] = o * c.lp[r][2];
                            const double nxt = wave_shift_down_zero(mine[r]);
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
                            const double recv = wave_shift_up_zero(mine[r]);
                            o = __builtin_fma(o, c.lp[r][1], recv);
                            e = sum * c.lp[r][0];
                        }
                        // (the row's offset in the lane's offset register, a constant in
                        // the scalar offset field, as for every store of rows here: with a
                        // scalar register there the compiler lets the next instruction
                        // overwrite the data registers of a store of 16 bytes per lane,
                        // which this hardware does not forgive)
                        // (two stores of a word each: the two high words lie in registers
                        // that are not neighbours, and to put them side by side for one
                        // store of 8 bytes takes two moves, which cost more than the store)
                        const unsigned to = full ? out_at[r] : out_lane + at;
                        __builtin_amdgcn_raw_buffer_store_b32((unsigned)__double2hiint(o), rows, to, 0, 0);
                        __builtin_amdgcn_raw_buffer_store_b32((unsigned)__double2hiint(e), rows, to + 4u, 0, 0);
                        at = BETA ? at - out_step : at + out_step;
                    }
                }
                // a field that had not been written is a NaN, and by now it sits in
                // the context next to the lane that plays the sender; a scale that
                // had not been written is 0
                const double probe = BETA ? e : o;
                const bool nan_in = ((__ballot(probe != probe) >> kProbe) & 1ULL) != 0ULL;
                return nan_in | !(coded > 0.0);
            };
            const bool incomplete = pass();
            if (HAS_IN && __builtin_expect(watch & incomplete, 0)) {
                // Back to the states kept; wait for the chunk's hand-over and fetch
                // it again, then once more through the chunk.
                e = e_kept, o = o_kept, S = S_kept;
                // (the frame index through an empty asm: the addresses below are then
                // computed here, on the rare path, not ahead of every chunk)
                int t_again = t_first;
                asm volatile("" : "+s"(t_again));
                unsigned state = 0u;
                for (int spins = 0;; ++spins) {
                    chunk_reload_mail_lin<BETA>(c, rows_in, in_bytes, third_bytes, in_step, Tn, t_again);
                    state = chunk_mail_state_lin<BETA, kGhost>(c, cnt);
                    if (state != 0u || spins >= max_spins) break;
                    __builtin_amdgcn_s_sleep(2);
                }
                // (What was fetched ahead for the next chunk is as old as what failed,
                // so that chunk will come through here too, without having to wait.
                // Fetching it again here instead would cost every chunk a wait for
                // all loads in flight where the two versions of it meet.)
                if (state <= 1u) lost = true, watch = false;
                // all was there now: a NaN that is still found is the sender's own
                if (pass()) watch = false;
            }
            out_row = BETA ? out_row - (size_t)(full ? R : cnt) * out_step
                           : out_row + (size_t)(full ? R : cnt) * out_step;
            if (has_out && !lost && lane == kEdge) {
                const __amdgpu_buffer_rsrc_t to = full ? __builtin_amdgcn_make_buffer_rsrc(
                                                             const_cast<char *>(lowest), 0, 0xffffffffu, 0x00020000)
                                                       : rows_in;
                unsigned at = (unsigned)t_first * in_step;
                __builtin_amdgcn_raw_buffer_store_b64(as_words((double)S + kScaleBias), to,
                                                      send_bytes + scale_field<BETA>(), full ? in_off[0] : at,
                                                      kAgentScope);
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if (full || r < cnt)
                        __builtin_amdgcn_raw_buffer_store_b64(as_words(mine[r]), to, send_bytes + kNextField,
                                                              full ? in_off[r] : at, kAgentScope);
                    at = BETA ? at - in_step : at + in_step;
                }
            }
            if (lane == 0) scales[1 + k] = S;
            // the largest state back into [0.5, 1) (not after the last chunk: the
            // cost below is taken from the rows as they were stored).  The states
            // are not negative, so the largest one has the largest high word, whose
            // bits 20.. are its exponent + 1023: scalar arithmetic from there on.
            // All states 0 (or below the normal range): nothing to scale; a state
            // that is not finite: the check behind the sweeps will say so.
            if (!last) {
                const int top = wave_max_nonneg(max(__double2hiint(e), __double2hiint(o)) & real_bits) >> 20;
                const int ex = (top > 0 && top < 0x7ff) ? top - 1022 : 0;
                e = __builtin_amdgcn_ldexp(e, -ex);
                o = __builtin_amdgcn_ldexp(o, -ex);
                S += ex;
            }
        };
        int s0 = 0;
        // four chunks per turn; while the chunk after the turn lies inside the
        // sample, the rows of units need no clamp
        if (5 * R <= Tn) {
            // the lowest row of chunk 0, and from one chunk to the next
            const char *lowest = reinterpret_cast<const char *>(units_n) +
                                 (size_t)(BETA ? t_start - (R - 1) : 0) * in_step;
            const ptrdiff_t onward = (ptrdiff_t)dir * R * (ptrdiff_t)in_step;
            int k = 0;
            do {
                chunk_load_whole_lin(b, lowest + onward, in_off, in_bytes, third_bytes);
                run_chunk(a, k, R, true, false, lowest);
                chunk_load_whole_lin(a, lowest + 2 * onward, in_off, in_bytes, third_bytes);
                run_chunk(b, k + 1, R, true, false, lowest + onward);
                chunk_load_whole_lin(b, lowest + 3 * onward, in_off, in_bytes, third_bytes);
                run_chunk(a, k + 2, R, true, false, lowest + 2 * onward);
                chunk_load_whole_lin(a, lowest + 4 * onward, in_off, in_bytes, third_bytes);
                run_chunk(b, k + 3, R, true, false, lowest + 3 * onward);
                lowest += 4 * onward;
                k += 4;
                s0 += 4 * R;
            } while (s0 + 5 * R <= Tn);
        }
        // the rest (fewer than five chunks), one chunk per turn
        while (s0 < Tn) {
            chunk_load_lin<BETA>(b, rows_in, in_bytes, third_bytes, in_step, Tn, t_start + dir * (s0 + R));
            run_chunk(a, s0 / R, min(Tn - s0, R), false, s0 + R >= Tn, nullptr);
            a = b;
            s0 += R;
        }
        if (lost) {
            // the log-domain kernels take over; whoever waits behind is told
            if (lane == 0) {
                atomicOr(flag, 1u);
                if (status) atomicOr(status, kStatusLostHandOver);
            }
            if (has_out && lane == kEdge) {
                v2u_lin gone;
                gone[0] = (unsigned)kLostBits, gone[1] = kLostHigh;
                for (int t = 0; t < Tn; ++t) {
                    __builtin_amdgcn_raw_buffer_store_b64(gone, rows_in, send_bytes + kNextField,
                                                          (unsigned)t * in_step, kAgentScope);
                    __builtin_amdgcn_raw_buffer_store_b64(gone, rows_in, send_bytes + scale_field<BETA>(),
                                                          (unsigned)t * in_step, kAgentScope);
                }
            }
        }
    }
    // cost = -ln(beta(0, state 0) * 2^S)
    if (BETA && real && u == 0) {
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
    double *__restrict__ units, const int *__restrict__ ys, const int *__restrict__ lx,
    const int *__restrict__ ly, unsigned *__restrict__ alphas, unsigned *__restrict__ betas,
    int *__restrict__ scales, float *__restrict__ costs, int N, int T, int U, int W, int chains_pad,
    const CostReduce red, int max_spins, unsigned *__restrict__ flag, unsigned *__restrict__ status) {
    // workgroup index = link * chains_pad + chain, chain = n * 2 + d (d = 0: beta,
    // 1: alpha), first sender first, as in lattice.hip
    const int chain = blockIdx.x % chains_pad, link = blockIdx.x / chains_pad;
    if (chain >= N * 2) return;
    const int n = chain / 2;
    const bool beta = (chain % 2) == 0;
    const int wave = beta ? W - 1 - link : link;
    const int Pl = 64 * W;
    const int Tn = min(max(lx[n], 0), T);
    const int Un = min(max(ly[n], 0), U);
    if (wave * kLinReal > Un) return;
    double *units_n = units + (size_t)n * T * Pl * kLinUnit;
    const int *y = ys + (size_t)n * U;
    const size_t lat = (size_t)(T + 1) * Pl * 2;
    const int chunks = lin_chunks(T);
    int *sc = scales + (((size_t)n * 2 + (beta ? 0 : 1)) * W + wave) * (size_t)(chunks + 1);
    const bool above = (wave + 1) * kLinReal <= Un;   // a wavefront holds contexts above this one's
    if (!beta) {
        if (wave > 0)
            sweep_lin<false, true>(units_n, y, Tn, Un, Pl, wave, alphas + (size_t)n * lat, sc, nullptr, above,
                                   max_spins, flag, status);
        else
            sweep_lin<false, false>(units_n, y, Tn, Un, Pl, wave, alphas + (size_t)n * lat, sc, nullptr, above,
                                    max_spins, flag, status);
        return;
    }
    if (above)
        sweep_lin<true, true>(units_n, y, Tn, Un, Pl, wave, betas + (size_t)n * lat, sc, costs + n, wave > 0,
                              max_spins, flag, status);
    else
        sweep_lin<true, false>(units_n, y, Tn, Un, Pl, wave, betas + (size_t)n * lat, sc, costs + n, wave > 0,
                               max_spins, flag, status);
    if (wave != 0) return;
    cost_reduce_tail(red, costs, lx, n, N, threadIdx.x);
}

}  // namespace

size_t lattice_lin_scales(int N, int T, int U) {
    return (size_t)N * 2 * lin_waves(U) * (size_t)(lin_chunks(T) + 1);
}

hipError_t launch_lattice_lin(const LatticeArgs &a, int *scales, unsigned *flag, hipStream_t stream) {
    if (a.N == 0) return hipSuccess;
    if (a.beta_only || !scales || !flag) return hipErrorInvalidValue;
    const int W = lin_waves(a.U);
    const long chains_pad = ((long)a.N * 2 + 7) / 8 * 8;
    if (chains_pad * W > 0x7fffffffL) return hipErrorInvalidValue;
    // a sample's units are addressed through 32-bit byte offsets
    if ((size_t)a.T * 64 * W * kCellBytes >= (1ULL << 31)) return hipErrorInvalidValue;
    const int max_spins = lattice_wait_limit_now();
    TIMED_LAUNCH(lattice_lin_kernel, dim3((unsigned)(chains_pad * W)), dim3(64), 0, stream,
                 const_cast<double *>(a.units), a.ys, a.lx, a.ly, reinterpret_cast<unsigned *>(a.alphas),
                 reinterpret_cast<unsigned *>(a.betas), scales, a.costs, a.N, a.T,
                 a.U, W, (int)chains_pad, a.reduce, max_spins, flag, device_status_word());
    return hipGetLastError();
}

}  // namespace wctct
