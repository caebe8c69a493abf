// The scan kernels. A row is one (b, m, d) sequence of length L. In the two general ones
// (scan_forward_kernel, scan_backward_kernel) W waves
// cooperate on one row: a tile is W*64 chunks of 16 bytes, consecutive in memory,
// one chunk per lane. Tiles of a row are walked serially (forward: first to
// last; backward: last to first) with the running state of the row in a
// register, so a row of any length costs one read of every input and one write
// of every output.
//
// Per tile a lane (1) folds its chunk into one (a, b) step pair, (2) the wave
// scans the 64 pairs with DPP, (3) with W > 1 the wave totals meet in LDS,
// (4) the lane replays its chunk from the state that enters it and stores.
// The chain that links one tile to the next is a single fma on the row state.
//
// A wave keeps the loads of the next P tiles of its row in flight while it scans the
// current one. The grid has one block per row (W > 1) or per R rows (W == 1); the
// host bounds how many blocks a compute unit holds at a time, because the HBM
// efficiency of this access pattern depends on how many rows stream concurrently.
//
// Few rows, long sequences: a row can be cut into `nseg` segments of `seg_tiles` tiles
// that are scanned as if they were rows of their own (two passes). Pass one
// (scan_aggregate_kernel) reduces every segment to its step pair (A, B); pass two is
// the ordinary scan kernel, whose block first folds the pairs of the segments that
// precede its own into the state that enters it.
#pragma once

#include <type_traits>

#include "fmscan_device.h"

namespace fmscan {

// Values that are the same in every lane of a wave but come out of vector instructions
// (integer division has no scalar form) are moved to scalar registers, so that the row
// pointers derived from them do not occupy two vector registers each.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform64(int64_t v) {
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)v);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readfirstlane((int)(uint32_t)((uint64_t)v >> 32));
    return (int64_t)(((uint64_t)hi << 32) | lo);
}

// Output row r = (b*M + m)*D + d  ->  gate row b*M + m, token row b*D + d
// (reference fm/scan/fm_scan.cuh:76-82).
struct RowMap {
    int64_t gate_row, token_row;
};
__device__ __forceinline__ RowMap map_row(int64_t row, int32_t M, int32_t D) {
    const uint32_t r = (uint32_t)row;  // rows < 2^31 is checked by the host
    const uint32_t gate_row = r / (uint32_t)D;
    const uint32_t b = gate_row / (uint32_t)M;
    RowMap m;
    m.gate_row = (int64_t)(uint32_t)uniform((int)gate_row);
    m.token_row = uniform64((int64_t)b * D + (r - gate_row * (uint32_t)D));
    return m;
}

// Which part of which row a slot of the grid works on. With nseg == 1 a slot is a row.
struct Segment {
    int64_t row;
    int32_t index;        // segment inside the row
    int64_t k_lo, k_hi;   // its tiles: [k_lo, k_hi)
};
__device__ __forceinline__ Segment locate_segment(int64_t slot, int32_t nseg, int64_t seg_tiles,
                                                  int64_t ntiles) {
    Segment s;
    s.row = nseg > 1 ? uniform64(slot / nseg) : slot;
    s.index = nseg > 1 ? (int32_t)(slot - s.row * nseg) : 0;
    s.k_lo = (int64_t)s.index * seg_tiles;
    s.k_hi = s.k_lo + seg_tiles < ntiles ? s.k_lo + seg_tiles : ntiles;
    return s;
}

// Which slot (row, or segment of a row) wave-group `local` of a block works on: rows in memory
// order, unless rows that share their inputs are better visited together. With M > 1 the M rows
// (b, :, d) read the same tokens; when the tokens of a batch element do not fit an L2 (4 MiB
// per XCD), going through the rows in memory order fetches them once per slot m instead of once
// (D = 2048, L = 8192: as many bytes fetched as written). Then blocks are renumbered so that
// every XCD (blocks go to the 8 XCDs round robin) takes a contiguous range of them, and inside
// a batch element the rows are taken in groups of d whose tokens (256 KiB) stay in the cache
// while the M slots are visited one after the other; within a slot the group's rows are
// consecutive in memory, so the output is still written in runs. Measured on the forward
// kernel at (1, 32, 2048, 8192): 0.24 -> 0.18 ms; shapes whose tokens fit are up to a quarter
// slower in that order (their writes jump by D rows from block to block) and keep memory order.
template <int R, bool FOLD>
__device__ __forceinline__ int64_t slot_of_block(int local, int32_t M, int32_t D, int32_t nseg, int64_t row_bytes) {
    uint32_t id = blockIdx.x;
    if constexpr (!FOLD) {
        if (nseg == 1 && M > 1 && D % R == 0 && D * row_bytes > (4 << 20)) {
            const uint32_t quads = (uint32_t)(D / R);  // blocks per slot
            uint32_t group = 1;                        // blocks of one slot visited before the next slot
            while (group * 2 <= quads && (int64_t)(group * 2) * R * row_bytes <= (256 << 10)) group *= 2;
            while (quads % group) group /= 2;
            if (gridDim.x % 8u == 0u) id = (id % 8u) * (gridDim.x / 8u) + id / 8u;
            const uint32_t per_b = (uint32_t)M * quads, per_group = (uint32_t)M * group;
            const uint32_t b = id / per_b, rest = id - b * per_b;
            const uint32_t grp = rest / per_group, in_group = rest - grp * per_group;
            const uint32_t m = in_group / group, dq = grp * group + (in_group - m * group);
            const uint32_t gate_row = (uint32_t)uniform((int)(b * (uint32_t)M + m));
            return (int64_t)gate_row * D + (int64_t)uniform((int)(dq * R)) + local;
        }
    }
    return (int64_t)id * R + local;
}

// Meets the W wave totals of one tile in LDS. `cin` leaves as the state that
// enters this wave's part of the tile, `carry` as the state after the tile.
// Slots alternate between consecutive tiles, so one barrier per tile is enough:
// a wave can only overwrite a slot after every wave has passed the barrier of
// the tile in between, i.e. has finished reading it.
template <int W>
__device__ __forceinline__ void combine_waves(float2 (*slots)[W], int parity, int w, int lane,
                                              float ta, float tb, float& cin, float& carry) {
    if (lane == 63) slots[parity][w] = make_float2(ta, tb);
    __syncthreads();
    float c = carry;
    cin = carry;
#pragma unroll
    for (int j = 0; j < W; ++j) {
        const float2 p = slots[parity][j];
        c = __builtin_fmaf(p.x, c, p.y);
        if (j + 1 == w) cin = c;
    }
    carry = c;
}

// ---- forward ------------------------------------------------------------------------
// h_t = g_t h_{t-1} + u_t,  u_t = (1 - g_t) x_t  (PLAIN: u_t = x_t)
// reference fm/scan/fm_scan.cuh:110,116,121-131,139-140; fm/scan/fm_pytorch.py:22,37.
// FOLD: M == D == 1, every gate and token row belongs to exactly one output row.
template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
__global__ __launch_bounds__(64 * W * R) void scan_forward_kernel(
    const T* __restrict__ gates, const T* __restrict__ tokens, const T* __restrict__ h0,
    T* __restrict__ out, int64_t rows, int32_t M, int32_t D, int64_t L, int32_t nseg,
    int64_t seg_tiles, const float2* __restrict__ seg_pairs) {
    static_assert(W == 1 || R == 1, "waves that share a barrier must share a row");
    constexpr int E = Elem<T>::E;
    constexpr int64_t TILE = (int64_t)E * 64 * W;
    const int lane = threadIdx.x & 63;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int w = wave % W;
    const int64_t slot = slot_of_block<R, FOLD>(wave / W, M, D, nseg, L * (int64_t)sizeof(T));
    if (slot >= rows * nseg) return;  // whole waves only, and only in barrier-free (W == 1) blocks
    const int64_t ntiles = (L + TILE - 1) / TILE;
    const Segment seg = locate_segment(slot, nseg, seg_tiles, ntiles);
    const int64_t r = seg.row;

    __shared__ float2 slots[2][W];

    const RowMap rm = map_row(r, M, D);
    const T* __restrict__ grow = gates + rm.gate_row * L;
    const T* __restrict__ xrow = tokens + rm.token_row * L;
    T* __restrict__ orow = out + r * L;
    float carry = h0 ? Elem<T>::widen(h0[r]) : 0.0f;
    for (int32_t j = 0; j < seg.index; ++j) {  // the segments before this one, oldest first
        const float2 p = seg_pairs[r * nseg + j];
        carry = __builtin_fmaf(p.x, carry, p.y);
    }

    const int64_t lane_off = (int64_t)(w * 64 + lane) * E;

    struct Entry {
        u32x4 g, x;
    };
    // loads stop at the end of the segment (the end of the row when rows are not cut);
    // tiles below k_whole lie wholly inside
    const int64_t t_end = seg.k_hi * TILE < L ? seg.k_hi * TILE : L;
    const int64_t k_whole = VEC ? t_end / TILE : 0;
    auto fetch_whole = [&](Entry& q, int64_t k) {  // no check of any kind
        const int64_t t0 = k * TILE + lane_off;
        q.g = load16<T, FOLD>(grow + t0);
        q.x = load16<T, FOLD>(xrow + t0);
    };
    auto fetch = [&](Entry& q, int64_t k) {
        const int64_t t0 = k * TILE + lane_off;
        q.g = load_chunk<T, VEC, FOLD>(grow, t0, t_end, Elem<T>::kOnes);
        q.x = load_chunk<T, VEC, FOLD>(xrow, t0, t_end, 0u);
    };

    // One tile: fold, wave scan, meet the other waves, replay, store. `whole` tiles store
    // without a bound check.
    auto scan_tile = [&](const Entry& cur, int64_t k, auto whole) {
        const int64_t t0 = k * TILE + lane_off;
        float g[E], u[E];
        Elem<T>::unpack(cur.g, g);
        Elem<T>::unpack(cur.x, u);
        if constexpr (!PLAIN) {
#pragma unroll
            for (int i = 0; i < E; ++i) u[i] = __builtin_fmaf(-g[i], u[i], u[i]);  // (1-g)x, one rounding
        }

        // the chunk as one step: h_out = a*h_in + b
        float a = g[0], b = u[0];
#pragma unroll
        for (int i = 1; i < E; ++i) {
            b = __builtin_fmaf(g[i], b, u[i]);
            a *= g[i];
        }
        wave_scan_inclusive(a, b);
        const float ea = dpp<kWaveShr1>(1.0f, a);  // composition of the chunks before this lane
        const float eb = dpp<kWaveShr1>(0.0f, b);
        const float ta = lane63(a), tb = lane63(b);

        float cin = carry;
        if constexpr (W > 1) {
            combine_waves<W>(slots, (int)(k & 1), w, lane, ta, tb, cin, carry);
        } else {
            carry = __builtin_fmaf(ta, carry, tb);
        }

        float h = __builtin_fmaf(ea, cin, eb);
        float o[E];
#pragma unroll
        for (int i = 0; i < E; ++i) {
            h = __builtin_fmaf(g[i], h, u[i]);
            o[i] = h;
        }
        if constexpr (decltype(whole)::value) store16<T>(orow + t0, Elem<T>::pack(o));
        else store_chunk<T, VEC>(orow, t0, L, Elem<T>::pack(o));
    };

    // The steady part of the row runs without a single conditional memory operation and
    // without bound checks (measured faster than the checked loop, which waits for every
    // load in flight before each use because it can no longer count the newer ones).
    // It covers the tiles whose prefetch target is still a whole tile; the rest of the row
    // takes the checked path. What the unrolled body does not do is wait tile by tile: the
    // compiler moves the first use of all P entries to its top, so the loads are waited
    // for as a group, once per P tiles. Keeping the tiles apart with scheduling barriers
    // gives true P-deep waits and was measured at the same speed (backward) or 3 % slower
    // (forward): with this many waves streaming, occupancy already covers the latency.
    Entry q[P];
    const int64_t count = seg.k_hi - seg.k_lo;
    const int64_t nwhole = k_whole - seg.k_lo;  // whole tiles at the start of the segment
    int64_t n = 0;
    if (nwhole >= 2 * P) {
#pragma unroll
        for (int s = 0; s < P; ++s) fetch_whole(q[s], seg.k_lo + s);
        for (; n + 2 * P <= nwhole; n += P) {
#pragma unroll
            for (int s = 0; s < P; ++s) {
                const int64_t k = seg.k_lo + n + s;
                const Entry cur = q[s];
                fetch_whole(q[s], k + P);
                scan_tile(cur, k, std::true_type{});
            }
        }
    } else {
#pragma unroll
        for (int s = 0; s < P; ++s) fetch(q[s], seg.k_lo + s);
    }
    for (; n < count; n += P) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
            if (n + s >= count) break;
            const int64_t k = seg.k_lo + n + s;
            const Entry cur = q[s];
            fetch(q[s], k + P);
            scan_tile(cur, k, std::false_type{});
        }
    }
}

// ---- backward -----------------------------------------------------------------------
// delta_t = G_t + g_{t+1} delta_{t+1}, delta_L = first_prop_grad (reference
// fm/scan/fm_scan.cuh:88,103-108,121). The kernel carries c_t = g_{t+1} delta_{t+1}
// instead (the part of delta_t that arrives from the future): c_{t-1} = g_t c_t + g_t G_t
// is the same operator with unshifted gates, walked from the end of the row.
// Lane l of wave w owns the chunk that is (w*64 + l) chunks before the end of the
// tile, so the suffix scan in memory order is a prefix scan in lane order.
//   token_grad_t = (1 - g_t) delta_t                  (:184-185)   PLAIN: delta_t
//   gate_grad_t  = (h_{t-1} - x_t) delta_t            (:188-208)   PLAIN: h_{t-1} delta_t
template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
__global__ __launch_bounds__(64 * W * R) void scan_backward_kernel(
    const T* __restrict__ gates, const T* __restrict__ out_grad, const T* __restrict__ first_prop_grad,
    T* __restrict__ token_grad, const T* __restrict__ h_saved, const T* __restrict__ tokens,
    T* __restrict__ gate_grad, const T* __restrict__ h0, T* __restrict__ h0_grad, int64_t rows,
    int32_t M, int32_t D, int64_t L, int32_t nseg, int64_t seg_tiles,
    const float2* __restrict__ seg_pairs) {
    static_assert(W == 1 || R == 1, "waves that share a barrier must share a row");
    constexpr int E = Elem<T>::E;
    constexpr int64_t TILE = (int64_t)E * 64 * W;
    const int lane = threadIdx.x & 63;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int w = wave % W;
    const int64_t slot = slot_of_block<R, FOLD>(wave / W, M, D, nseg, L * (int64_t)sizeof(T));
    if (slot >= rows * nseg) return;
    const int64_t ntiles = (L + TILE - 1) / TILE;
    const Segment seg = locate_segment(slot, nseg, seg_tiles, ntiles);
    const int64_t r = seg.row;

    __shared__ float2 slots[2][W];

    const RowMap rm = map_row(r, M, D);
    const T* __restrict__ grow = gates + rm.gate_row * L;
    const T* __restrict__ Grow = out_grad + r * L;
    const T* __restrict__ hrow = h_saved + r * L;
    const T* __restrict__ xrow = tokens + rm.token_row * L;  // never read when PLAIN
    T* __restrict__ dxrow = token_grad + r * L;
    T* __restrict__ dgrow = gate_grad + r * L;
    float carry = first_prop_grad ? Elem<T>::widen(first_prop_grad[r]) : 0.0f;
    for (int32_t j = nseg - 1; j > seg.index; --j) {  // the segments after this one, last first
        const float2 p = seg_pairs[r * nseg + j];
        carry = __builtin_fmaf(p.x, carry, p.y);
    }
    const float hinit = h0 ? Elem<T>::widen(h0[r]) : 0.0f;

    const int64_t lane_off = (int64_t)(64 * W - 1 - (w * 64 + lane)) * E;

    // PLAIN reads the saved states (its gate gradient needs nothing else). Otherwise the
    // states of a tile are not read but made again, in float32, from the tile's gates and
    // tokens (already in registers) and the one saved state just before this wave's part of
    // the tile: a second wave scan, forward in time, in place of a fourth 16-byte stream.
    const uint32_t vzero = opaque_zero();
    struct Entry {
        u32x4 g, G;
        u32x4 hx;  // PLAIN: saved states; otherwise tokens
        float hb;  // h just before this wave's part of the tile (h[-1] at t = 0)
        float h_first;  // checked tiles only, when this wave's part begins the row (`first`): the saved h[0]
        bool first;
    };
    // tiles in [k_lo, k_whole) lie wholly inside the row
    const int64_t k_whole = VEC ? L / TILE : 0;
    // first position of this wave's part of a tile, relative to the tile: what lane 63 owns
    const int64_t wave_off = (int64_t)(64 * W - 64 - w * 64) * E;
    // a whole tile that is not the first of the row: no check of any kind
    auto fetch_whole = [&](Entry& q, int64_t k) {
        const int64_t t0 = k * TILE + lane_off;
        q.g = load16<T, FOLD>(grow + t0);
        q.G = load16<T, true>(Grow + t0);
        if constexpr (PLAIN) q.hx = load16<T, true>(hrow + t0);
        else q.hx = load16<T, FOLD>(xrow + t0);
        q.hb = Elem<T>::widen(load_by_wave(hrow + (k * TILE + wave_off - 1), vzero));
        q.h_first = 0.0f;  // never looked at: whole tiles are not the first of a row
        q.first = false;
    };
    auto fetch = [&](Entry& q, int64_t k) {
        // k < k_lo (before the segment): t0 = L, which every bound check rejects
        const int64_t t0 = k >= seg.k_lo ? k * TILE + lane_off : L;
        q.g = load_chunk<T, VEC, FOLD>(grow, t0, L, Elem<T>::kOnes);
        q.G = load_chunk<T, VEC, true>(Grow, t0, L, 0u);
        if constexpr (PLAIN) q.hx = load_chunk<T, VEC, true>(hrow, t0, L, 0u);
        else q.hx = load_chunk<T, VEC, FOLD>(xrow, t0, L, 0u);
        // h just before this wave's part of the tile: one address for the whole wave,
        // always loaded (position 0 stands in where there is nothing before) and replaced by
        // h[-1] at the start of the row
        const int64_t tw = k * TILE + wave_off;
        const bool before = k >= seg.k_lo && tw > 0 && tw < L;
        const float loaded = Elem<T>::widen(load_by_wave(hrow + (before ? tw - 1 : 0), vzero));
        q.hb = before ? loaded : hinit;
        // Where the part begins the row, `hinit` is what the gate gradient at t = 0 is to see,
        // which need not be the state the forward call started from (a caller that passes no
        // initial state gets the reference's first_prop_grad there). The states after it are
        // therefore made from the saved h[0], which `loaded` then holds.
        q.h_first = loaded;
        q.first = k >= seg.k_lo && tw == 0;
    };

    // One tile: fold, wave scan, meet the other waves, replay with both epilogues, store.
    // `whole` tiles store without a bound check.
    auto scan_tile = [&](const Entry& cur, int64_t k, auto whole) {
        const int64_t t0 = k * TILE + lane_off;
        float g[E], G[E], p[E];
        Elem<T>::unpack(cur.g, g);
        Elem<T>::unpack(cur.G, G);
#pragma unroll
        for (int i = 0; i < E; ++i) p[i] = g[i] * G[i];

        // the chunk as one step on the incoming part: c_out = a*c_in + b
        float a = g[E - 1], b = p[E - 1];
#pragma unroll
        for (int i = E - 2; i >= 0; --i) {
            b = __builtin_fmaf(g[i], b, p[i]);
            a *= g[i];
        }
        float fa = a;  // the product of the chunk's gates serves the forward step pair too
        wave_scan_inclusive(a, b);
        const float ea = dpp<kWaveShr1>(1.0f, a);
        const float eb = dpp<kWaveShr1>(0.0f, b);
        const float ta = lane63(a), tb = lane63(b);

        // hp[i] = h at the position before element i of the chunk; x[] the tokens
        float hp[E], x[E];
        if constexpr (PLAIN) {
            float h[E];
            Elem<T>::unpack(cur.hx, h);
            // the last element of the chunk before this one in memory, which the next lane
            // holds; lane 63 takes the look-behind value
            hp[0] = dpp<kWaveShl1>(cur.hb, h[E - 1]);
#pragma unroll
            for (int i = 1; i < E; ++i) hp[i] = h[i - 1];
        } else {
            float u[E];
            Elem<T>::unpack(cur.hx, x);
#pragma unroll
            for (int i = 0; i < E; ++i) u[i] = __builtin_fmaf(-g[i], x[i], x[i]);  // as the forward kernel forms it
            float g0 = g[0];
            if constexpr (!decltype(whole)::value) {
                // first step of the row: whatever enters, the saved h[0] leaves
                if (lane == 63 && cur.first) {
                    g0 = 0.0f;
                    u[0] = cur.h_first;
                    fa = 0.0f;
                }
            }
            float fb = u[0];
#pragma unroll
            for (int i = 1; i < E; ++i) fb = __builtin_fmaf(g[i], fb, u[i]);
            // positions past the end of the row carry g = 1, x = 0: identity steps
            row_scan_inclusive_down(fa, fb);
            hp[0] = state_entering_lane_down(fa, fb, cur.hb, lane);
            hp[1] = __builtin_fmaf(g0, hp[0], u[0]);
#pragma unroll
            for (int i = 2; i < E; ++i) hp[i] = __builtin_fmaf(g[i - 1], hp[i - 1], u[i - 1]);
        }

        float cin = carry;
        if constexpr (W > 1) {
            combine_waves<W>(slots, (int)(k & 1), w, lane, ta, tb, cin, carry);
        } else {
            carry = __builtin_fmaf(ta, carry, tb);
        }

        float c = __builtin_fmaf(ea, cin, eb);
        float dx[E], dg[E];
#pragma unroll
        for (int i = E - 1; i >= 0; --i) {
            const float delta = G[i] + c;
            c = __builtin_fmaf(g[i], c, p[i]);
            if constexpr (PLAIN) {
                dx[i] = delta;
                dg[i] = hp[i] * delta;
            } else {
                dx[i] = __builtin_fmaf(-g[i], delta, delta);
                dg[i] = (hp[i] - x[i]) * delta;
            }
        }
        if constexpr (decltype(whole)::value) {
            store16<T>(dxrow + t0, Elem<T>::pack(dx));
            store16<T>(dgrow + t0, Elem<T>::pack(dg));
        } else {
            store_chunk<T, VEC>(dxrow, t0, L, Elem<T>::pack(dx));
            store_chunk<T, VEC>(dgrow, t0, L, Elem<T>::pack(dg));
        }
    };

    // Tiles are taken from the end of the segment: n = 0 is tile k_hi - 1. As in the
    // forward kernel the steady part has no conditional memory operation. It starts after
    // a first checked group when the last tile of the row is ragged, and ends where the
    // prefetch target would fall before the segment (or on the first tile of the row,
    // whose look-behind value is h[-1]).
    Entry q[P];
    const int64_t count = seg.k_hi - seg.k_lo;
    const bool ragged_top = seg.k_hi > k_whole;
    int64_t n = 0;
    if (VEC && !ragged_top && count >= 2 * P + 1) {
#pragma unroll
        for (int s = 0; s < P; ++s) fetch_whole(q[s], seg.k_hi - 1 - s);
    } else {
#pragma unroll
        for (int s = 0; s < P; ++s) fetch(q[s], seg.k_hi - 1 - s);
        if (VEC && ragged_top && count >= 3 * P + 1) {  // one checked group, then whole tiles follow
#pragma unroll
            for (int s = 0; s < P; ++s) {
                const int64_t k = seg.k_hi - 1 - s;
                const Entry cur = q[s];
                fetch(q[s], k - P);
                scan_tile(cur, k, std::false_type{});
            }
            n = P;
        } else {
            n = count;  // marks "no steady part": the checked loop below starts from zero
        }
    }
    if (n < count) {
        // prefetch targets n + P .. n + 2P - 1 must stay above the first tile of the segment
        for (; n + 2 * P + 1 <= count; n += P) {
#pragma unroll
            for (int s = 0; s < P; ++s) {
                const int64_t k = seg.k_hi - 1 - (n + s);
                const Entry cur = q[s];
                fetch_whole(q[s], k - P);
                scan_tile(cur, k, std::true_type{});
            }
        }
    } else {
        n = 0;
    }
    for (; n < count; n += P) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
            if (n + s >= count) break;
            const int64_t k = seg.k_hi - 1 - (n + s);
            const Entry cur = q[s];
            fetch(q[s], k - P);
            scan_tile(cur, k, std::false_type{});
        }
    }

    // what is left after the first step is g_0 * delta_0: the gradient of the state before the row
    if (h0_grad && seg.index == 0 && w == 0 && lane == 0) {
        float v[E] = {carry};
        const u32x4 packed = Elem<T>::pack(v);
        if constexpr (sizeof(T) == 4) reinterpret_cast<uint32_t*>(h0_grad)[r] = packed.x;
        else reinterpret_cast<uint16_t*>(h0_grad)[r] = (uint16_t)(packed.x & 0xffffu);
    }
}

// ---- pass one of a segmented scan ------------------------------------------------------
// Reduces every segment to its step pair. Forward: pairs (g_t, u_t) composed left to
// right, so that state_after = A * state_before + B. Backward: pairs (g_t, g_t G_t)
// composed right to left (the carried quantity is c_t, see scan_backward_kernel).
// One wave per segment, no LDS. The last segment of a row (forward) / the first
// (backward) is never needed and is skipped.
template <typename T, int R, int P, bool PLAIN, bool VEC, bool BACKWARD>
__global__ __launch_bounds__(64 * R) void scan_aggregate_kernel(
    const T* __restrict__ gates, const T* __restrict__ other /* tokens | out_grad */,
    float2* __restrict__ seg_pairs, int64_t rows, int32_t M, int32_t D, int64_t L, int32_t nseg,
    int64_t seg_tiles) {
    constexpr int E = Elem<T>::E;
    constexpr int64_t TILE = (int64_t)E * 64;
    const int lane = threadIdx.x & 63;
    const int wave = uniform((int)(threadIdx.x >> 6));
    const int64_t slot = (int64_t)blockIdx.x * R + wave;
    if (slot >= rows * nseg) return;
    const int64_t ntiles = (L + TILE - 1) / TILE;
    const Segment seg = locate_segment(slot, nseg, seg_tiles, ntiles);
    if (seg.index == (BACKWARD ? 0 : nseg - 1)) return;
    const int64_t r = seg.row;

    const RowMap rm = map_row(r, M, D);
    const T* __restrict__ grow = gates + rm.gate_row * L;
    const T* __restrict__ orow = other + (BACKWARD ? r : rm.token_row) * L;
    const int64_t lane_off = (int64_t)(BACKWARD ? 63 - lane : lane) * E;

    struct Entry {
        u32x4 g, o;
    };
    auto fetch = [&](Entry& q, int64_t k) {
        const int64_t t0 = (k >= seg.k_lo && k < seg.k_hi) ? k * TILE + lane_off : L;
        q.g = load_chunk<T, VEC, false>(grow, t0, L, Elem<T>::kOnes);
        q.o = load_chunk<T, VEC, false>(orow, t0, L, 0u);
    };
    const int64_t first = BACKWARD ? seg.k_hi - 1 : seg.k_lo;
    constexpr int64_t step = BACKWARD ? -1 : 1;

    Entry q[P];
#pragma unroll
    for (int s = 0; s < P; ++s) fetch(q[s], first + step * s);

    float A = 1.0f, B = 0.0f;
    const int64_t count = seg.k_hi - seg.k_lo;
    for (int64_t n0 = 0; n0 < count; n0 += P) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
            const int64_t n = n0 + s;
            if (n >= count) break;
            const Entry cur = q[s];
            fetch(q[s], first + step * (n + P));
            float g[E], v[E];
            Elem<T>::unpack(cur.g, g);
            Elem<T>::unpack(cur.o, v);
#pragma unroll
            for (int i = 0; i < E; ++i) {
                if constexpr (BACKWARD) v[i] = g[i] * v[i];
                else if constexpr (!PLAIN) v[i] = __builtin_fmaf(-g[i], v[i], v[i]);
            }
            float a, b;
            if constexpr (BACKWARD) {
                a = g[E - 1];
                b = v[E - 1];
#pragma unroll
                for (int i = E - 2; i >= 0; --i) {
                    b = __builtin_fmaf(g[i], b, v[i]);
                    a *= g[i];
                }
            } else {
                a = g[0];
                b = v[0];
#pragma unroll
                for (int i = 1; i < E; ++i) {
                    b = __builtin_fmaf(g[i], b, v[i]);
                    a *= g[i];
                }
            }
            wave_scan_inclusive(a, b);
            const float ta = lane63(a), tb = lane63(b);
            B = __builtin_fmaf(ta, B, tb);  // segment so far, then this tile
            A *= ta;
        }
    }
    if (lane == 0) seg_pairs[r * nseg + seg.index] = make_float2(A, B);
}

}  // namespace fmscan
