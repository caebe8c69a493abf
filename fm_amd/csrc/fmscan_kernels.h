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
    const int64_t slot = (int64_t)blockIdx.x * R + wave / W;
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
    const int64_t slot = (int64_t)blockIdx.x * R + wave / W;
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

    struct Entry {
        u32x4 g, G, h, x;
        float hb;  // lane 63 only: h just before this wave's part of the tile (h[-1] at t = 0)
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
        q.h = load16<T, true>(hrow + t0);
        if constexpr (!PLAIN) q.x = load16<T, FOLD>(xrow + t0);
        q.hb = Elem<T>::widen(hrow[k * TILE + wave_off - 1]);
    };
    auto fetch = [&](Entry& q, int64_t k) {
        // k < k_lo (before the segment): t0 = L, which every bound check rejects
        const int64_t t0 = k >= seg.k_lo ? k * TILE + lane_off : L;
        q.g = load_chunk<T, VEC, FOLD>(grow, t0, L, Elem<T>::kOnes);
        q.G = load_chunk<T, VEC, true>(Grow, t0, L, 0u);
        q.h = load_chunk<T, VEC, true>(hrow, t0, L, 0u);
        if constexpr (!PLAIN) q.x = load_chunk<T, VEC, FOLD>(xrow, t0, L, 0u);
        // h just before this wave's part of the tile: one address for the whole wave,
        // always loaded (position 0 stands in where there is nothing before) and replaced by
        // h[-1] at the start of the row
        const int64_t tw = k * TILE + wave_off;
        const bool before = k >= seg.k_lo && tw > 0 && tw < L;
        const float loaded = Elem<T>::widen(hrow[before ? tw - 1 : 0]);
        q.hb = before ? loaded : hinit;
    };

    // One tile: fold, wave scan, meet the other waves, replay with both epilogues, store.
    // `whole` tiles store without a bound check.
    auto scan_tile = [&](const Entry& cur, int64_t k, auto whole) {
        const int64_t t0 = k * TILE + lane_off;
        float g[E], G[E], h[E], p[E];
        Elem<T>::unpack(cur.g, g);
        Elem<T>::unpack(cur.G, G);
        Elem<T>::unpack(cur.h, h);
#pragma unroll
        for (int i = 0; i < E; ++i) p[i] = g[i] * G[i];

        // the chunk as one step on the incoming part: c_out = a*c_in + b
        float a = g[E - 1], b = p[E - 1];
#pragma unroll
        for (int i = E - 2; i >= 0; --i) {
            b = __builtin_fmaf(g[i], b, p[i]);
            a *= g[i];
        }
        wave_scan_inclusive(a, b);
        const float ea = dpp<kWaveShr1>(1.0f, a);
        const float eb = dpp<kWaveShr1>(0.0f, b);
        const float ta = lane63(a), tb = lane63(b);
        // h at the position before this chunk: last element of the chunk before it
        // in memory, which the next lane holds; lane 63 takes the look-behind value.
        const float hprev0 = dpp<kWaveShl1>(cur.hb, h[E - 1]);

        float cin = carry;
        if constexpr (W > 1) {
            combine_waves<W>(slots, (int)(k & 1), w, lane, ta, tb, cin, carry);
        } else {
            carry = __builtin_fmaf(ta, carry, tb);
        }

        float c = __builtin_fmaf(ea, cin, eb);
        float dx[E], dg[E];
        if constexpr (!PLAIN) Elem<T>::unpack(cur.x, dg);  // dg[] starts as x_t
#pragma unroll
        for (int i = E - 1; i >= 0; --i) {
            const float delta = G[i] + c;
            c = __builtin_fmaf(g[i], c, p[i]);
            const float hp = (i > 0) ? h[i > 0 ? i - 1 : 0] : hprev0;
            if constexpr (PLAIN) {
                dx[i] = delta;
                dg[i] = hp * delta;
            } else {
                dx[i] = __builtin_fmaf(-g[i], delta, delta);
                dg[i] = (hp - dg[i]) * delta;
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

// ---- backward with the D and M sums inside -------------------------------------------
// For M > 1 and D > 1 the per-pair gradients are only ever summed: d_gates = sum over d,
// d_tokens = sum over m (reference fm/scan/fm_scan.py:76-78; its kernel writes both
// (B, M, D, L) tensors "to avoid atomicAdd", fm_scan.cuh:200-207, and torch.sum reads them
// back). This kernel never writes them. A block is one batch element b and DG
// consecutive d (one wave each). Its waves walk their rows from the end in chunks of C
// tiles; for a chunk they visit the M rows (b, m, d) one after the other and, in each, the
// C tiles of the chunk from the last to the first, all waves on the same step:
//   * token gradient: summed over m in registers (C tiles of accumulators), stored once
//     per chunk as d_tokens[b, d, :]
//   * gate gradient: the DG waves add their tiles up in LDS (one barrier per step) and
//     store the sum for this group of d, gate_partial[b, m, group, :] in float32; the
//     caller adds the ceil(D / DG) groups.
// Each wave keeps the running state of its M rows in LDS (one float per row). The visits
// (chunk, m) form one linear sequence; a ring holds the loads of the next R visits, and
// every step issues the same loads whatever its position (addresses are clamped into
// the row), so the number of loads in flight is known at compile time and a step waits
// for its own entry only. A larger C makes the pieces a wave reads from one row longer
// (C KiB at a time), which the memory likes, at C tiles of accumulators.
// HBM traffic: G and h once (2s per element) plus 4/DG bytes per element of partials,
// against 6s for the unfused kernel plus the two torch.sum passes. This kernel, unlike the two
// above, does depend on per-entry waits: its 8 waves meet at a barrier every tile, so a wave
// that waits for its newest loads stalls the block (measured: 0.75 -> 0.50 ms on the
// (1, 32, 2048, 8192) shape when the waits became per entry).
//
// LAYER: the gradient that arrives at the states is not read but made on the spot from what
// the layer around the scan holds (reference fm/scan/fm_scan.py:124-131 differentiated):
//   G[b,m,d,t] = coef_out[b,m,t] * layer_out_grad[b,d,t] - coef_self[b,m,t] * out_grad[b,m,d,t]
// where `out_grad` then carries the normalised states; the (B, M, D, L) gradient tensor is
// never written or read. LAYER == 2: the scanned states themselves are not read either
// (h_saved is NULL) but taken back from the normalised ones, h = out_grad * rms, so that
// the layer has to keep nothing of size (B, M, D, L) besides the states it returns.
template <typename T, int DG, int C, int R, bool PLAIN, int LAYER>
__global__ __launch_bounds__(64 * DG) void scan_backward_reduced_kernel(
    const T* __restrict__ gates, const T* __restrict__ out_grad, const T* __restrict__ first_prop_grad,
    T* __restrict__ token_grad /* (B, D, L) */, const T* __restrict__ h_saved,
    const T* __restrict__ tokens, float* __restrict__ gate_partial /* (B, M, NG, L) */,
    const T* __restrict__ h0, T* __restrict__ h0_grad, const T* __restrict__ coef_out /* (B, M, L) */,
    const T* __restrict__ coef_self /* (B, M, L) */, const T* __restrict__ layer_out_grad /* (B, D, L) */,
    const T* __restrict__ rms /* (B, M, L): 1 / inv_rms */, int32_t M, int32_t D, int64_t L) {
    constexpr int E = Elem<T>::E;
    constexpr int TILE = E * 64;
    constexpr int SLICE = TILE / DG;  // elements of a summed tile each wave adds up and stores
    constexpr bool HOIST = C <= 2;    // keep the chunk's tokens widened across its M rows
    static_assert(TILE % DG == 0, "a tile must split evenly over the waves");
    extern __shared__ float lds[];
    float* red = lds;                            // [2][DG][TILE]
    float* carries = lds + 2 * DG * TILE;        // [DG][M]

    const int lane = threadIdx.x & 63;
    const int w = uniform((int)(threadIdx.x >> 6));
    const int32_t NG = (D + DG - 1) / DG;
    // (the division runs on the vector unit; everything derived from b is an address, so
    // bring it back to a scalar register)
    // Blocks go to the 8 XCDs (each with its own L2) round robin. The blocks of one b read the
    // same gates (and coefficient vectors), so they are renumbered to share an XCD: XCD x takes
    // the x-th eighth of the (b, group) pairs.
    uint32_t id = blockIdx.x;
    if (gridDim.x % 8u == 0u) id = (id % 8u) * (gridDim.x / 8u) + id / 8u;
    const int32_t b32 = uniform((int)(id / (uint32_t)NG));
    const int64_t b = b32;
    const int32_t grp = uniform((int)id - b32 * NG);
    const bool active = grp * DG + w < D;        // a wave past the last d still joins every barrier
    const int64_t d = active ? grp * DG + w : D - 1;
    const int32_t ntiles = (int32_t)((L + TILE - 1) / TILE);
    const int32_t nchunks = (ntiles + C - 1) / C;
    const int64_t lane_off = (int64_t)(63 - lane) * E;
    float* mycarry = carries + w * M;

    for (int32_t m = lane; m < M; m += 64)
        mycarry[m] = first_prop_grad ? Elem<T>::widen(first_prop_grad[(b * M + m) * D + d]) : 0.0f;

    const T* __restrict__ xrow = tokens + (b * D + d) * L;  // never read when PLAIN
    const T* __restrict__ yrow = layer_out_grad + (b * D + d) * L;  // never read unless LAYER
    T* __restrict__ dxrow = token_grad + (b * D + d) * L;

    // What a step loads, exactly as it arrives: anything computed from a loaded value at
    // the time of the load would have to be finished before the loop comes round, which
    // means waiting for every load in flight. Fill values for chunks beyond L and the
    // choice of h[-1] are therefore applied when the entry is used.
    struct Entry {
        u32x4 g, G, h, x;
        u32x4 co, cs, y;  // LAYER only
        u32x4 rr;         // LAYER == 2: rms of the chunk's steps
        T hb;
        T hbr;            // LAYER == 2: rms at the step hb belongs to
    };
    // Where a visit is: chunk `chunk` of row (b, m, d), with the offsets that go with it
    // kept as running sums in scalar registers (a 64-bit product per step would run on the
    // vector unit, at a quarter of the rate).
    struct Cursor {
        int32_t chunk, m;
        int64_t row;   // (b * M + m) * D + d
        int64_t hoff;  // row * L: where the row starts in out_grad and h
        int64_t goff;  // (b * M + m) * L: in gates
        int64_t poff;  // ((b * M + m) * NG + grp) * L: in gate_partial
    };
    const int64_t row_step = D, hoff_step = (int64_t)D * L, goff_step = L, poff_step = (int64_t)NG * L;
    // the visit after: the next row at the same chunk, then row 0 of the chunk before
    auto advance = [&](Cursor& c) {
        const bool wrap = c.m + 1 == M;
        c.chunk = wrap ? c.chunk - 1 : c.chunk;
        c.m = wrap ? 0 : c.m + 1;
        c.row = uniform64(wrap ? c.row - (M - 1) * row_step : c.row + row_step);
        c.hoff = uniform64(wrap ? c.hoff - (M - 1) * hoff_step : c.hoff + hoff_step);
        c.goff = uniform64(wrap ? c.goff - (M - 1) * goff_step : c.goff + goff_step);
        c.poff = uniform64(wrap ? c.poff - (M - 1) * poff_step : c.poff + poff_step);
    };
    const int32_t lane_off32 = (63 - lane) * E;
    // tile i of the chunk; addresses are clamped into the row (a chunk before the first, or
    // a tile past the last, reads the nearest tile of the row)
    auto fetch = [&](Entry& e, const Cursor& c, int i) {
        int32_t k = c.chunk * C + i;
        k = k < 0 ? 0 : (k > ntiles - 1 ? ntiles - 1 : k);
        const int64_t tw = (int64_t)k * TILE;
        const int64_t left = L - tw;
        const int32_t rem = left < TILE ? (int32_t)left : TILE;
        const uint32_t loff = (uint32_t)(lane_off32 < rem ? lane_off32 : rem - E) * (uint32_t)sizeof(T);
        auto at = [&](const T* base) {  // scalar base + 32-bit lane offset
            return reinterpret_cast<const T*>(reinterpret_cast<const char*>(base) + loff);
        };
        // where h comes from: the saved states, or the normalised ones (LAYER == 2)
        const T* __restrict__ hrow = (LAYER == 2 ? out_grad : h_saved) + c.hoff;
        e.g = load16<T, false>(at(gates + c.goff + tw));
        e.G = load16<T, true>(at(out_grad + c.hoff + tw));
        e.h = u32x4{0u, 0u, 0u, 0u};
        if constexpr (LAYER != 2) e.h = load16<T, true>(at(hrow + tw));
        e.x = u32x4{0u, 0u, 0u, 0u};
        if constexpr (!PLAIN) e.x = load16<T, false>(at(xrow + tw));
        e.co = e.cs = e.y = u32x4{0u, 0u, 0u, 0u};
        if constexpr (LAYER != 0) {
            e.co = load16<T, false>(at(coef_out + c.goff + tw));
            e.cs = load16<T, false>(at(coef_self + c.goff + tw));
            e.y = load16<T, false>(at(yrow + tw));
        }
        e.rr = u32x4{0u, 0u, 0u, 0u};
        e.hbr = e.hb;
        if constexpr (LAYER == 2) {
            e.rr = load16<T, false>(at(rms + c.goff + tw));
            e.hbr = rms[c.goff + (tw > 0 ? tw - 1 : 0)];
        }
        // h just before the tile (h[-1] at the start of the row): one address for the whole wave
        const T* src = tw > 0 ? hrow + (tw - 1) : (h0 != nullptr ? h0 + c.row : hrow);
        e.hb = *src;
    };

    Entry q[R][C];
    Cursor ahead = {nchunks - 1, 0, uniform64(b * M * D + d), uniform64((b * M * D + d) * L),
                    uniform64(b * M * L), uniform64((b * M * NG + grp) * L)};
    Cursor at = ahead;
#pragma unroll
    for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int i = C - 1; i >= 0; --i) fetch(q[r][i], ahead, i);
        advance(ahead);
    }

    __syncthreads();  // carries are in place

    float dtok[C][E], xf[HOIST ? C : 1][E], yf[HOIST ? C : 1][E];
#pragma unroll
    for (int i = 0; i < C; ++i) {
#pragma unroll
        for (int j = 0; j < E; ++j) dtok[i][j] = 0.0f;
    }
#pragma unroll
    for (int i = 0; i < (HOIST ? C : 1); ++i) {
#pragma unroll
        for (int j = 0; j < E; ++j) xf[i][j] = yf[i][j] = 0.0f;
    }
    int parity = 0;
    const int32_t visits = nchunks * M;  // the host checks that this fits
    for (int32_t n = 0; n < visits; n += R) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            if (n + r >= visits) break;  // same for every wave of the block
            const int32_t m = at.m;
            float carry = mycarry[m];
#pragma unroll
            for (int i = C - 1; i >= 0; --i) {
                Entry cur = q[r][i];
                fetch(q[r][i], ahead, i);

                const int32_t k = at.chunk * C + i;  // may be past the last tile in the last chunk
                const int64_t tw = (int64_t)k * TILE;
                if (tw + TILE > L && tw + lane_off >= L) {  // short or absent tile: nothing there
                    cur.g = u32x4{Elem<T>::kOnes, Elem<T>::kOnes, Elem<T>::kOnes, Elem<T>::kOnes};
                    cur.G = cur.h = cur.x = cur.co = cur.cs = cur.y = u32x4{0u, 0u, 0u, 0u};
                    cur.rr = u32x4{0u, 0u, 0u, 0u};
                }
                float hb = (k > 0 || h0 != nullptr) ? Elem<T>::widen(cur.hb) : 0.0f;
                if constexpr (LAYER == 2) {
                    if (k > 0) hb *= Elem<T>::widen(cur.hbr);  // at k == 0 it is the initial state itself
                }
                float g[E], G[E], h[E], p[E], xs[E];
                Elem<T>::unpack(cur.g, g);
                Elem<T>::unpack(cur.G, G);
                Elem<T>::unpack(cur.h, h);
                if constexpr (!PLAIN) {
                    if constexpr (HOIST) {
                        if (m == 0) Elem<T>::unpack(cur.x, xf[i]);  // the M rows share their tokens
                    } else {
                        Elem<T>::unpack(cur.x, xs);
                    }
                }
                if constexpr (LAYER == 2) {  // h = normalised state * rms (G[] holds the normalised state)
                    float r[E];
                    Elem<T>::unpack(cur.rr, r);
#pragma unroll
                    for (int j = 0; j < E; ++j) h[j] = G[j] * r[j];
                }
                if constexpr (LAYER != 0) {
                    float co[E], cs[E], ys[E];
                    Elem<T>::unpack(cur.co, co);
                    Elem<T>::unpack(cur.cs, cs);
                    if constexpr (HOIST) {
                        if (m == 0) Elem<T>::unpack(cur.y, yf[i]);  // shared by the M rows, like the tokens
                    } else {
                        Elem<T>::unpack(cur.y, ys);
                    }
#pragma unroll
                    for (int j = 0; j < E; ++j) {
                        const float y = HOIST ? yf[HOIST ? i : 0][j] : ys[j];
                        G[j] = __builtin_fmaf(-cs[j], G[j], co[j] * y);  // G[] held the normalised state
                    }
                }
#pragma unroll
                for (int j = 0; j < E; ++j) p[j] = g[j] * G[j];
                float a = g[E - 1], bb = p[E - 1];
#pragma unroll
                for (int j = E - 2; j >= 0; --j) {
                    bb = __builtin_fmaf(g[j], bb, p[j]);
                    a *= g[j];
                }
                wave_scan_inclusive(a, bb);
                const float ea = dpp<kWaveShr1>(1.0f, a);
                const float eb = dpp<kWaveShr1>(0.0f, bb);
                const float ta = lane63(a), tb = lane63(bb);
                const float hprev0 = dpp<kWaveShl1>(hb, h[E - 1]);

                float c = __builtin_fmaf(ea, carry, eb);
                carry = __builtin_fmaf(ta, carry, tb);
                float dg[E];
#pragma unroll
                for (int j = E - 1; j >= 0; --j) {
                    const float delta = G[j] + c;
                    c = __builtin_fmaf(g[j], c, p[j]);
                    const float hp = (j > 0) ? h[j > 0 ? j - 1 : 0] : hprev0;
                    if constexpr (PLAIN) {
                        dtok[i][j] += delta;
                        dg[j] = hp * delta;
                    } else {
                        dtok[i][j] += __builtin_fmaf(-g[j], delta, delta);
                        const float x = HOIST ? xf[HOIST ? i : 0][j] : xs[j];
                        dg[j] = (hp - x) * delta;
                    }
                }
                if (!active) {  // whole wave: a wave past the last d adds nothing
#pragma unroll
                    for (int j = 0; j < E; ++j) dg[j] = 0.0f;
                }

                // add the gate gradient tiles of the DG waves: each wave lays its tile out in
                // memory order, then sums one slice of the tile over all waves and stores it
                float* mine = red + (parity * DG + w) * TILE + lane_off;
#pragma unroll
                for (int j = 0; j < E; j += 4)
                    *reinterpret_cast<float4*>(mine + j) = make_float4(dg[j], dg[j + 1], dg[j + 2], dg[j + 3]);
                __syncthreads();
                const float* all = red + parity * DG * TILE + w * SLICE;
                float* __restrict__ prow = gate_partial + at.poff + tw + w * SLICE;
                for (int e = lane; e < SLICE; e += 64) {
                    float sum = 0.0f;
#pragma unroll
                    for (int v = 0; v < DG; ++v) sum += all[v * TILE + e];
                    if (tw + w * SLICE + e < L) __builtin_nontemporal_store(sum, prow + e);
                }
                parity ^= 1;
            }
            if (lane == 0) mycarry[m] = carry;

            if (m + 1 == M) {  // the chunk's token gradient is complete
#pragma unroll
                for (int i = 0; i < C; ++i) {
                    const int64_t t0 = (int64_t)(at.chunk * C + i) * TILE + lane_off;
                    if (active) store_chunk<T, true>(dxrow, t0, L, Elem<T>::pack(dtok[i]));
#pragma unroll
                    for (int j = 0; j < E; ++j) dtok[i][j] = 0.0f;
                }
            }
            advance(at);
            advance(ahead);
        }
    }

    if (h0_grad && active) {
        __builtin_amdgcn_wave_barrier();  // lane 0's carry writes precede the reads below
        for (int32_t mm = lane; mm < M; mm += 64) {
            float v[E] = {mycarry[mm]};
            const u32x4 packed = Elem<T>::pack(v);
            const int64_t row = (b * M + mm) * D + d;
            if constexpr (sizeof(T) == 4) reinterpret_cast<uint32_t*>(h0_grad)[row] = packed.x;
            else reinterpret_cast<uint16_t*>(h0_grad)[row] = (uint16_t)(packed.x & 0xffffu);
        }
    }
}

}  // namespace fmscan
