// The two scan kernels. A row is one (b, m, d) sequence of length L. W waves
// cooperate on one row: a tile is W*64 chunks of 16 bytes, consecutive in memory,
// one chunk per lane. Tiles of a row are walked serially (forward: first to
// last; backward: last to first) with the running state of the row in a
// register, so a row of any length costs one read of every input and one write
// of every output.
//
// Per tile a lane (1) folds its chunk into one (a, b) step pair, (2) the wave
// scans the 64 pairs with DPP, (3) with W > 1 the wave totals meet in LDS,
// (4) the lane replays its chunk from the state that enters it and stores.
// The chain that links one tile to the next is a single fma on the row state, so
// the loads of the following tiles (issued two tiles ahead) and the scan of the
// next tile overlap with the current one.
#pragma once

#include "fmscan_device.h"

namespace fmscan {

// Output row r = (b*M + m)*D + d  ->  gate row b*M + m, token row b*D + d
// (reference fm/scan/fm_scan.cuh:76-82).
struct RowMap {
    int64_t gate_row, token_row;
};
__device__ __forceinline__ RowMap map_row(int64_t r, int32_t M, int32_t D) {
    RowMap m;
    m.gate_row = r / D;
    const int64_t b = m.gate_row / M;
    m.token_row = b * D + (r - m.gate_row * D);
    return m;
}

// Meets the W wave totals of one tile in LDS. `cin` leaves as the state that
// enters this wave's part of the tile, `carry` as the state after the tile.
// Slots alternate between consecutive tiles, so one barrier per tile is enough:
// a wave can only overwrite a slot after every wave has passed the barrier of
// the tile in between, i.e. has finished reading it.
template <int W>
__device__ __forceinline__ void combine_waves(float2 (*slots)[W], int tile_parity, int w, int lane,
                                              float ta, float tb, float& cin, float& carry) {
    if (lane == 63) slots[tile_parity][w] = make_float2(ta, tb);
    __syncthreads();
    float c = carry;
    cin = carry;
#pragma unroll
    for (int j = 0; j < W; ++j) {
        const float2 p = slots[tile_parity][j];
        c = __builtin_fmaf(p.x, c, p.y);
        if (j + 1 == w) cin = c;
    }
    carry = c;
}

// ---- forward ------------------------------------------------------------------------
// h_t = g_t h_{t-1} + u_t,  u_t = (1 - g_t) x_t  (PLAIN: u_t = x_t)
// reference fm/scan/fm_scan.cuh:110,116,121-131,139-140; fm/scan/fm_pytorch.py:22,37.
template <typename T, int W, int R, bool PLAIN, bool VEC>
__global__ __launch_bounds__(64 * W * R) void scan_forward_kernel(
    const T* __restrict__ gates, const T* __restrict__ tokens, const T* __restrict__ h0,
    T* __restrict__ out, int64_t rows, int32_t M, int32_t D, int64_t L) {
    static_assert(W == 1 || R == 1, "waves that share a barrier must share a row");
    constexpr int E = Elem<T>::E;
    constexpr int64_t TILE = (int64_t)E * 64 * W;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int w = wave % W;
    const int64_t r = (int64_t)blockIdx.x * R + wave / W;
    if (r >= rows) return;  // whole waves only, and only in barrier-free (W == 1) blocks

    __shared__ float2 slots[2][W];

    const RowMap rm = map_row(r, M, D);
    const T* __restrict__ grow = gates + rm.gate_row * L;
    const T* __restrict__ xrow = tokens + rm.token_row * L;
    T* __restrict__ orow = out + r * L;
    float carry = h0 ? Elem<T>::widen(h0[r]) : 0.0f;

    const int64_t lane_off = (int64_t)(w * 64 + lane) * E;
    const int64_t ntiles = (L + TILE - 1) / TILE;

    u32x4 g_n0 = load_chunk<T, VEC>(grow, lane_off, L, Elem<T>::kOnes);
    u32x4 x_n0 = load_chunk<T, VEC>(xrow, lane_off, L, 0u);
    u32x4 g_n1 = load_chunk<T, VEC>(grow, TILE + lane_off, L, Elem<T>::kOnes);
    u32x4 x_n1 = load_chunk<T, VEC>(xrow, TILE + lane_off, L, 0u);

    for (int64_t k = 0; k < ntiles; ++k) {
        const int64_t t0 = k * TILE + lane_off;
        const u32x4 g_raw = g_n0, x_raw = x_n0;
        g_n0 = g_n1;
        x_n0 = x_n1;
        g_n1 = load_chunk<T, VEC>(grow, t0 + 2 * TILE, L, Elem<T>::kOnes);
        x_n1 = load_chunk<T, VEC>(xrow, t0 + 2 * TILE, L, 0u);

        float g[E], u[E];
        Elem<T>::unpack(g_raw, g);
        Elem<T>::unpack(x_raw, u);
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
        store_chunk<T, VEC>(orow, t0, L, Elem<T>::pack(o));
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
template <typename T, int W, int R, bool PLAIN, bool VEC>
__global__ __launch_bounds__(64 * W * R) void scan_backward_kernel(
    const T* __restrict__ gates, const T* __restrict__ out_grad, const T* __restrict__ first_prop_grad,
    T* __restrict__ token_grad, const T* __restrict__ h_saved, const T* __restrict__ tokens,
    T* __restrict__ gate_grad, const T* __restrict__ h0, int64_t rows, int32_t M, int32_t D,
    int64_t L) {
    static_assert(W == 1 || R == 1, "waves that share a barrier must share a row");
    constexpr int E = Elem<T>::E;
    constexpr int64_t TILE = (int64_t)E * 64 * W;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int w = wave % W;
    const int64_t r = (int64_t)blockIdx.x * R + wave / W;
    if (r >= rows) return;

    __shared__ float2 slots[2][W];

    const RowMap rm = map_row(r, M, D);
    const T* __restrict__ grow = gates + rm.gate_row * L;
    const T* __restrict__ Grow = out_grad + r * L;
    const T* __restrict__ hrow = h_saved + r * L;
    const T* __restrict__ xrow = tokens + rm.token_row * L;  // never read when PLAIN
    T* __restrict__ dxrow = token_grad + r * L;
    T* __restrict__ dgrow = gate_grad + r * L;
    float carry = first_prop_grad ? Elem<T>::widen(first_prop_grad[r]) : 0.0f;
    const float hinit = h0 ? Elem<T>::widen(h0[r]) : 0.0f;

    const int64_t lane_off = (int64_t)(64 * W - 1 - (w * 64 + lane)) * E;
    const int64_t ntiles = (L + TILE - 1) / TILE;

    struct Tile {
        u32x4 g, G, h, x;
        float hb;  // lane 63 only: h just before this wave's part of the tile
    };
    auto fetch = [&](int64_t k, Tile& q) {
        const int64_t t0 = k * TILE + lane_off;  // k < 0 never loads: t0 < 0 is tested below
        const bool live = k >= 0;
        q.g = load_chunk<T, VEC>(grow, live ? t0 : L, L, Elem<T>::kOnes);
        q.G = load_chunk<T, VEC>(Grow, live ? t0 : L, L, 0u);
        q.h = load_chunk<T, VEC>(hrow, live ? t0 : L, L, 0u);
        if constexpr (!PLAIN) q.x = load_chunk<T, VEC>(xrow, live ? t0 : L, L, 0u);
        q.hb = hinit;
        if (live && lane == 63 && t0 > 0 && t0 < L) q.hb = Elem<T>::widen(hrow[t0 - 1]);
    };

    Tile q0, q1;
    fetch(ntiles - 1, q0);
    fetch(ntiles - 2, q1);

    for (int64_t k = ntiles - 1; k >= 0; --k) {
        const int64_t t0 = k * TILE + lane_off;
        const Tile cur = q0;
        q0 = q1;
        fetch(k - 2, q1);

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
        // in memory, which the next lane holds; lane 63 fetched it (or h[-1]) itself.
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
        store_chunk<T, VEC>(dxrow, t0, L, Elem<T>::pack(dx));
        store_chunk<T, VEC>(dgrow, t0, L, Elem<T>::pack(dg));
    }
}

}  // namespace fmscan
