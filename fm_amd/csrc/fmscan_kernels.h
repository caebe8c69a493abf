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
// The chain that links one tile to the next is a single fma on the row state.
//
// A wave keeps the loads of the next P tiles of its row in flight while it scans the
// current one. The grid has one block per row (W > 1) or per R rows (W == 1); the
// host bounds how many blocks a compute unit holds at a time, because the HBM
// efficiency of this access pattern depends on how many rows stream concurrently.
#pragma once

#include "fmscan_device.h"

namespace fmscan {

__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }

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
    m.gate_row = gate_row;
    m.token_row = (int64_t)b * D + (r - gate_row * (uint32_t)D);
    return m;
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
    T* __restrict__ out, int64_t rows, int32_t M, int32_t D, int64_t L) {
    static_assert(W == 1 || R == 1, "waves that share a barrier must share a row");
    constexpr int E = Elem<T>::E;
    constexpr int64_t TILE = (int64_t)E * 64 * W;
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
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

    struct Entry {
        u32x4 g, x;
    };
    auto fetch = [&](Entry& q, int64_t k) {  // k >= ntiles loads nothing
        const int64_t t0 = k * TILE + lane_off;
        q.g = load_chunk<T, VEC, FOLD>(grow, t0, L, Elem<T>::kOnes);
        q.x = load_chunk<T, VEC, FOLD>(xrow, t0, L, 0u);
    };

    Entry q[P];
#pragma unroll
    for (int s = 0; s < P; ++s) fetch(q[s], s);

    for (int64_t k0 = 0; k0 < ntiles; k0 += P) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
            const int64_t k = k0 + s;
            if (k >= ntiles) break;
            const Entry cur = q[s];
            fetch(q[s], k + P);
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
            store_chunk<T, VEC>(orow, t0, L, Elem<T>::pack(o));
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
    T* __restrict__ gate_grad, const T* __restrict__ h0, int64_t rows, int32_t M, int32_t D,
    int64_t L) {
    static_assert(W == 1 || R == 1, "waves that share a barrier must share a row");
    constexpr int E = Elem<T>::E;
    constexpr int64_t TILE = (int64_t)E * 64 * W;
    const int lane = threadIdx.x & 63;
    const int wave = uniform(threadIdx.x >> 6);
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

    struct Entry {
        u32x4 g, G, h, x;
        float hb;  // lane 63 only: h just before this wave's part of the tile (h[-1] at t = 0)
    };
    auto fetch = [&](Entry& q, int64_t k) {
        // k < 0 (before the row): t0 = L, which every bound check below rejects
        const int64_t t0 = k >= 0 ? k * TILE + lane_off : L;
        q.g = load_chunk<T, VEC, FOLD>(grow, t0, L, Elem<T>::kOnes);
        q.G = load_chunk<T, VEC, true>(Grow, t0, L, 0u);
        q.h = load_chunk<T, VEC, true>(hrow, t0, L, 0u);
        if constexpr (!PLAIN) q.x = load_chunk<T, VEC, FOLD>(xrow, t0, L, 0u);
        q.hb = hinit;
        if (lane == 63 && t0 > 0 && t0 < L) q.hb = Elem<T>::widen(hrow[t0 - 1]);
    };

    Entry q[P];
#pragma unroll
    for (int s = 0; s < P; ++s) fetch(q[s], ntiles - 1 - s);

    for (int64_t k0 = ntiles - 1; k0 >= 0; k0 -= P) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
            const int64_t k = k0 - s;
            if (k < 0) break;
            const Entry cur = q[s];
            fetch(q[s], k - P);
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
}

}  // namespace fmscan
