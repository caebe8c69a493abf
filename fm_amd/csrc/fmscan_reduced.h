// The backward scan of Factorization-Memory shapes (M > 1 and D > 1) with the sums over D
// and M inside, and its forms for the layer around the scan. Building blocks (rows,
// lanes, the wave scan): fmscan_kernels.h, fmscan_device.h.
#pragma once

#include "fmscan_kernels.h"

namespace fmscan {

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
        e.hbr = T(0);
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
