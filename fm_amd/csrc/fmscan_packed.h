// The scan kernels for short rows: several rows per wave.
//
// The general kernels (fmscan_kernels.h) give a wave one row at a time, a chunk of 16 bytes per lane, so a
// row of fewer than 64 chunks leaves lanes without work (a row of 128 bytes: 56 of 64). Here a row of CL
// chunks (CL <= 64) takes a group of LPR lanes, LPR the power of two at or above CL, and a wave holds
// 64 / LPR consecutive rows: its accesses still cover one contiguous stretch of memory. The wave scan
// runs inside each group (a segmented scan): four shifted steps inside the 16-lane rows that DPP knows, a
// fifth and a sixth that hand the total of a 16-lane row to the one after it and of the first 32 lanes to
// the other 32 when a group is that wide; a lane takes a step only when the source lane belongs to its own
// group, by selection and not by multiplying with zero, so that a row's result never depends on its
// neighbours' values (NaN and infinity included) and is the same bit for bit wherever the row sits in the
// wave.
//
// Rows of whole 16-byte vectors at aligned addresses move as such (VEC); any other row of up to 64 chunks
// with accesses at the alignment of an element and a ragged last chunk. One tile per row: no loop, no LDS,
// no workspace. Arithmetic as in the general kernels (float32, one fma per step); the
// backward kernel reads the saved states (a fourth stream) instead of making them again.
#pragma once

#include "fmscan_kernels.h"

namespace fmscan {

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ void segmented_level(float& a, float& b, bool take) {
    const float as = dpp<CTRL, ROW_MASK>(1.0f, a);
    const float bs = dpp<CTRL, ROW_MASK>(0.0f, b);
    const float nb = __builtin_fmaf(bs, a, b);  // the pair of the lanes before, then this lane's
    const float na = a * as;
    b = take ? nb : b;
    a = take ? na : a;
}

// On entry lane l holds the step pair of its chunk; on exit the composition of the chunks of its group
// from the group's first lane to l. `p` is the lane's place in its group (groups are aligned powers of two).
__device__ __forceinline__ void group_scan_inclusive(float& a, float& b, int p) {
    segmented_level<0x111, 0xf>(a, b, p >= 1);   // row_shr:1
    segmented_level<0x112, 0xf>(a, b, p >= 2);   // row_shr:2
    segmented_level<0x114, 0xf>(a, b, p >= 4);   // row_shr:4
    segmented_level<0x118, 0xf>(a, b, p >= 8);   // row_shr:8
    segmented_level<0x142, 0xa>(a, b, p >= 16);  // row_bcast:15 into the 16-lane rows 1 and 3
    segmented_level<0x143, 0xc>(a, b, p >= 32);  // row_bcast:31 into the 16-lane rows 2 and 3
}

// The chunk at position t0 of a row. VEC: rows are whole 16-byte vectors at 16-byte aligned addresses.
// Otherwise a row starts wherever an element may, and its last chunk may be ragged: whole chunks move as
// one access at the alignment of an element, the ragged one element by element, positions past the end as `fill`.
template <typename T, bool VEC, bool ONCE>
__device__ __forceinline__ u32x4 packed_load(const T* __restrict__ row, int32_t t0, int32_t L, uint32_t fill) {
    if constexpr (VEC) return load16<T, ONCE>(row + t0);
    else return load_chunk<T, false, ONCE>(row, t0, L, fill);
}

// Where a lane works: its row, its place in the group, the chunk it owns.
struct PackedLane {
    int64_t row;      // clamped to the last row for lanes without one (they load it and drop it)
    int64_t gate_row, token_row;
    int32_t p;        // place in the group
    bool has_row;     // the group has a row
};
template <bool FOLD>
__device__ __forceinline__ PackedLane locate_packed(int64_t rows, int32_t M, int32_t D, int32_t lpr_log2) {
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    PackedLane q;
    q.p = lane & ((1 << lpr_log2) - 1);
    const int64_t row = (wave << (6 - lpr_log2)) + (lane >> lpr_log2);
    q.has_row = row < rows;
    q.row = q.has_row ? row : rows - 1;
    if constexpr (FOLD) {
        q.gate_row = q.token_row = q.row;
    } else {
        const uint32_t r = (uint32_t)q.row;  // rows < 2^31 is checked by the host
        const uint32_t gate_row = r / (uint32_t)D;
        const uint32_t b = gate_row / (uint32_t)M;
        q.gate_row = gate_row;
        q.token_row = (int64_t)b * D + (r - gate_row * (uint32_t)D);
    }
    return q;
}

// h_t = g_t h_{t-1} + u_t,  u_t = (1 - g_t) x_t  (PLAIN: u_t = x_t); see scan_forward_kernel.
template <typename T, bool PLAIN, bool VEC, bool FOLD>
__global__ __launch_bounds__(256) void scan_forward_packed_kernel(
    const T* __restrict__ gates, const T* __restrict__ tokens, const T* __restrict__ h0, T* __restrict__ out,
    int64_t rows, int32_t M, int32_t D, int32_t L, int32_t lpr_log2) {
    constexpr int E = Elem<T>::E;
    const int32_t CL = (L + E - 1) / E;  // chunks per row (VEC: all whole)
    if ((((int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) << (6 - lpr_log2)) >= rows) return;  // whole waves
    const PackedLane q = locate_packed<FOLD>(rows, M, D, lpr_log2);
    const bool active = q.has_row && q.p < CL;
    const int32_t t0 = (q.p < CL ? q.p : CL - 1) * E;
    u32x4 gq = packed_load<T, VEC, FOLD>(gates + q.gate_row * L, t0, L, Elem<T>::kOnes);
    u32x4 xq = packed_load<T, VEC, FOLD>(tokens + q.token_row * L, t0, L, 0u);
    const float hin = (h0 && q.p == 0) ? Elem<T>::widen(h0[q.row]) : 0.0f;
    if (!active) {  // identity steps
        gq = u32x4{Elem<T>::kOnes, Elem<T>::kOnes, Elem<T>::kOnes, Elem<T>::kOnes};
        xq = u32x4{0u, 0u, 0u, 0u};
    }
    float g[E], u[E];
    Elem<T>::unpack(gq, g);
    Elem<T>::unpack(xq, u);
    if constexpr (!PLAIN) {
#pragma unroll
        for (int i = 0; i < E; ++i) u[i] = __builtin_fmaf(-g[i], u[i], u[i]);  // (1-g)x, one rounding
    }
    float a = g[0], b = u[0];
#pragma unroll
    for (int i = 1; i < E; ++i) {
        b = __builtin_fmaf(g[i], b, u[i]);
        a *= g[i];
    }
    if (q.p == 0) b = __builtin_fmaf(a, hin, b);  // the state before the row enters the group's first chunk
    group_scan_inclusive(a, b, q.p);
    const float before = dpp<kWaveShr1>(0.0f, b);  // the state after the chunk of the lane before
    float h = q.p == 0 ? hin : before;
    float o[E];
#pragma unroll
    for (int i = 0; i < E; ++i) {
        h = __builtin_fmaf(g[i], h, u[i]);
        o[i] = h;
    }
    if (active) store_chunk<T, VEC>(out + q.row * L, t0, L, Elem<T>::pack(o));
}

// delta_t = G_t + g_{t+1} delta_{t+1}; token_grad_t = (1 - g_t) delta_t, gate_grad_t = (h_{t-1} - x_t) delta_t
// (PLAIN: delta_t, h_{t-1} delta_t); see scan_backward_kernel. The lanes of a group take the row's chunks
// from the last to the first, so the suffix scan in memory order is a prefix scan in lane order.
template <typename T, bool PLAIN, bool VEC, bool FOLD>
__global__ __launch_bounds__(256) void scan_backward_packed_kernel(
    const T* __restrict__ gates, const T* __restrict__ out_grad, const T* __restrict__ first_prop_grad,
    T* __restrict__ token_grad, const T* __restrict__ h_saved, const T* __restrict__ tokens,
    T* __restrict__ gate_grad, const T* __restrict__ h0, T* __restrict__ h0_grad, int64_t rows, int32_t M,
    int32_t D, int32_t L, int32_t lpr_log2) {
    constexpr int E = Elem<T>::E;
    const int32_t CL = (L + E - 1) / E;
    if ((((int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6)) << (6 - lpr_log2)) >= rows) return;
    const PackedLane q = locate_packed<FOLD>(rows, M, D, lpr_log2);
    const bool active = q.has_row && q.p < CL;
    const int32_t c = q.p < CL ? CL - 1 - q.p : 0;  // the chunk of this lane, counted from the row's start
    const int32_t t0 = c * E;
    u32x4 gq = packed_load<T, VEC, FOLD>(gates + q.gate_row * L, t0, L, Elem<T>::kOnes);
    u32x4 Gq = packed_load<T, VEC, true>(out_grad + q.row * L, t0, L, 0u);
    const u32x4 hq = packed_load<T, VEC, true>(h_saved + q.row * L, t0, L, 0u);
    u32x4 xq = u32x4{0u, 0u, 0u, 0u};
    if constexpr (!PLAIN) xq = packed_load<T, VEC, FOLD>(tokens + q.token_row * L, t0, L, 0u);
    const float cinit = (first_prop_grad && q.p == 0) ? Elem<T>::widen(first_prop_grad[q.row]) : 0.0f;
    const float hinit = (h0 && c == 0) ? Elem<T>::widen(h0[q.row]) : 0.0f;
    if (!active) {
        gq = u32x4{Elem<T>::kOnes, Elem<T>::kOnes, Elem<T>::kOnes, Elem<T>::kOnes};
        Gq = u32x4{0u, 0u, 0u, 0u};
    }
    float g[E], G[E], pr[E], h[E];
    Elem<T>::unpack(gq, g);
    Elem<T>::unpack(Gq, G);
    Elem<T>::unpack(hq, h);
#pragma unroll
    for (int i = 0; i < E; ++i) pr[i] = g[i] * G[i];
    // the chunk as one step on the part of delta that arrives from the future: c_out = a*c_in + b
    float a = g[E - 1], b = pr[E - 1];
#pragma unroll
    for (int i = E - 2; i >= 0; --i) {
        b = __builtin_fmaf(g[i], b, pr[i]);
        a *= g[i];
    }
    if (q.p == 0) b = __builtin_fmaf(a, cinit, b);  // what arrives at the end of the row
    group_scan_inclusive(a, b, q.p);
    const float before = dpp<kWaveShr1>(0.0f, b);
    float cc = q.p == 0 ? cinit : before;
    // what is left after the first step is g_0 * delta_0: the gradient of the state before the row
    if (h0_grad && active && c == 0) {
        float v[E] = {b};
        const u32x4 packed = Elem<T>::pack(v);
        if constexpr (sizeof(T) == 4) reinterpret_cast<uint32_t*>(h0_grad)[q.row] = packed.x;
        else reinterpret_cast<uint16_t*>(h0_grad)[q.row] = (uint16_t)(packed.x & 0xffffu);
    }
    // hp[i] = the state before element i: the last element of the chunk before this one in memory is with
    // the next lane; the row's first chunk takes the state before the row
    float hp[E];
    const float behind = dpp<kWaveShl1>(0.0f, h[E - 1]);
    hp[0] = c == 0 ? hinit : behind;
#pragma unroll
    for (int i = 1; i < E; ++i) hp[i] = h[i - 1];
    float x[E];
    if constexpr (!PLAIN) Elem<T>::unpack(xq, x);
    float dx[E], dg[E];
#pragma unroll
    for (int i = E - 1; i >= 0; --i) {
        const float delta = G[i] + cc;
        cc = __builtin_fmaf(g[i], cc, pr[i]);
        if constexpr (PLAIN) {
            dx[i] = delta;
            dg[i] = hp[i] * delta;
        } else {
            dx[i] = __builtin_fmaf(-g[i], delta, delta);
            dg[i] = (hp[i] - x[i]) * delta;
        }
    }
    if (active) {
        store_chunk<T, VEC>(token_grad + q.row * L, t0, L, Elem<T>::pack(dx));
        store_chunk<T, VEC>(gate_grad + q.row * L, t0, L, Elem<T>::pack(dg));
    }
}

// ---- backward with the sums inside, for short rows ---------------------------------------------------
// What scan_backward_packed_kernel computes, summed as the reference sums it afterwards (fm_scan.py:76-78):
// the token gradient over the M slots and the gate gradient over the D rows of a slot, in float32. A wave
// is a batch element b and a tile of 64 >> lpr_log2 consecutive rows d, and walks the M slots: the token
// gradient of its rows adds up in registers and is stored once; the gate gradient of a slot is added
// across the wave's groups (the halves of the wave, then the 16-lane rows, trade the values the other is
// to keep; rotations inside the rows finish) and stored as one of G = ceil(D / rows of a tile) float32
// partial sums, gate_grad_partial (B * M, G, L), which fmscan_sum_groups adds. No LDS, no barrier; the
// loads of the next slot are in flight while a slot is worked on. Sums are taken in a fixed order.
// v + (v of the lane 16 or 32 away): the two halves change places in a copy and meet in an add
template <int AWAY>
__device__ __forceinline__ float add_across(float v) {
    uint32_t mine = f2u(v), copy;
    asm volatile("v_mov_b32 %0, %1" : "=v"(copy) : "v"(mine));  // a copy the compiler cannot identify with `mine`
    if constexpr (AWAY == 32) {
        const auto r = __builtin_amdgcn_permlane32_swap(mine, copy, false, false);
        return u2f(r[0]) + u2f(r[1]);
    } else {
        const auto r = __builtin_amdgcn_permlane16_swap(mine, copy, false, false);
        return u2f(r[0]) + u2f(r[1]);
    }
}

// Every lane's E values summed over the lanes that hold the same chunk in the wave's other groups
// (groups are 1 << lpr_log2 lanes, at most 16): rotations inside the 16-lane rows, then the two exchanges
// across them. Every lane ends with the sum.
template <int E>
__device__ __forceinline__ void sum_over_groups(float (&v)[E], int32_t lpr_log2) {
    if (lpr_log2 <= 3) {
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] += dpp<0x128, 0xf>(v[e], v[e]);  // row_ror:8
    }
    if (lpr_log2 <= 2) {
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] += dpp<0x124, 0xf>(v[e], v[e]);  // row_ror:4
    }
    if (lpr_log2 <= 1) {
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] += dpp<0x122, 0xf>(v[e], v[e]);  // row_ror:2
    }
    if (lpr_log2 <= 0) {
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] += dpp<0x121, 0xf>(v[e], v[e]);  // row_ror:1
    }
#pragma unroll
    for (int e = 0; e < E; ++e) v[e] = add_across<32>(add_across<16>(v[e]));
}

// LAYER (as in scan_backward_reduced_kernel): the gradient that arrives at the states is made on the spot,
//   G[b,m,d,t] = coef_out[b,m,t] * layer_out_grad[b,d,t] - coef_self[b,m,t] * out_grad[b,m,d,t],
// `out_grad` then carrying the normalised states; LAYER == 2: the scanned states are not read either but
// taken back from the normalised ones, h = out_grad * rms (h_saved is NULL). coef_out, coef_self, rms: float32.
template <typename T, bool PLAIN, int LAYER>
__global__ __launch_bounds__(256) void scan_backward_reduced_packed_kernel(
    const T* __restrict__ gates, const T* __restrict__ out_grad, const T* __restrict__ first_prop_grad,
    T* __restrict__ token_grad /* (B, D, L) */, const T* __restrict__ h_saved, const T* __restrict__ tokens,
    float* __restrict__ gate_grad_partial /* (B * M, G, L) */, const T* __restrict__ h0, T* __restrict__ h0_grad,
    const float* __restrict__ coef_out, const float* __restrict__ coef_self, const T* __restrict__ layer_out_grad,
    const float* __restrict__ rms, int32_t B, int32_t M, int32_t D, int32_t L, int32_t lpr_log2, int32_t G) {
    static_assert(LAYER == 0 || !PLAIN, "the layer's scan is the Factorization-Memory form");
    constexpr int E = Elem<T>::E;
    const int32_t CL = L / E;  // rows are whole 16-byte vectors
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + uniform((int)(threadIdx.x >> 6));
    if (wave >= (int64_t)B * G) return;  // whole waves
    const int32_t b = uniform((int)(wave / G));
    const int32_t tile = uniform((int)(wave - (int64_t)b * G));
    const int32_t p = lane & ((1 << lpr_log2) - 1);
    const int32_t group = lane >> lpr_log2;
    const int32_t d_mine = (tile << (6 - lpr_log2)) + group;
    const bool active = d_mine < D && p < CL;
    const int32_t d = d_mine < D ? d_mine : D - 1;            // lanes without a row load the last one and drop it
    const int32_t c = p < CL ? CL - 1 - p : 0;                // the chunk of this lane, counted from the row's start
    const int32_t t0 = c * E;
    const int64_t token_row = (int64_t)b * D + d;

    float x[E];
    if constexpr (!PLAIN) Elem<T>::unpack(load16<T, false>(tokens + token_row * L + t0), x);
    [[maybe_unused]] float y[E];  // LAYER: the gradient of the layer's output at this row
    if constexpr (LAYER != 0) Elem<T>::unpack(load16<T, false>(layer_out_grad + token_row * L + t0), y);
    float dtok[E];
#pragma unroll
    for (int e = 0; e < E; ++e) dtok[e] = 0.0f;

    struct In {
        u32x4 g, G;
        u32x4 h;                    // LAYER != 2: the saved states
        FloatChunk<E> co, cs, rr;   // LAYER; rr: LAYER == 2
        float cinit, hinit;
    };
    auto fetch = [&](In& n, int32_t m) {
        const int64_t gate_row = (int64_t)b * M + m;
        const int64_t row = gate_row * D + d;
        n.g = load16<T, false>(gates + gate_row * L + t0);
        n.G = load16<T, true>(out_grad + row * L + t0);
        if constexpr (LAYER != 2) n.h = load16<T, true>(h_saved + row * L + t0);
        if constexpr (LAYER != 0) {
            n.co = load_float_chunk<E>(coef_out + gate_row * L + t0);
            n.cs = load_float_chunk<E>(coef_self + gate_row * L + t0);
        }
        if constexpr (LAYER == 2) n.rr = load_float_chunk<E>(rms + gate_row * L + t0);
        n.cinit = (first_prop_grad && p == 0) ? Elem<T>::widen(first_prop_grad[row]) : 0.0f;
        n.hinit = (h0 && c == 0) ? Elem<T>::widen(h0[row]) : 0.0f;
    };
    In cur, next;
    fetch(cur, 0);
    for (int32_t m = 0; m < M; ++m) {
        fetch(next, m + 1 < M ? m + 1 : m);
        const int64_t gate_row = (int64_t)b * M + m;
        float g[E], Gv[E], pr[E], h[E];
        Elem<T>::unpack(cur.g, g);
        Elem<T>::unpack(cur.G, Gv);
        if constexpr (LAYER == 2) {
#pragma unroll
            for (int e = 0; e < E; ++e) h[e] = Gv[e];  // the normalised states; their factor follows below
        } else {
            Elem<T>::unpack(cur.h, h);
        }
        if constexpr (LAYER != 0) {
            float co[E], cs[E];
            spread<E>(cur.co, co);
            spread<E>(cur.cs, cs);
#pragma unroll
            for (int e = 0; e < E; ++e) Gv[e] = __builtin_fmaf(-cs[e], Gv[e], co[e] * y[e]);
        }
        if (!active) {  // identity steps
#pragma unroll
            for (int e = 0; e < E; ++e) {
                g[e] = 1.0f;
                Gv[e] = 0.0f;
            }
        }
#pragma unroll
        for (int e = 0; e < E; ++e) pr[e] = g[e] * Gv[e];
        float a = g[E - 1], bb = pr[E - 1];
#pragma unroll
        for (int e = E - 2; e >= 0; --e) {
            bb = __builtin_fmaf(g[e], bb, pr[e]);
            a *= g[e];
        }
        if (p == 0) bb = __builtin_fmaf(a, cur.cinit, bb);  // what arrives at the end of the row
        group_scan_inclusive(a, bb, p);
        const float before = dpp<kWaveShr1>(0.0f, bb);
        float cc = p == 0 ? cur.cinit : before;
        if (h0_grad && active && c == 0) {  // g_0 * delta_0: the gradient of the state before the row
            float v[E] = {bb};
            const u32x4 packed = Elem<T>::pack(v);
            const int64_t row = gate_row * D + d;
            if constexpr (sizeof(T) == 4) reinterpret_cast<uint32_t*>(h0_grad)[row] = packed.x;
            else reinterpret_cast<uint16_t*>(h0_grad)[row] = (uint16_t)(packed.x & 0xffffu);
        }
        // hp[e] = the state before element e: the last element of the chunk before this one in memory is with
        // the next lane; the row's first chunk takes the state before the row
        const float behind = dpp<kWaveShl1>(0.0f, h[E - 1]);
        float hp[E];
        hp[0] = behind;
#pragma unroll
        for (int e = 1; e < E; ++e) hp[e] = h[e - 1];
        if constexpr (LAYER == 2) {  // h = normalised state * rms, each at the step before
            float rr[E];
            spread<E>(cur.rr, rr);
            const float rr_behind = dpp<kWaveShl1>(1.0f, rr[E - 1]);
            hp[0] *= rr_behind;
#pragma unroll
            for (int e = 1; e < E; ++e) hp[e] *= rr[e - 1];
        }
        if (c == 0) hp[0] = cur.hinit;  // the state before the row, as it is
        float dg[E];
#pragma unroll
        for (int e = E - 1; e >= 0; --e) {
            const float delta = Gv[e] + cc;
            cc = __builtin_fmaf(g[e], cc, pr[e]);
            float mine;
            if constexpr (PLAIN) {
                dtok[e] += delta;
                mine = hp[e] * delta;
            } else {
                dtok[e] = __builtin_fmaf(-g[e], delta, dtok[e] + delta);
                mine = (hp[e] - x[e]) * delta;
            }
            dg[e] = active ? mine : 0.0f;
        }
        // The sum over the wave's groups, each quarter of the wave ending with a quarter of the values: the
        // halves of the wave, then the 16-lane rows of a half, trade what the other is to keep (one exchange
        // and one add per pair of values), and only what is left is summed inside the 16-lane rows.
        float kept[E / 4];
        {
            float half[E / 2];
#pragma unroll
            for (int e = 0; e < E / 2; ++e) {
                const auto r = __builtin_amdgcn_permlane32_swap(f2u(dg[e]), f2u(dg[e + E / 2]), false, false);
                half[e] = u2f(r[0]) + u2f(r[1]);  // lanes 0-31: value e, lanes 32-63: value e + E/2
            }
#pragma unroll
            for (int e = 0; e < E / 4; ++e) {
                const auto r = __builtin_amdgcn_permlane16_swap(f2u(half[e]), f2u(half[e + E / 4]), false, false);
                kept[e] = u2f(r[0]) + u2f(r[1]);  // even 16-lane rows: value e of the half, odd ones: e + E/4
            }
#pragma unroll
            for (int e = 0; e < E / 4; ++e) {
                if (lpr_log2 <= 3) kept[e] += dpp<0x128, 0xf>(kept[e], kept[e]);  // row_ror:8
                if (lpr_log2 <= 2) kept[e] += dpp<0x124, 0xf>(kept[e], kept[e]);  // row_ror:4
                if (lpr_log2 <= 1) kept[e] += dpp<0x122, 0xf>(kept[e], kept[e]);  // row_ror:2
                if (lpr_log2 <= 0) kept[e] += dpp<0x121, 0xf>(kept[e], kept[e]);  // row_ror:1
            }
        }
        // the first group of every 16-lane row stores its quarter: values (half * E/2 + odd row * E/4) onwards
        if ((lane & 15) < (1 << lpr_log2) && p < CL) {
            const int32_t first = (lane >> 5) * (E / 2) + ((lane >> 4) & 1) * (E / 4);
            float* dst = gate_grad_partial + (gate_row * G + tile) * L + t0 + first;
            if constexpr (E == 8) *reinterpret_cast<float2*>(dst) = make_float2(kept[0], kept[1]);
            else dst[0] = kept[0];
        }
        cur = next;
    }
    if (active) store16<T>(token_grad + token_row * L + t0, Elem<T>::pack(dtok));
}

// ---- scan and norm in one kernel, for short rows ---------------------------------------------------
// What scan_forward_normed_kernel computes (fmscan_normed.h: the states scanned, rounded as stored states
// are, their mean square over the D rows of a slot, states_n = state * inv_rms and inv_rms itself), with
// several rows to a wave. A wave is a slot (b, m): it walks the slot's rows in NT tiles of 64 >> lpr_log2
// rows, keeps every tile's rounded states packed in registers (NT <= NT_MAX), adds up their squares per
// lane, sums those over the wave's groups (every lane ends with the sum over all D rows at its steps),
// and scales and stores what it holds. The gates are the same for all rows of a slot: their half of the
// segmented scan is done once, a tile scans the other half only. No LDS, no barrier.
template <typename T, int NT_MAX>
__global__ __launch_bounds__(256) void scan_forward_normed_packed_kernel(
    const T* __restrict__ gates, const T* __restrict__ tokens, const T* __restrict__ h0,
    T* __restrict__ states_n /* (B, M, D, L) */, float* __restrict__ inv_rms /* (B, M, L) */, int64_t slots,
    int32_t M, int32_t D, int32_t L, float eps, int32_t lpr_log2, int32_t NT) {
    constexpr int E = Elem<T>::E;
    const int32_t CL = L / E;  // rows are whole 16-byte vectors
    const int lane = threadIdx.x & 63;
    const int64_t bm = (int64_t)blockIdx.x * (blockDim.x >> 6) + uniform((int)(threadIdx.x >> 6));
    if (bm >= slots) return;  // whole waves
    const int64_t b = (int64_t)uniform((int)((uint32_t)bm / (uint32_t)M));
    const int32_t p = lane & ((1 << lpr_log2) - 1);
    const int32_t group = lane >> lpr_log2;
    const int32_t per_tile = 64 >> lpr_log2;
    const bool in_row = p < CL;
    const int32_t t0 = (in_row ? p : CL - 1) * E;

    // the gates' half of the scan, once: the product of the chunk's gates before each of the four steps
    // inside a group (groups are at most 16 lanes here)
    float g[E];
    Elem<T>::unpack(load16<T, false>(gates + bm * L + t0), g);
    if (!in_row) {
#pragma unroll
        for (int e = 0; e < E; ++e) g[e] = 1.0f;
    }
    float a_chunk = g[0];
#pragma unroll
    for (int e = 1; e < E; ++e) a_chunk *= g[e];
    float a_before[4];
    {
        float a = a_chunk;
        a_before[0] = a;
        a = p >= 1 ? a * dpp<0x111, 0xf>(1.0f, a) : a;
        a_before[1] = a;
        a = p >= 2 ? a * dpp<0x112, 0xf>(1.0f, a) : a;
        a_before[2] = a;
        a = p >= 4 ? a * dpp<0x114, 0xf>(1.0f, a) : a;
        a_before[3] = a;
    }

    auto row_of = [&](int32_t i) {  // the row of this lane in tile i (clamped: lanes without one load the last)
        const int32_t d = i * per_tile + group;
        return d < D ? d : D - 1;
    };
    constexpr int RING = 4;  // token tiles in flight
    u32x4 xq[RING];
#pragma unroll
    for (int i = 0; i < RING; ++i)
        xq[i] = load16<T, false>(tokens + (b * D + row_of(i < NT ? i : 0)) * L + t0);

    u32x4 held[NT_MAX];
    float sumsq[E];
#pragma unroll
    for (int e = 0; e < E; ++e) sumsq[e] = 0.0f;
#pragma unroll
    for (int i = 0; i < NT_MAX; ++i) {
        if (i >= NT) continue;  // the whole wave
        const int32_t d = row_of(i);
        const bool active = i * per_tile + group < D && in_row;
        float u[E];
        Elem<T>::unpack(xq[i % RING], u);
        if (i + RING < NT_MAX) xq[i % RING] = load16<T, false>(tokens + (b * D + row_of(i + RING < NT ? i + RING : i)) * L + t0);
        const float hin = (h0 && p == 0) ? Elem<T>::widen(h0[bm * D + d]) : 0.0f;
#pragma unroll
        for (int e = 0; e < E; ++e) u[e] = in_row ? __builtin_fmaf(-g[e], u[e], u[e]) : 0.0f;  // (1 - g) x, one rounding
        float bb = u[0];
#pragma unroll
        for (int e = 1; e < E; ++e) bb = __builtin_fmaf(g[e], bb, u[e]);
        if (p == 0) bb = __builtin_fmaf(a_chunk, hin, bb);  // the state before the row enters the group's first chunk
        {
            float nb = __builtin_fmaf(dpp<0x111, 0xf>(0.0f, bb), a_before[0], bb);
            bb = p >= 1 ? nb : bb;
            nb = __builtin_fmaf(dpp<0x112, 0xf>(0.0f, bb), a_before[1], bb);
            bb = p >= 2 ? nb : bb;
            nb = __builtin_fmaf(dpp<0x114, 0xf>(0.0f, bb), a_before[2], bb);
            bb = p >= 4 ? nb : bb;
            nb = __builtin_fmaf(dpp<0x118, 0xf>(0.0f, bb), a_before[3], bb);
            bb = p >= 8 ? nb : bb;
        }
        const float before = dpp<kWaveShr1>(0.0f, bb);
        float h = p == 0 ? hin : before;
        float o[E];
#pragma unroll
        for (int e = 0; e < E; ++e) {
            h = __builtin_fmaf(g[e], h, u[e]);
            o[e] = h;
        }
        held[i] = Elem<T>::pack(o);
        Elem<T>::unpack(held[i], o);  // the norm sees the states as they would be stored
#pragma unroll
        for (int e = 0; e < E; ++e) sumsq[e] = active ? __builtin_fmaf(o[e], o[e], sumsq[e]) : sumsq[e];
    }
    sum_over_groups<E>(sumsq, lpr_log2);
    float r[E];
#pragma unroll
    for (int e = 0; e < E; ++e) r[e] = 1.0f / __builtin_sqrtf(sumsq[e] / (float)D + eps);
    if (group == 0 && in_row) {
        float* dst = inv_rms + bm * L + t0;
#pragma unroll
        for (int e = 0; e < E; e += 4) *reinterpret_cast<float4*>(dst + e) = make_float4(r[e], r[e + 1], r[e + 2], r[e + 3]);
    }
#pragma unroll
    for (int i = 0; i < NT_MAX; ++i) {
        if (i < NT && i * per_tile + group < D && in_row) {
            float o[E];
            Elem<T>::unpack(held[i], o);
#pragma unroll
            for (int e = 0; e < E; ++e) o[e] *= r[e];
            store16<T>(states_n + (bm * D + i * per_tile + group) * L + t0, Elem<T>::pack(o));
        }
    }
}

// ---- the layer's read-out and its dot, for short rows ------------------------------------------------
// output[b,d,t] = sum_m read[b,m,t] * states[b,m,d,t] (readout_forward_kernel without the norm,
// fmscan_readout.h; reference fm/scan/fm_scan.py:130-131). A wave is a batch element and a tile of
// 64 >> lpr_log2 rows d and walks the M slots, the next slot's loads in flight.
template <typename T>
__global__ __launch_bounds__(256) void readout_forward_packed_kernel(
    const T* __restrict__ states /* (B, M, D, L) */, const T* __restrict__ read /* (B, M, L) */,
    T* __restrict__ output /* (B, D, L) */, int32_t B, int32_t M, int32_t D, int32_t L, int32_t lpr_log2, int32_t G) {
    constexpr int E = Elem<T>::E;
    const int32_t CL = L / E;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + uniform((int)(threadIdx.x >> 6));
    if (wave >= (int64_t)B * G) return;  // whole waves
    const int32_t b = uniform((int)(wave / G));
    const int32_t tile = uniform((int)(wave - (int64_t)b * G));
    const int32_t p = lane & ((1 << lpr_log2) - 1);
    const int32_t d_mine = (tile << (6 - lpr_log2)) + (lane >> lpr_log2);
    const bool active = d_mine < D && p < CL;
    const int32_t d = d_mine < D ? d_mine : D - 1;
    const int32_t t0 = (p < CL ? p : CL - 1) * E;
    float acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = 0.0f;
    struct In {
        u32x4 h, wr;
    };
    auto fetch = [&](In& n, int32_t m) {
        const int64_t bm = (int64_t)b * M + m;
        n.h = load16<T, true>(states + (bm * D + d) * L + t0);
        n.wr = load16<T, false>(read + bm * L + t0);
    };
    In cur, next;
    fetch(cur, 0);
    for (int32_t m = 0; m < M; ++m) {
        fetch(next, m + 1 < M ? m + 1 : m);
        float h[E], wr[E];
        Elem<T>::unpack(cur.h, h);
        Elem<T>::unpack(cur.wr, wr);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] = __builtin_fmaf(wr[e], h[e], acc[e]);
        cur = next;
    }
    if (active) store16<T>(output + ((int64_t)b * D + d) * L + t0, Elem<T>::pack(acc));
}

// q[b,m,t] = sum_d out_grad[b,d,t] * states_n[b,m,d,t] and what the layer's backward kernel takes with it
// (rowdot_kernel in its dot form, fmscan_readout.h). A wave is a slot and walks its rows in tiles; the
// lanes' sums meet across the wave's groups.
template <typename T, bool EXT>
__global__ __launch_bounds__(256) void readout_dot_packed_kernel(
    const T* __restrict__ states_n /* (B, M, D, L) */, const T* __restrict__ out_grad /* (B, D, L) */,
    const T* __restrict__ ext_grad /* (B, M, D, L); EXT */, float* __restrict__ q /* (B, M, L) */,
    float* __restrict__ qe /* (B, M, L); EXT: sum_d ext_grad * states_n */, const float* __restrict__ inv_rms,
    const T* __restrict__ read,
    float* __restrict__ coef_out, float* __restrict__ coef_self, float* __restrict__ rms_out, int64_t slots,
    int32_t M, int32_t D, int32_t L, int32_t lpr_log2, int32_t NT) {
    constexpr int E = Elem<T>::E;
    const int32_t CL = L / E;
    const int lane = threadIdx.x & 63;
    const int64_t bm = (int64_t)blockIdx.x * (blockDim.x >> 6) + uniform((int)(threadIdx.x >> 6));
    if (bm >= slots) return;  // whole waves
    const int64_t b = (int64_t)uniform((int)((uint32_t)bm / (uint32_t)M));
    const int32_t p = lane & ((1 << lpr_log2) - 1);
    const int32_t group = lane >> lpr_log2;
    const int32_t per_tile = 64 >> lpr_log2;
    const bool in_row = p < CL;
    const int32_t t0 = (in_row ? p : CL - 1) * E;
    float acc[E], acc_ext[E];
#pragma unroll
    for (int e = 0; e < E; ++e) acc[e] = acc_ext[e] = 0.0f;
    struct In {
        u32x4 h, y, x;
    };
    auto fetch = [&](In& n, int32_t i) {
        const int32_t d_mine = i * per_tile + group;
        const int32_t d = d_mine < D ? d_mine : D - 1;
        n.h = load16<T, true>(states_n + (bm * D + d) * L + t0);
        n.y = load16<T, false>(out_grad + (b * D + d) * L + t0);
        if constexpr (EXT) n.x = load16<T, true>(ext_grad + (bm * D + d) * L + t0);
    };
    In cur, next;
    fetch(cur, 0);
    for (int32_t i = 0; i < NT; ++i) {
        fetch(next, i + 1 < NT ? i + 1 : i);
        const bool active = i * per_tile + group < D && in_row;
        float h[E], y[E];
        Elem<T>::unpack(cur.h, h);
        Elem<T>::unpack(cur.y, y);
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] = active ? __builtin_fmaf(h[e], y[e], acc[e]) : acc[e];
        if constexpr (EXT) {
            Elem<T>::unpack(cur.x, y);
#pragma unroll
            for (int e = 0; e < E; ++e) acc_ext[e] = active ? __builtin_fmaf(h[e], y[e], acc_ext[e]) : acc_ext[e];
        }
        cur = next;
    }
    sum_over_groups<E>(acc, lpr_log2);
    if constexpr (EXT) sum_over_groups<E>(acc_ext, lpr_log2);
    if (group == 0 && in_row) {
        const int64_t at = bm * L + t0;
#pragma unroll
        for (int e = 0; e < E; e += 4) {
            *reinterpret_cast<float4*>(q + at + e) = make_float4(acc[e], acc[e + 1], acc[e + 2], acc[e + 3]);
            if constexpr (EXT)
                *reinterpret_cast<float4*>(qe + at + e) = make_float4(acc_ext[e], acc_ext[e + 1], acc_ext[e + 2], acc_ext[e + 3]);
        }
        if (coef_out != nullptr || rms_out != nullptr) {
            float r[E], wr[E];
#pragma unroll
            for (int e = 0; e < E; ++e) r[e] = 1.0f;
            if (inv_rms != nullptr) spread<E>(load_float_chunk<E>(inv_rms + at), r);
            if (coef_out != nullptr) {
                Elem<T>::unpack(load16<T, false>(read + at), wr);
#pragma unroll
                for (int e = 0; e < E; ++e) {
                    const float c = r[e] * wr[e];
                    coef_out[at + e] = c;
                    coef_self[at + e] = inv_rms != nullptr ? c * acc[e] / (float)D : 0.0f;
                }
            }
            if (rms_out != nullptr) {
#pragma unroll
                for (int e = 0; e < E; ++e) rms_out[at + e] = 1.0f / r[e];
            }
        }
    }
}

// dn = read * out_grad (+ ext_grad); with the norm  d h = inv_rms * (dn - states_n * s / D), s = read * q (+ qe)
// (readout_backward_kernel, fmscan_readout.h). A wave is a batch element and a tile of rows and walks the slots.
// state_grad may be ext_grad itself: a lane reads its chunk before it writes it.
template <typename T, bool NORM, bool EXT>
__global__ __launch_bounds__(256) void readout_backward_packed_kernel(
    const T* __restrict__ states_n, const float* __restrict__ inv_rms, const T* __restrict__ read,
    const T* __restrict__ out_grad /* (B, D, L) */, const T* ext_grad /* (B, M, D, L) */, const float* __restrict__ q,
    const float* __restrict__ qe, T* state_grad /* (B, M, D, L) */, int32_t B, int32_t M, int32_t D, int32_t L,
    int32_t lpr_log2, int32_t G) {
    constexpr int E = Elem<T>::E;
    const int32_t CL = L / E;
    const int lane = threadIdx.x & 63;
    const int64_t wave = (int64_t)blockIdx.x * (blockDim.x >> 6) + uniform((int)(threadIdx.x >> 6));
    if (wave >= (int64_t)B * G) return;  // whole waves
    const int32_t b = uniform((int)(wave / G));
    const int32_t tile = uniform((int)(wave - (int64_t)b * G));
    const int32_t p = lane & ((1 << lpr_log2) - 1);
    const int32_t d_mine = (tile << (6 - lpr_log2)) + (lane >> lpr_log2);
    const bool active = d_mine < D && p < CL;
    const int32_t d = d_mine < D ? d_mine : D - 1;
    const int32_t t0 = (p < CL ? p : CL - 1) * E;
    float dout[E];
    Elem<T>::unpack(load16<T, false>(out_grad + ((int64_t)b * D + d) * L + t0), dout);
    const float inv_d = 1.0f / (float)D;
    struct In {
        u32x4 wr, x, hn;
        FloatChunk<E> r, s, se;
    };
    auto fetch = [&](In& n, int32_t m) {
        const int64_t bm = (int64_t)b * M + m;
        const int64_t row = (bm * D + d) * L + t0;
        n.wr = load16<T, false>(read + bm * L + t0);
        if constexpr (EXT) n.x = load16<T, true>(ext_grad + row);
        if constexpr (NORM) {
            n.hn = load16<T, true>(states_n + row);
            n.r = load_float_chunk<E>(inv_rms + bm * L + t0);
            n.s = load_float_chunk<E>(q + bm * L + t0);
            if constexpr (EXT) n.se = load_float_chunk<E>(qe + bm * L + t0);
        }
    };
    In cur, next;
    fetch(cur, 0);
    for (int32_t m = 0; m < M; ++m) {
        fetch(next, m + 1 < M ? m + 1 : m);
        float wr[E], g[E];
        Elem<T>::unpack(cur.wr, wr);
#pragma unroll
        for (int e = 0; e < E; ++e) g[e] = wr[e] * dout[e];
        if constexpr (EXT) {
            float x[E];
            Elem<T>::unpack(cur.x, x);
#pragma unroll
            for (int e = 0; e < E; ++e) g[e] += x[e];
        }
        if constexpr (NORM) {
            float r[E], sv[E], hn[E];
            spread<E>(cur.r, r);
            spread<E>(cur.s, sv);
            Elem<T>::unpack(cur.hn, hn);
#pragma unroll
            for (int e = 0; e < E; ++e) sv[e] *= wr[e];
            if constexpr (EXT) {
                float se[E];
                spread<E>(cur.se, se);
#pragma unroll
                for (int e = 0; e < E; ++e) sv[e] += se[e];
            }
#pragma unroll
            for (int e = 0; e < E; ++e) g[e] = r[e] * __builtin_fmaf(-hn[e], sv[e] * inv_d, g[e]);
        }
        if (active) store16<T>(state_grad + (((int64_t)b * M + m) * D + d) * L + t0, Elem<T>::pack(g));
        cur = next;
    }
}

}  // namespace fmscan
