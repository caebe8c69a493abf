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

}  // namespace fmscan
