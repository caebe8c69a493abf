// The part of the Factorization-Memory layer that consumes the scanned states
// (reference fm/scan/fm_scan.py:124-131): RMS norm over the D axis of every memory
// slot, then the read-out  output[b,t,d] = sum_m read[b,t,m] * states[b,m,d,t].
// The reference runs it as five PyTorch operations over (B, M, D, L) tensors (square,
// mean, rsqrt, multiply, einsum), each a full pass through HBM, and autograd doubles
// that. Here, forward and backward are two kernels each:
//
//   rowdot_kernel     one value per (b, m, t) from all D rows of a slot:
//                       SUMSQ: inv_rms = rsqrt(mean_d h^2 + eps)
//                       DOT:   q = sum_d out_grad[b,d,t] * hn[b,m,d,t]   (= d read)
//                              qe = sum_d ext_grad[b,m,d,t] * hn[b,m,d,t] (optional)
//   readout_forward   hn = h * inv_rms (stored), out[b,d,t] = sum_m read * hn
//   readout_backward  d h = inv_rms * (dhn - hn * mean_d(dhn * hn)),
//                       dhn = read * out_grad (+ ext_grad)
//
// All of them stream rows the way the scan kernels do: a wave instruction covers 1 KiB
// of one row (16 bytes per lane), fp32 arithmetic, one rounding on store. Time is the
// innermost axis of every tensor here, as the scan leaves it: output is (B, D, L).
#pragma once

#include "fmscan_device.h"

namespace fmscan {

// E consecutive floats of a per-(b, m) vector (inv_rms, q): row + t0 .. t0 + E - 1
template <int E, bool VEC>
__device__ __forceinline__ void load_floats(const float* __restrict__ row, int64_t t0, int64_t L,
                                            float (&v)[E], float fill) {
#pragma unroll
    for (int i = 0; i < E; ++i) v[i] = fill;
    if (t0 >= L) return;
    if constexpr (VEC) {  // L is a multiple of E and rows start 16-byte aligned
#pragma unroll
        for (int i = 0; i < E; i += 4) {
            const float4 f = *reinterpret_cast<const float4*>(row + t0 + i);
            v[i] = f.x; v[i + 1] = f.y; v[i + 2] = f.z; v[i + 3] = f.w;
        }
    } else {
#pragma unroll
        for (int i = 0; i < E; ++i)
            if (t0 + i < L) v[i] = row[t0 + i];
    }
}

enum class RowDot { kSumSq, kDot };

// One block per (b, m, tile of L), blockIdx.x = (b * M + m) * tiles + tile; WV waves take
// the D rows of the slot in turn.
template <typename T, int WV, RowDot MODE, bool EXT, bool VEC>
__global__ __launch_bounds__(64 * WV) void rowdot_kernel(
    const T* __restrict__ states /* (B, M, D, L) */, const T* __restrict__ out_grad /* (B, D, L) */,
    const T* __restrict__ ext_grad /* (B, M, D, L) */, float* __restrict__ result /* (B, M, L) */,
    float* __restrict__ result_ext /* (B, M, L) */, const float* __restrict__ inv_rms /* (B, M, L) */,
    const T* __restrict__ read /* (B, M, L) */, float* __restrict__ coef_out, float* __restrict__ coef_self,
    float* __restrict__ rms_out /* (B, M, L) */, int32_t M, int32_t D, int64_t L, int32_t tiles, float eps) {
    constexpr int E = Elem<T>::E;
    constexpr int TILE = E * 64;
    __shared__ float part[EXT ? 2 : 1][WV][TILE];
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    const int64_t bm = blockIdx.x / (uint32_t)tiles;
    const int64_t tile = blockIdx.x - bm * tiles;
    const int64_t b = bm / M;
    const int64_t t0 = tile * TILE + (int64_t)lane * E;

    float acc[E], acc_ext[E];
#pragma unroll
    for (int i = 0; i < E; ++i) acc[i] = acc_ext[i] = 0.0f;
#pragma unroll 4
    for (int32_t d = w; d < D; d += WV) {
        float h[E];
        Elem<T>::unpack(load_chunk<T, VEC, true>(states + (bm * D + d) * L, t0, L, 0u), h);
        if constexpr (MODE == RowDot::kSumSq) {
#pragma unroll
            for (int i = 0; i < E; ++i) acc[i] = __builtin_fmaf(h[i], h[i], acc[i]);
        } else {
            float y[E];
            Elem<T>::unpack(load_chunk<T, VEC, false>(out_grad + (b * D + d) * L, t0, L, 0u), y);
#pragma unroll
            for (int i = 0; i < E; ++i) acc[i] = __builtin_fmaf(h[i], y[i], acc[i]);
            if constexpr (EXT) {
                Elem<T>::unpack(load_chunk<T, VEC, true>(ext_grad + (bm * D + d) * L, t0, L, 0u), y);
#pragma unroll
                for (int i = 0; i < E; ++i) acc_ext[i] = __builtin_fmaf(h[i], y[i], acc_ext[i]);
            }
        }
    }
#pragma unroll
    for (int i = 0; i < E; ++i) {
        part[0][w][lane * E + i] = acc[i];
        if constexpr (EXT) part[1][w][lane * E + i] = acc_ext[i];
    }
    __syncthreads();
    for (int e = threadIdx.x; e < TILE; e += 64 * WV) {
        const int64_t t = tile * TILE + e;
        if (t >= L) break;
        float s = 0.0f, se = 0.0f;
#pragma unroll
        for (int v = 0; v < WV; ++v) {  // fixed order: run-to-run identical
            s += part[0][v][e];
            if constexpr (EXT) se += part[1][v][e];
        }
        if constexpr (MODE == RowDot::kSumSq) s = 1.0f / __builtin_sqrtf(s / (float)D + eps);
        result[bm * L + t] = s;
        if constexpr (EXT) result_ext[bm * L + t] = se;
        if constexpr (MODE == RowDot::kDot) {
            // what scan_backward_reduced_kernel<..., LAYER> takes: the states' gradient is
            // coef_out * out_grad - coef_self * normalised state
            if (coef_out != nullptr) {
                const float c = (inv_rms ? inv_rms[bm * L + t] : 1.0f) * (float)read[bm * L + t];
                coef_out[bm * L + t] = c;
                coef_self[bm * L + t] = inv_rms ? c * s / (float)D : 0.0f;
            }
            // ... and what takes the scanned states back from the normalised ones
            if (rms_out != nullptr) rms_out[bm * L + t] = 1.0f / inv_rms[bm * L + t];
        }
    }
}

// grid (B * tiles of L, groups of 4 * J consecutive d); wave w of a block owns J
// consecutive d and walks the M slots; the per-slot vectors (inv_rms, read) are loaded
// once per slot and reused for the J rows.
template <typename T, int J, bool NORM, bool VEC>
__global__ __launch_bounds__(256) void readout_forward_kernel(
    const T* states /* (B, M, D, L) */, const float* __restrict__ inv_rms /* (B, M, L) */,
    const T* __restrict__ read /* (B, M, L) */, T* states_out /* (B, M, D, L); may be `states` itself */,
    T* __restrict__ output /* (B, D, L) */, int32_t M, int32_t D, int64_t L, int32_t tiles) {
    constexpr int E = Elem<T>::E;
    constexpr int TILE = E * 64;
    const int lane = threadIdx.x & 63;
    const int w = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));  // the same in all lanes: scalar branches on d
    const int64_t b = blockIdx.x / (uint32_t)tiles;
    const int32_t d0 = ((int32_t)blockIdx.y * 4 + w) * J;
    if (d0 >= D) return;  // whole waves; no barrier in this kernel
    const int64_t t0 = (blockIdx.x - b * tiles) * TILE + (int64_t)lane * E;

    float acc[J][E];
#pragma unroll
    for (int j = 0; j < J; ++j) {
#pragma unroll
        for (int i = 0; i < E; ++i) acc[j][i] = 0.0f;
    }
    if constexpr (VEC) {
        // A wave walks the M slots one after the other, and what it has in flight is what bounds its
        // pace: the loads of the slot after the one at work are issued before the work starts (a slot
        // beyond the last is the last again, unused: every pass issues the same loads, so the waits
        // are counted). Rows of d beyond D (last block) are loaded as row D - 1 and dropped. In place
        // (states_out == states) this is safe: a slot's rows are read before any of them is written,
        // and no other slot's rows are written in between.
        struct Slot {
            u32x4 wr;
            FloatChunk<E> r;
            u32x4 h[J];
        };
        const bool live = t0 < L;                            // this lane's chunk lies in the row
        const int64_t tl = live ? t0 : L - E;                // a chunk past the end reads the last one
        auto fetch = [&](Slot& q, int32_t m) {
            const int64_t bm = b * M + (m < M ? m : M - 1);
            q.wr = load16<T, false>(read + bm * L + tl);
            if constexpr (NORM) q.r = load_float_chunk<E>(inv_rms + bm * L + tl);
#pragma unroll
            for (int j = 0; j < J; ++j) {
                const int32_t d = d0 + j < D ? d0 + j : D - 1;
                q.h[j] = load16<T, true>(states + (bm * D + d) * L + tl);
            }
        };
        auto work = [&](const Slot& q, int32_t m) {
            const int64_t bm = b * M + m;
            float r[E], wr[E];
            Elem<T>::unpack(q.wr, wr);
            if constexpr (NORM) spread<E>(q.r, r);
#pragma unroll
            for (int j = 0; j < J; ++j) {
                if (d0 + j >= D) continue;  // the whole wave
                float h[E];
                Elem<T>::unpack(q.h[j], h);
                if constexpr (NORM) {
#pragma unroll
                    for (int i = 0; i < E; ++i) h[i] *= r[i];
                    const u32x4 packed = Elem<T>::pack(h);
                    if (live) store16<T>(states_out + (bm * D + d0 + j) * L + t0, packed);
                    Elem<T>::unpack(packed, h);  // the read-out sees what was stored
                }
#pragma unroll
                for (int i = 0; i < E; ++i) acc[j][i] = __builtin_fmaf(wr[i], h[i], acc[j][i]);
            }
        };
        Slot qa, qb;  // two sets of registers that swap roles: no copy from one to the other
        fetch(qa, 0);
        for (int32_t m = 0; m < M; m += 2) {
            fetch(qb, m + 1);
            work(qa, m);
            fetch(qa, m + 2);
            if (m + 1 < M) work(qb, m + 1);
        }
        if (live) {
#pragma unroll
            for (int j = 0; j < J; ++j)
                if (d0 + j < D) store16<T>(output + (b * D + d0 + j) * L + t0, Elem<T>::pack(acc[j]));
        }
        return;
    }
    for (int32_t m = 0; m < M; ++m) {
        const int64_t bm = b * M + m;
        float r[E], wr[E];
        if constexpr (NORM) load_floats<E, VEC>(inv_rms + bm * L, t0, L, r, 0.0f);
        Elem<T>::unpack(load_chunk<T, VEC, false>(read + bm * L, t0, L, 0u), wr);
#pragma unroll
        for (int j = 0; j < J; ++j) {
            if (d0 + j < D) {
                const int64_t row = (bm * D + d0 + j) * L;
                float h[E];
                Elem<T>::unpack(load_chunk<T, VEC, true>(states + row, t0, L, 0u), h);
                if constexpr (NORM) {
#pragma unroll
                    for (int i = 0; i < E; ++i) h[i] *= r[i];
                    const u32x4 packed = Elem<T>::pack(h);
                    store_chunk<T, VEC>(states_out + row, t0, L, packed);
                    Elem<T>::unpack(packed, h);  // the read-out sees what was stored
                }
#pragma unroll
                for (int i = 0; i < E; ++i) acc[j][i] = __builtin_fmaf(wr[i], h[i], acc[j][i]);
            }
        }
    }
#pragma unroll
    for (int j = 0; j < J; ++j)
        if (d0 + j < D) store_chunk<T, VEC>(output + (b * D + d0 + j) * L, t0, L, Elem<T>::pack(acc[j]));
}

// Same grid. dhn = read * out_grad (+ ext_grad); with the norm
// d h = inv_rms * (dhn - hn * s / D), s = sum_d dhn * hn = read * q (+ qe).
template <typename T, int J, bool NORM, bool EXT, bool VEC>
__global__ __launch_bounds__(256) void readout_backward_kernel(
    const T* __restrict__ states_n /* (B, M, D, L), normalised; unused without the norm */,
    const float* __restrict__ inv_rms, const T* __restrict__ read, const T* __restrict__ out_grad /* (B, D, L) */,
    const T* ext_grad /* (B, M, D, L) */, const float* __restrict__ q, const float* __restrict__ qe,
    T* state_grad /* (B, M, D, L); may be `ext_grad` itself */, int32_t M, int32_t D, int64_t L, int32_t tiles) {
    constexpr int E = Elem<T>::E;
    constexpr int TILE = E * 64;
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    const int64_t b = blockIdx.x / (uint32_t)tiles;
    const int32_t d0 = ((int32_t)blockIdx.y * 4 + w) * J;
    if (d0 >= D) return;
    const int64_t t0 = (blockIdx.x - b * tiles) * TILE + (int64_t)lane * E;

    float dout[J][E];
#pragma unroll
    for (int j = 0; j < J; ++j) {
#pragma unroll
        for (int i = 0; i < E; ++i) dout[j][i] = 0.0f;
        if (d0 + j < D)
            Elem<T>::unpack(load_chunk<T, VEC, false>(out_grad + (b * D + d0 + j) * L, t0, L, 0u), dout[j]);
    }
    const float inv_d = 1.0f / (float)D;
    for (int32_t m = 0; m < M; ++m) {
        const int64_t bm = b * M + m;
        float wr[E], r[E], s[E];
        Elem<T>::unpack(load_chunk<T, VEC, false>(read + bm * L, t0, L, 0u), wr);
        if constexpr (NORM) {
            load_floats<E, VEC>(inv_rms + bm * L, t0, L, r, 0.0f);
            load_floats<E, VEC>(q + bm * L, t0, L, s, 0.0f);
#pragma unroll
            for (int i = 0; i < E; ++i) s[i] *= wr[i];
            if constexpr (EXT) {
                float se[E];
                load_floats<E, VEC>(qe + bm * L, t0, L, se, 0.0f);
#pragma unroll
                for (int i = 0; i < E; ++i) s[i] += se[i];
            }
#pragma unroll
            for (int i = 0; i < E; ++i) s[i] *= inv_d;
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            if (d0 + j < D) {
                const int64_t row = (bm * D + d0 + j) * L;
                float g[E];
#pragma unroll
                for (int i = 0; i < E; ++i) g[i] = wr[i] * dout[j][i];
                if constexpr (EXT) {
                    float e[E];
                    Elem<T>::unpack(load_chunk<T, VEC, true>(ext_grad + row, t0, L, 0u), e);
#pragma unroll
                    for (int i = 0; i < E; ++i) g[i] += e[i];
                }
                if constexpr (NORM) {
                    float hn[E];
                    Elem<T>::unpack(load_chunk<T, VEC, true>(states_n + row, t0, L, 0u), hn);
#pragma unroll
                    for (int i = 0; i < E; ++i) g[i] = r[i] * __builtin_fmaf(-hn[i], s[i], g[i]);
                }
                store_chunk<T, VEC>(state_grad + row, t0, L, Elem<T>::pack(g));
            }
        }
    }
}

// dst[b, c, r] = src[b, r, c]: the layer takes (B, L, *) tensors and the kernels want time
// last (reference fm_scan.py:117-118 does it with transpose().contiguous()). 64 x 64
// tiles through LDS, so that both the reads and the writes are whole 128- or 256-byte
// runs; U is an unsigned integer of the element's size.
template <typename U>
__global__ __launch_bounds__(256) void swap_last_two_kernel(const U* __restrict__ src, U* __restrict__ dst,
                                                            int64_t R, int64_t C, int32_t tiles_c,
                                                            int32_t tiles_r) {
    __shared__ U tile[64][65];
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    const int64_t per_b = (int64_t)tiles_c * tiles_r;
    const int64_t b = blockIdx.x / per_b;
    const int64_t rest = blockIdx.x - b * per_b;
    const int64_t r0 = (rest / tiles_c) * 64, c0 = (rest % tiles_c) * 64;
    const U* __restrict__ s = src + b * R * C;
    U* __restrict__ d = dst + b * R * C;
#pragma unroll 4
    for (int i = w; i < 64; i += 4)
        if (r0 + i < R && c0 + lane < C) tile[i][lane] = s[(r0 + i) * C + c0 + lane];
    __syncthreads();
#pragma unroll 4
    for (int i = w; i < 64; i += 4)
        if (c0 + i < C && r0 + lane < R) d[(c0 + i) * R + r0 + lane] = tile[lane][i];
}

// The same for 2-byte elements when R and C are even and both pointers 4-byte aligned: every
// lane moves two neighbouring elements (4 bytes) on both sides, half a wave per row, so a wave
// instruction covers two 128-byte runs instead of one.
__global__ __launch_bounds__(256) void swap_last_two_pairs_kernel(const uint16_t* __restrict__ src,
                                                                  uint16_t* __restrict__ dst, int64_t R, int64_t C,
                                                                  int32_t tiles_c, int32_t tiles_r) {
    __shared__ uint16_t tile[64][66];  // 132-byte rows: 4-byte aligned, odd in 4-byte words
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    const int half = lane >> 5, pair = lane & 31;
    const int64_t per_b = (int64_t)tiles_c * tiles_r;
    const int64_t b = blockIdx.x / per_b;
    const int64_t rest = blockIdx.x - b * per_b;
    const int64_t r0 = (rest / tiles_c) * 64, c0 = (rest % tiles_c) * 64;
    const uint16_t* __restrict__ s = src + b * R * C;
    uint16_t* __restrict__ d = dst + b * R * C;
#pragma unroll 4
    for (int i = 2 * w + half; i < 64; i += 8)
        if (r0 + i < R && c0 + 2 * pair < C)
            *reinterpret_cast<uint32_t*>(&tile[i][2 * pair]) =
                *reinterpret_cast<const uint32_t*>(s + (r0 + i) * C + c0 + 2 * pair);
    __syncthreads();
#pragma unroll 4
    for (int j = 2 * w + half; j < 64; j += 8)
        if (c0 + j < C && r0 + 2 * pair < R)
            *reinterpret_cast<uint32_t*>(d + (c0 + j) * R + r0 + 2 * pair) =
                (uint32_t)tile[2 * pair][j] | ((uint32_t)tile[2 * pair + 1][j] << 16);
}

// The same for 2-byte elements when R and C are multiples of 8 and both pointers 16-byte aligned:
// every lane moves 8 neighbouring elements (16 bytes) on both sides, 8 lanes per 128-byte run of a
// 64 x 64 tile; between the two, each lane gathers its 8 elements of one column from LDS.
__global__ __launch_bounds__(256) void swap_last_two_wide_kernel(const uint16_t* __restrict__ src,
                                                                 uint16_t* __restrict__ dst, int64_t R, int64_t C,
                                                                 int32_t tiles_c, int32_t tiles_r) {
    constexpr int PITCH = 66;  // elements: rows of 33 words, so that the gather below meets each bank at most twice
    __shared__ __attribute__((aligned(4))) uint16_t tile[64 * PITCH];
    const int64_t per_b = (int64_t)tiles_c * tiles_r;
    const int64_t b = blockIdx.x / per_b;
    const int64_t rest = blockIdx.x - b * per_b;
    const int64_t r0 = (rest / tiles_c) * 64, c0 = (rest % tiles_c) * 64;
    const uint16_t* __restrict__ s = src + b * R * C;
    uint16_t* __restrict__ d = dst + b * R * C;
    const int group = threadIdx.x & 7, line = threadIdx.x >> 3;  // 8 lanes of 16 bytes per run, 32 runs per pass
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int i = line + 32 * pass;
        if (r0 + i < R && c0 + 8 * group < C) {
            const u32x4 v = *reinterpret_cast<const u32x4*>(s + (r0 + i) * C + c0 + 8 * group);
            uint32_t* row = reinterpret_cast<uint32_t*>(&tile[i * PITCH + 8 * group]);  // 4-byte aligned only
            row[0] = v.x; row[1] = v.y; row[2] = v.z; row[3] = v.w;
        }
    }
    __syncthreads();
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int j = line + 32 * pass;  // the column of the tile this lane writes a run of
        if (c0 + j < C && r0 + 8 * group < R) {
            uint32_t v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k)
                v[k] = (uint32_t)tile[(8 * group + 2 * k) * PITCH + j] |
                       ((uint32_t)tile[(8 * group + 2 * k + 1) * PITCH + j] << 16);
            *reinterpret_cast<u32x4*>(d + (c0 + j) * R + r0 + 8 * group) = u32x4{v[0], v[1], v[2], v[3]};
        }
    }
}

// gates[b, m, t] = 1 - alpha[b, t, m] * update_scale[b, t], read[b, m, t] = alpha[b, t, m] *
// output_scale[b, t] (reference fm_scan.py:116,118-119,130: two products, two transposed
// copies and a subtraction). The reference's `update_weight = alpha * update_scale` is a tensor
// of the storage type and `1.0 - update_weight` another: the product is rounded to T, and one
// minus the rounded product is rounded to T again. The same two roundings are made here (a gate
// near one decides a decay: it has to be the gate the reference forms, bit for bit); the
// multiply and the subtraction are kept apart (no fused multiply-add), so that float32 gets the
// two roundings of its two operations as well. read is one product, one rounding.
// 64 x 64 tiles of (t, m) through LDS. grid: B * tiles_t * tiles_m.
__device__ __forceinline__ float product_rounded(float a, float b) {
#pragma clang fp contract(off)  // a product of its own, never one half of a fused multiply-add
    return a * b;
}

template <typename T>
__global__ __launch_bounds__(256) void layer_prepare_kernel(
    const T* __restrict__ alpha /* (B, L, M) */, const T* __restrict__ update_scale /* (B, L) */,
    const T* __restrict__ output_scale /* (B, L) */, T* __restrict__ gates /* (B, M, L) */,
    T* __restrict__ read /* (B, M, L) */, int64_t L, int64_t M, int32_t tiles_t, int32_t tiles_m) {
    __shared__ float tg[64][65], tr[64][65];
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    const int64_t per_b = (int64_t)tiles_t * tiles_m;
    const int64_t b = blockIdx.x / per_b;
    const int64_t rest = blockIdx.x - b * per_b;
    const int64_t t0 = (rest / tiles_m) * 64, m0 = (rest % tiles_m) * 64;
#pragma unroll 4
    for (int i = w; i < 64; i += 4) {
        const int64_t t = t0 + i;
        if (t < L && m0 + lane < M) {
            const float a = (float)alpha[(b * L + t) * M + m0 + lane];
            const T update_weight = (T)product_rounded(a, (float)update_scale[b * L + t]);
            tg[i][lane] = 1.0f - (float)update_weight;
            tr[i][lane] = product_rounded(a, (float)output_scale[b * L + t]);
        }
    }
    __syncthreads();
#pragma unroll 4
    for (int i = w; i < 64; i += 4) {
        const int64_t m = m0 + i;
        if (m < M && t0 + lane < L) {
            gates[(b * M + m) * L + t0 + lane] = (T)tg[lane][i];
            read[(b * M + m) * L + t0 + lane] = (T)tr[lane][i];
        }
    }
}

// The gradients of those lines: with dg = sum over the G partials of the gates' gradient
// and dr the gradient of read (both (B, M, L), float32),
//   alpha_grad[b,t,m] = dr * output_scale - dg * update_scale
//   update_scale_grad[b,t] = -sum_m dg * alpha,   output_scale_grad[b,t] = sum_m dr * alpha.
// A block is one b and 64 consecutive t; its four waves share the m of each 64-wide tile.
template <typename T>
__global__ __launch_bounds__(256) void layer_finish_kernel(
    const float* __restrict__ gate_grad_partial /* (B, M, G, L) */, int32_t G,
    const float* __restrict__ read_grad /* (B, M, L) */, const T* __restrict__ alpha /* (B, L, M) */,
    const T* __restrict__ update_scale, const T* __restrict__ output_scale, T* __restrict__ alpha_grad,
    T* __restrict__ update_scale_grad, T* __restrict__ output_scale_grad, int64_t L, int64_t M,
    int32_t tiles_t) {
    __shared__ float ta[64][65], td[64][65], red[2][4][64];
    const int lane = threadIdx.x & 63;
    const int w = threadIdx.x >> 6;
    const int64_t b = blockIdx.x / tiles_t;
    const int64_t t0 = (blockIdx.x - b * tiles_t) * 64;
    const int64_t t = t0 + lane;  // the step this lane owns in the (m, t) view
    const float us = t < L ? (float)update_scale[b * L + t] : 0.0f;
    const float os = t < L ? (float)output_scale[b * L + t] : 0.0f;
    float d_us = 0.0f, d_os = 0.0f;
    for (int64_t m0 = 0; m0 < M; m0 += 64) {
        __syncthreads();  // the tiles of the pass before are no longer read
#pragma unroll 4
        for (int i = w; i < 64; i += 4)  // alpha tile, rows are steps
            ta[i][lane] = (t0 + i < L && m0 + lane < M) ? (float)alpha[(b * L + t0 + i) * M + m0 + lane] : 0.0f;
        __syncthreads();
#pragma unroll 2
        for (int i = w; i < 64; i += 4) {  // row i of this pass: slot m0 + i, lanes are steps
            const int64_t m = m0 + i;
            float dg = 0.0f, dr = 0.0f;
            if (m < M && t < L) {
                const float* __restrict__ p = gate_grad_partial + ((b * M + m) * G) * L + t;
                float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};  // eight loads in flight per lane
                int32_t g = 0;
                for (; g + 8 <= G; g += 8) {
#pragma unroll
                    for (int u = 0; u < 8; ++u) acc[u] += p[(int64_t)(g + u) * L];
                }
                for (; g < G; ++g) acc[0] += p[(int64_t)g * L];
                dg = ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
                dr = read_grad[(b * M + m) * L + t];
            }
            const float a = ta[lane][i];
            td[lane][i] = dr * os - dg * us;
            d_us -= dg * a;
            d_os += dr * a;
        }
        __syncthreads();
#pragma unroll 4
        for (int i = w; i < 64; i += 4)
            if (t0 + i < L && m0 + lane < M) alpha_grad[(b * L + t0 + i) * M + m0 + lane] = (T)td[i][lane];
    }
    red[0][w][lane] = d_us;
    red[1][w][lane] = d_os;
    __syncthreads();
    if (w == 0 && t < L) {
        update_scale_grad[b * L + t] = (T)(red[0][0][lane] + red[0][1][lane] + red[0][2][lane] + red[0][3][lane]);
        output_scale_grad[b * L + t] = (T)(red[1][0][lane] + red[1][1][lane] + red[1][2][lane] + red[1][3][lane]);
    }
}

}  // namespace fmscan
