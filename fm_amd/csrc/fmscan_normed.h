// Forward scan and RMS norm of the Factorization-Memory layer in one kernel (reference
// fm/scan/fm_scan.py:121-127: fm_scan, then states * rsqrt(mean(states^2, dim=2) + eps)):
// the scanned states never reach memory, only the normalised ones the layer returns.
#pragma once

#include "fmscan_kernels.h"

namespace fmscan {

// A block is one memory slot (b, m) with all its D rows: wave w owns the J consecutive rows
// d = w*J .. w*J + J - 1 (NW * J >= D). The block walks the tiles of the sequence from the
// first to the last. In a tile every wave scans its J rows one after the other (the gate
// half of the wave scan once for all of them), rounds the states to the storage type as a
// stored state would be, keeps them packed in registers and adds up their squares; the
// waves' sums meet in LDS, where each wave adds one slice of the tile over all waves and
// turns it into inv_rms[b, m, t] = rsqrt(mean_d h^2 + eps) (stored as float32: the
// read-out's gradient takes it); then every wave scales the states it holds and stores
// them. Two barriers per tile. Only the gates and tokens are read (from the caches
// mostly: the tokens serve all M slots of a batch element) and one (B, M, D, L) tensor is
// written, against one written and read twice plus one more written when the scan, the sum
// of squares and the scaling are separate kernels.
// Needs 16-byte aligned rows (vector access only).
//
// WHOLE == false, for D beyond what one block holds: a block is NW * J consecutive rows of a
// slot (blockIdx = ((b * DB + db) * M + m): the M blocks that read the same token rows follow
// each other, and every XCD takes a contiguous range of blocks); it stores the scanned states
// as they are and, in place of inv_rms, the sum of squares over its rows,
// inv_rms[(b * M + m) * DB + db][t]: (B, M, DB, L) partial sums that sumsq_finish_kernel turns
// into inv_rms. One barrier per tile. The sum of squares then costs no pass over the states.
//
// nseg > 1, for few slots and long rows: the sequence is cut into nseg segments of seg_tiles tiles and a
// block is one segment of a slot (blockIdx = (b, segment, m)). The state that enters a segment comes
// from the step pairs of the segments before it, which scan_aggregate_kernel has left in seg_pairs (the
// first pass of the segmented scan kernels: it reads only the gates and tokens, which are small here).
template <typename T, int J, int NW, bool WHOLE = true>
__global__ __launch_bounds__(64 * NW) void scan_forward_normed_kernel(
    const T* __restrict__ gates, const T* __restrict__ tokens, const T* __restrict__ h0,
    T* __restrict__ states_n /* (B, M, D, L) */, float* __restrict__ inv_rms /* (B, M, L) */, int32_t M,
    int32_t D, int64_t L, float eps, int32_t DB, int32_t nseg, int32_t seg_tiles,
    const float2* __restrict__ seg_pairs /* (B * M * D, nseg): scan_aggregate_kernel's, or NULL */) {
    constexpr int E = Elem<T>::E;
    constexpr int TILE = E * 64;
    constexpr int SLICE = TILE / NW;  // elements of a tile's sum of squares each wave finishes
    static_assert(TILE % NW == 0 && SLICE <= 64, "a wave finishes at most one element per lane");
    __shared__ float part[2][NW][TILE];  // every wave's sum of squares over its rows
    __shared__ float scale[2][TILE];     // inv_rms of the tile

    const int lane = threadIdx.x & 63;
    const int w = uniform((int)(threadIdx.x >> 6));
    // Blocks go to the 8 XCDs (each with its own L2) round robin. The M blocks of one b read
    // the same tokens, so they are renumbered to share an XCD.
    uint32_t id = blockIdx.x;
    if (gridDim.x % 8u == 0u) id = (id % 8u) * (gridDim.x / 8u) + id / 8u;
    // the slot runs fastest, then the segment: the M blocks of one stretch of b's tokens follow each other
    const uint32_t m_of = id % (uint32_t)M;
    uint32_t rest = id / (uint32_t)M;
    int32_t seg = 0;
    if (nseg > 1) {
        seg = uniform((int)(rest % (uint32_t)nseg));
        rest /= (uint32_t)nseg;
    }
    int32_t db = 0;
    if constexpr (!WHOLE) {
        db = uniform((int)(rest % (uint32_t)DB));
        rest /= (uint32_t)DB;
    }
    const int64_t b = uniform((int)rest);
    const int64_t bm = (int64_t)uniform((int)(rest * (uint32_t)M + m_of));  // b * M + m
    const int32_t d0 = (db * NW + w) * J;
    const int32_t ntiles = (int32_t)((L + TILE - 1) / TILE);
    const int32_t lane_off = lane * E;
    auto d_of = [&](int j) { return d0 + j < D ? d0 + j : D - 1; };  // a row past D is loaded as D - 1 and dropped
    auto counted = [&](int j) { return d0 + j < D; };                // the same for the whole wave

    // the tiles of this block: all of them, or those of its segment
    const int32_t k_lo = seg * seg_tiles;
    const int32_t k_hi = nseg > 1 && k_lo + seg_tiles < ntiles ? k_lo + seg_tiles : ntiles;
    if (k_lo >= ntiles) return;  // the whole block (the host cuts so that this does not happen)

    float carry[J];
#pragma unroll
    for (int j = 0; j < J; ++j) {
        const int64_t row = bm * D + d_of(j);
        carry[j] = h0 ? Elem<T>::widen(h0[row]) : 0.0f;
        for (int32_t sg = 0; sg < seg; ++sg) {  // the segments before this one, oldest first
            const float2 p = seg_pairs[row * nseg + sg];
            carry[j] = __builtin_fmaf(p.x, carry[j], p.y);
        }
    }

    // lane offset (elements) inside tile k, clamped into the row (a chunk past the end reads the last one)
    auto lane_elems = [&](int32_t k) {
        const int64_t left = L - (int64_t)k * TILE;
        const int32_t rem = left < TILE ? (int32_t)left : TILE;
        return (uint32_t)(lane_off < rem ? lane_off : rem - E);
    };
    // Token tiles in flight: RING of them (a row's tile is loaded RING rows ahead of its use: the first
    // rows of the next tile while the last rows of this one are worked on).
    constexpr int RING = J >= 8 ? J / 2 : J;
    struct Loads {
        u32x4 g;
        u32x4 x[RING];
    };
    // k beyond the last tile: the last tile again (not used)
    auto fetch_gates = [&](Loads& q, int32_t k) {
        k = k < ntiles ? k : ntiles - 1;
        q.g = load16<T, false>(gates + bm * L + (int64_t)k * TILE + lane_elems(k));
    };
    auto fetch_tokens = [&](Loads& q, int32_t k, int j) {
        k = k < ntiles ? k : ntiles - 1;
        q.x[j % RING] = load16<T, false>(tokens + (b * D + d_of(j)) * L + (int64_t)k * TILE + lane_elems(k));
    };

    // The loads run ahead (the gates a tile, the tokens RING rows), each into the registers it was
    // just unpacked from: a second set of registers handed over at the end of a tile would make that
    // hand-over wait for the tile's stores as well.
    Loads q;
    fetch_gates(q, k_lo);
#pragma unroll
    for (int j = 0; j < RING; ++j) fetch_tokens(q, k_lo, j);
    int parity = 0;
    wait_for_loads();
    // One tile. `whole`: it lies wholly inside the row and nothing is tested per lane, so that
    // every pass of the loop over such tiles issues the same loads and stores, and the waits for
    // loads can be counted past the stores in flight. The last tile of a row that is not a
    // whole number of tiles is done after the loop, with the tests.
    auto tile = [&](int32_t k, auto whole) __attribute__((always_inline)) {
        constexpr bool WHOLE_TILE = decltype(whole)::value;
        const int64_t tw = (int64_t)k * TILE;
        const bool inside = WHOLE_TILE || tw + lane_off < L;  // this lane's chunk lies in the row (tiles are whole chunks)

        float g[E];
        Elem<T>::unpack(q.g, g);
        fetch_gates(q, k + 1);
        if constexpr (!WHOLE_TILE) {
#pragma unroll
            for (int i = 0; i < E; ++i) g[i] = inside ? g[i] : 1.0f;
        }
        float a = g[0];
#pragma unroll
        for (int i = 1; i < E; ++i) a *= g[i];
        const GateLevels levels = scan_gates(a);

        u32x4 held[J];
        float sumsq[E];
#pragma unroll
        for (int i = 0; i < E; ++i) sumsq[i] = 0.0f;
#pragma unroll
        for (int j = 0; j < J; ++j) {
            float u[E];
            Elem<T>::unpack(q.x[j % RING], u);
            if (j + RING < J) fetch_tokens(q, k, j + RING);
            else fetch_tokens(q, k + 1, j + RING - J);
#pragma unroll
            for (int i = 0; i < E; ++i) u[i] = __builtin_fmaf(-g[i], u[i], u[i]);  // (1 - g) x, one rounding
            float bb = u[0];
#pragma unroll
            for (int i = 1; i < E; ++i) bb = __builtin_fmaf(g[i], bb, u[i]);
            scan_values(bb, levels);
            const float eb = dpp<kWaveShr1>(0.0f, bb);
            const float tb = lane63(bb);
            float h = __builtin_fmaf(levels.ea, carry[j], eb);
            carry[j] = __builtin_fmaf(levels.ta, carry[j], tb);
            float o[E];
#pragma unroll
            for (int i = 0; i < E; ++i) {
                h = __builtin_fmaf(g[i], h, u[i]);
                o[i] = h;
            }
            held[j] = Elem<T>::pack(o);
            if (counted(j)) {
                if constexpr (!WHOLE) {
                    if (inside)
                        __builtin_nontemporal_store(held[j], reinterpret_cast<u32x4*>(states_n + (bm * D + d0 + j) * L +
                                                                                      tw + lane_off));
                }
                Elem<T>::unpack(held[j], o);  // the norm sees the states as they would be stored
#pragma unroll
                for (int i = 0; i < E; ++i) sumsq[i] = __builtin_fmaf(o[i], o[i], sumsq[i]);
            }
        }

        // the waves' sums meet: every wave lays its own out in time order, then finishes a slice
        float* mine = &part[parity][w][lane_off];
#pragma unroll
        for (int i = 0; i < E; i += 4)
            *reinterpret_cast<float4*>(mine + i) = make_float4(sumsq[i], sumsq[i + 1], sumsq[i + 2], sumsq[i + 3]);
        __syncthreads();
        if (lane < SLICE) {
            const int e = w * SLICE + lane;
            float s = 0.0f;
#pragma unroll
            for (int v = 0; v < NW; ++v) s += part[parity][v][e];  // fixed order: run-to-run identical
            if constexpr (WHOLE) {
                s = 1.0f / __builtin_sqrtf(s / (float)D + eps);
                scale[parity][e] = s;
                if (WHOLE_TILE || tw + e < L) inv_rms[bm * L + tw + e] = s;
            } else {
                if (WHOLE_TILE || tw + e < L) inv_rms[(bm * DB + db) * L + tw + e] = s;
            }
        }
        if constexpr (!WHOLE) {
            parity ^= 1;  // the other buffer next: no wave writes this one again before all have read it
            return;
        }
        __syncthreads();
        float r[E];
#pragma unroll
        for (int i = 0; i < E; i += 4) {
            const float4 v = *reinterpret_cast<const float4*>(&scale[parity][lane_off + i]);
            r[i] = v.x; r[i + 1] = v.y; r[i + 2] = v.z; r[i + 3] = v.w;
        }
        if (inside) {
#pragma unroll
            for (int j = 0; j < J; ++j) {
                if (counted(j)) {
                    float o[E];
                    Elem<T>::unpack(held[j], o);
#pragma unroll
                    for (int i = 0; i < E; ++i) o[i] *= r[i];
                    __builtin_nontemporal_store(Elem<T>::pack(o),
                                                reinterpret_cast<u32x4*>(states_n + (bm * D + d0 + j) * L + tw + lane_off));
                }
            }
        }
        parity ^= 1;
    };
    const int32_t whole_tiles = (int32_t)(L / TILE);
    const int32_t k_whole = k_hi < whole_tiles ? k_hi : whole_tiles;
    for (int32_t k = k_lo; k < k_whole; ++k) tile(k, std::true_type{});
    if (whole_tiles < k_hi) tile(whole_tiles, std::false_type{});  // (k_hi == ntiles: the row's last, short tile)
}

// inv_rms[r][t] = rsqrt(sum_g partial[r][g][t] / D + eps) for the (B, M, G, L) partial sums of
// squares the kernel above leaves (r = b * M + m). One thread per (r, t).
__global__ __launch_bounds__(256) void sumsq_finish_kernel(const float* __restrict__ partial, float* __restrict__ inv_rms,
                                                           int64_t rows, int32_t G, int64_t L, int32_t D, float eps) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * L) return;
    const int64_t r = i / L, t = i - r * L;
    float s = 0.0f;
    for (int32_t g = 0; g < G; ++g) s += partial[(r * G + g) * L + t];
    inv_rms[i] = 1.0f / __builtin_sqrtf(s / (float)D + eps);
}

}  // namespace fmscan
