// The backward scan of Factorization-Memory shapes (M > 1 and D > 1) with the sums over D
// and M inside, and its forms for the layer around the scan. Building blocks (lanes, the
// wave scan): fmscan_kernels.h, fmscan_device.h.
#pragma once

#include "fmscan_kernels.h"

namespace fmscan {

// ---- backward with the D and M sums inside -------------------------------------------
// For M > 1 and D > 1 the per-pair gradients are only ever summed: d_gates = sum over d,
// d_tokens = sum over m (reference fm/scan/fm_scan.py:76-78; its kernel writes both
// (B, M, D, L) tensors "to avoid atomicAdd", fm_scan.cuh:200-207, and torch.sum reads them
// back). This kernel never writes them.
//
// A block is one batch element b and J consecutive d; its NW waves split the M memory
// slots between them (Mw consecutive slots each). A wave walks the tiles of the sequence
// from the last to the first and, in each tile, its Mw x J rows (b, m, d): slot after slot,
// and for a slot the J rows one after the other. So
//   * what depends on the slot only (gates, the layer's coefficient vectors, the gate half
//     of the wave scan) is prepared once per J rows;
//   * the gate gradient of a slot, summed over the J rows, builds up in registers and is
//     stored as float32 partial gate_partial[b, m, group, :]; the caller adds the
//     ceil(D / J) groups;
//   * the token gradients of the J rows, summed over the wave's slots, build up in
//     registers over the whole tile; at its end the waves of the block hand them on from
//     wave to wave through LDS (each adds its own; fixed order, hence deterministic) and the
//     last stores d_tokens[b, d, tile].
// No wave waits for another except in that hand-over, once per tile. The running state of
// every row lives in LDS (one float per row, private to its wave). Loads run ahead: the
// per-slot vectors by one slot, the rows' tiles by J rows, or by J / 2 where J = 8 and the
// elements have 2 bytes (the first rows of the next slot, or of the first slot of the tile
// before, are then loaded while the last rows of this one are worked on: half the registers
// for tiles in flight, which the compiler turns into a shorter schedule of the whole step);
// every step issues the same loads whatever its position (addresses are clamped into the
// tensors), so the count of loads in flight is a compile-time number. (The per-slot vectors
// of the step at work and of the step after it sit in two sets of registers that swap roles,
// steps come in pairs; what a step needs only at its end, the layer form's rms vector, is
// loaded at its start.)
// HBM traffic per element of (B, M, D, L): G and h (2s), or the normalised states alone in
// the layer form (s), plus 4/J bytes of partials, against 6s for the unfused kernel plus the
// two torch.sum passes.
//
// LAYER: the gradient that arrives at the states is not read but made on the spot from what
// the layer around the scan holds (reference fm/scan/fm_scan.py:124-131 differentiated):
//   G[b,m,d,t] = coef_out[b,m,t] * layer_out_grad[b,d,t] - coef_self[b,m,t] * out_grad[b,m,d,t]
// where `out_grad` then carries the normalised states; the (B, M, D, L) gradient tensor is
// never written or read. LAYER == 2: the scanned states themselves are not read either
// (h_saved is NULL) but taken back from the normalised ones, h = out_grad * rms, so that
// the layer has to keep nothing of size (B, M, D, L) besides the states it returns.
// coef_out, coef_self and rms are float32.
//
// split > 1, for problems with too few (b, group of d) pairs to fill the GPU: the M slots of a batch
// element are dealt to `split` blocks instead of one. The caller states it as a problem of B * split
// batch elements of M / split slots each, which is the same memory for everything indexed by (b, m);
// the kernel only has to find the token rows (and the layer's output-gradient rows) of its batch element
// at b / split, and to leave its token gradient, a sum over its own slots only, as float32 in
// token_partial[b / split, d, b % split, :] for a sum over the blocks of a batch element that rounds once.
//
// MODE 1 and 2, for few blocks and long rows (not PLAIN): the sequence is cut into nseg segments of
// seg_tiles tiles and a block takes one segment of its rows (blockIdx = ((b, segment), group)). What arrives
// at a segment from the steps after it comes from the step pairs of the later segments: MODE 2 is the pass
// that makes them (for every row and segment but the first: the segment's gate product and what leaves it
// when nothing enters; no gradient is accumulated or stored), MODE 1 the kernel proper started inside the row.
template <typename T, int J, int NW, bool PLAIN, int LAYER, int MODE = 0>
__global__ __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(2))) void scan_backward_reduced_kernel(
    const T* __restrict__ gates, const T* __restrict__ out_grad, const T* __restrict__ first_prop_grad,
    T* __restrict__ token_grad /* (B, D, L) */, const T* __restrict__ h_saved,
    const T* __restrict__ tokens, float* __restrict__ gate_partial /* (B, M, NG, L) */,
    const T* __restrict__ h0, T* __restrict__ h0_grad, const float* __restrict__ coef_out /* (B, M, L) */,
    const float* __restrict__ coef_self /* (B, M, L) */, const T* __restrict__ layer_out_grad /* (B, D, L) */,
    const float* __restrict__ rms /* (B, M, L): 1 / inv_rms */, int32_t M, int32_t D, int64_t L, int32_t Mw,
    float* __restrict__ token_partial /* (B / split, D, split, L), or NULL */, int32_t split,
    int32_t nseg, int32_t seg_tiles, float2* __restrict__ seg_pairs /* (B * M * D, nseg); MODE 1: read, 2: written */) {
    static_assert(MODE == 0 || !PLAIN, "rows are cut in the Factorization-Memory form only");
    constexpr int E = Elem<T>::E;
    constexpr int TILE = E * 64;
    extern __shared__ float lds[];
    constexpr int SH = (J + NW - 1) / NW;  // token rows a wave loads for the block (the last waves fewer, or none)
    float* handover = lds;                    // [2][J][E / 4][64][4]: token gradients on their way down the waves
    u32x4* shared_xy = reinterpret_cast<u32x4*>(lds + 2 * J * TILE);  // [2][J][2][64]: tokens and layer_out_grad of a tile
    float* carries = lds + 2 * J * TILE + 2 * J * 2 * 64 * 4;         // [NW][Mw * J]
    float* staging = carries + NW * Mw * J;                          // [NW][TILE], 8-element chunks only: see the partials' stores
    [[maybe_unused]] float* gate_products = staging + NW * TILE;     // [NW][Mw] (MODE 2): a segment's gate product, per slot

    const int lane = threadIdx.x & 63;
    const int w = uniform((int)(threadIdx.x >> 6));
    const int32_t NG = (D + J - 1) / J;
    // Blocks go to the 8 XCDs (each with its own L2) round robin. The blocks of one b read the
    // same gates, tokens and coefficient vectors, so they are renumbered to share an XCD: XCD x
    // takes the x-th eighth of the (b, group) pairs.
    uint32_t id = blockIdx.x;
    if (gridDim.x % 8u == 0u) id = (id % 8u) * (gridDim.x / 8u) + id / 8u;
    // Cut rows: the groups of one (b, segment) follow each other (they read the same stretch of the gates
    // and coefficient vectors), then the blocks that share b's tokens, then the segments.
    [[maybe_unused]] int32_t seg = 0;
    if constexpr (MODE != 0) {
        const uint32_t g = id % (uint32_t)NG, r = id / (uint32_t)NG;
        const uint32_t s = r % (uint32_t)split, r2 = r / (uint32_t)split;
        seg = uniform((int)(r2 % (uint32_t)nseg));
        id = ((r2 / (uint32_t)nseg) * (uint32_t)split + s) * (uint32_t)NG + g;
    }
    const int64_t b = uniform((int)(id / (uint32_t)NG));
    const int32_t grp = uniform((int)id - (int32_t)b * NG);
    const int32_t d0 = grp * J;
    const int32_t m0 = w * Mw;
    const int32_t mcount = uniform(M - m0 < 0 ? 0 : (M - m0 < Mw ? M - m0 : Mw));  // slots of this wave
    const int32_t ntiles = (int32_t)((L + TILE - 1) / TILE);
    // the tiles of this block: all of them, or those of its segment
    const int32_t k_lo = MODE != 0 ? seg * seg_tiles : 0;
    const int32_t k_hi = MODE != 0 && k_lo + seg_tiles < ntiles ? k_lo + seg_tiles : ntiles;
    if constexpr (MODE != 0) {
        if (k_lo >= ntiles) return;  // the whole block (the host cuts so that this does not happen)
    }
    if constexpr (MODE == 2) {
        if (seg == 0) return;  // nothing lies before the first segment: its pair is never asked for
    }
    const int32_t lane_off = (63 - lane) * E;  // lane l owns the chunk l chunks before the end of the tile
    float* mycarry = carries + w * Mw * J;
    const int32_t rows_here = uniform(D - d0 < J ? D - d0 : J);  // rows of this block that exist (the last group may be short)
    const int64_t b_tok = split > 1 ? uniform((int)((uint32_t)b / (uint32_t)split)) : b;  // whose tokens these are

    // (the trip count is the same for all lanes and only the access is predicated: a loop that
    // some lanes skip would leave the values it shares with the code below in vector registers,
    // and every address would then be computed there)
    for (int32_t base = 0; base < mcount * J; base += 64) {
        const int32_t idx = base + lane;
        const int32_t mi = idx / J, j = idx - mi * J;
        const int32_t d = d0 + j < D ? d0 + j : D - 1;
        if (idx < mcount * J) {
            const int64_t row = (b * M + m0 + mi) * D + d;
            float c = 0.0f;
            if constexpr (MODE != 2) {
                c = first_prop_grad ? Elem<T>::widen(first_prop_grad[row]) : 0.0f;
                if constexpr (MODE == 1) {
                    for (int32_t sg = nseg - 1; sg > seg; --sg) {  // the segments after this one, from the row's end
                        const float2 p = seg_pairs[row * nseg + sg];
                        c = __builtin_fmaf(p.x, c, p.y);
                    }
                }
            }
            mycarry[idx] = c;
        }
    }
    if constexpr (MODE == 2) {
        for (int32_t mi = lane; mi < mcount; mi += 64) gate_products[w * Mw + mi] = 1.0f;
    }
    // Everything here is wave-uniform. A row j of the block's group past the last d (last group) is
    // loaded like any other (as row D - 1), never accumulated or stored.
    auto slot_of = [&](int32_t mi) {  // clamped: a wave without slots still issues (unused) loads
        const int32_t m = m0 + mi;
        return m < M ? m : M - 1;
    };


    // What a step loads, exactly as it arrives: anything computed from a loaded value at
    // the time of the load would have to be finished before the loop comes round, which
    // means waiting for every load in flight.
    // Where the saved states are at hand (LAYER != 2) and there are tokens (!PLAIN), the states
    // of a tile are not read but made again from its gates and tokens and the one saved state
    // before the tile, as scan_backward_kernel does.
    constexpr bool REMAKE = LAYER != 2 && !PLAIN && MODE != 2;  // (pass one has no use for the states)
    const uint32_t vzero = opaque_zero();
    struct Row {
        u32x4 a;   // out_grad, or the normalised states (LAYER)
        u32x4 h;   // saved states (PLAIN only)
        T hb;      // what stands before the tile in the row that `h` comes from
        T h_first; // REMAKE, first tile: the saved h[0] (elsewhere: hb again)
    };
    struct Slot {
        u32x4 g;
        FloatChunk<E> co, cs;  // LAYER
    };
    struct Rms {  // LAYER == 2; needed at the end of a step only, so loaded at its start and not a step ahead
        FloatChunk<E> rr;
        float hbr;  // rms at the step hb belongs to
    };
    // lane offset (elements) inside tile k, clamped into the row (a chunk past the end reads the last one)
    auto lane_elems = [&](int32_t k) {
        const int64_t left = L - (int64_t)k * TILE;
        const int32_t rem = left < TILE ? (int32_t)left : TILE;
        return (uint32_t)(lane_off < rem ? lane_off : rem - E);
    };
    // What the addresses of a step's J rows share, all of it wave-uniform: made once per step.
    struct Place {
        int64_t row0;  // (b, slot, d0) as a row of the (B, M, D) tensors
        int64_t base;  // where that row's tile starts in the (B, M, D, L) tensors
        int32_t k;     // the tile
    };
    auto place_of = [&](int32_t k, int32_t mi) {
        Place p;
        p.row0 = (b * M + slot_of(mi)) * D + d0;
        p.base = p.row0 * L + (int64_t)k * TILE;
        p.k = k;
        return p;
    };
    // (the tile comes from a uniform base and a 32-bit lane offset: no vector address arithmetic)
    auto fetch_row = [&](Row& r, const Place& p, int j) {
        const int32_t jc = j < rows_here ? j : rows_here - 1;  // (past the last d: row D - 1 again)
        const int64_t base = p.base + (int64_t)jc * L;
        const uint32_t lo = lane_elems(p.k) * (uint32_t)sizeof(T);
        r.a = load16<char, true>(reinterpret_cast<const char*>(out_grad + base) + lo);
        r.h = u32x4{0u, 0u, 0u, 0u};
        if constexpr (LAYER != 2 && !REMAKE) r.h = load16<char, true>(reinterpret_cast<const char*>(h_saved + base) + lo);
        const T* __restrict__ hsrc = LAYER == 2 ? out_grad : h_saved;
        // h just before the tile (h[-1] at the start of the row): one address for the whole wave
        const T* src = p.k > 0 ? hsrc + (base - 1) : (h0 != nullptr ? h0 + (p.row0 + jc) : hsrc + base);
        r.hb = load_by_wave(src, vzero);
        r.h_first = T(0);
        // (no new cache line except in the first tile)
        if constexpr (REMAKE) r.h_first = load_by_wave(hsrc + (p.k > 0 ? base - 1 : base), vzero);
    };
    auto fetch_slot = [&](Slot& s, int32_t k, int32_t mi) {
        const int64_t tw = (int64_t)k * TILE;
        const uint32_t lo = lane_elems(k);
        const int64_t base = (b * M + slot_of(mi)) * L + tw;
        s.g = load16<T, false>(gates + base + lo);
        if constexpr (LAYER != 0) {
            s.co = load_float_chunk<E>(coef_out + base + lo);
            s.cs = load_float_chunk<E>(coef_self + base + lo);
        }
    };
    auto fetch_rms = [&](Rms& s, int32_t k, int32_t mi) {
        const int64_t tw = (int64_t)k * TILE;
        const int64_t base = (b * M + slot_of(mi)) * L + tw;
        s.rr = load_float_chunk<E>(rms + base + lane_elems(k));
        s.hbr = load_by_wave(rms + (base - (tw > 0 ? 1 : 0)), vzero);
    };
    // The steps of a tile come in pairs (below), so an odd count of slots is padded with one step
    // that only loads.
    const int32_t mpad = (mcount + 1) & ~1;
    // the position one step ahead of (k, mi): the next slot of the tile, else the first slot of
    // the tile before; before the first tile there is nothing: stay (the loads are not used)
    auto ahead = [&](int32_t& k, int32_t& mi) {
        if (mi + 1 < mpad) {
            ++mi;
        } else if (k > k_lo) {
            --k;
            mi = 0;
        }
    };

    // The J token rows of the block (and the J rows of the layer's output gradient) are the same
    // for every slot and every wave: each tile of them is loaded once per block, about J / NW rows
    // per wave, and passed through LDS, a tile ahead of its use.
    constexpr bool kSharedX = !PLAIN && MODE != 2, kSharedY = LAYER != 0;
    struct TokenShare {
        u32x4 x[SH], y[SH];
    };
    auto fetch_share = [&](TokenShare& ts, int32_t k) {
        const int64_t tw = (int64_t)k * TILE;
        const uint32_t lo = lane_elems(k);
#pragma unroll
        for (int s = 0; s < SH; ++s) {
            const int32_t jj = w * SH + s < J ? w * SH + s : J - 1;  // (a wave beyond the J rows loads the last again, unused)
            const int32_t d = d0 + jj < D ? d0 + jj : D - 1;
            const int64_t off = (b_tok * D + d) * L + tw + lo;
            ts.x[s] = ts.y[s] = u32x4{0u, 0u, 0u, 0u};
            if constexpr (kSharedX) ts.x[s] = load16<T, false>(tokens + off);
            if constexpr (kSharedY) ts.y[s] = load16<T, false>(layer_out_grad + off);
        }
    };
    auto publish_share = [&](const TokenShare& ts, int par) {
#pragma unroll
        for (int s = 0; s < SH; ++s) {
            const int32_t jj = w * SH + s;
            if (jj >= J) break;
            if constexpr (kSharedX) shared_xy[((par * J + jj) * 2 + 0) * 64 + lane] = ts.x[s];
            if constexpr (kSharedY) shared_xy[((par * J + jj) * 2 + 1) * 64 + lane] = ts.y[s];
        }
    };

    // The rows' tiles in flight: RING of them, so a row is loaded RING rows ahead of its use (the first
    // rows of the next step from the last rows of this one).
    constexpr int RING = (J >= 8 && sizeof(T) == 2) ? J / 2 : J;
    Row rows[RING];
    // The per-slot vectors of the step at work and of the step after it, which is loading, sit in
    // two sets of registers that swap roles from step to step: handing one set over to the other
    // at the end of a step would have to wait for every load and store in flight.
    Slot slot_a, slot_b;
    int32_t kf = k_hi - 1, mf = 0;  // the step after the one at work: where the loads that run ahead are
    fetch_slot(slot_a, kf, mf);
    Place place_next = place_of(kf, mf), place_now = place_next;
#pragma unroll
    for (int j = 0; j < RING; ++j) fetch_row(rows[j], place_next, j);

    int parity = 0;
    if constexpr (kSharedX || kSharedY) {
        TokenShare first;
        fetch_share(first, k_hi - 1);
        publish_share(first, parity);
    }
    __syncthreads();  // carries and the first tile of the shared rows are in place

    for (int32_t k = k_hi - 1; k >= k_lo; --k) {
        const int64_t tw = (int64_t)k * TILE;
        TokenShare upcoming;  // the tile before this one, on its way to LDS
        if constexpr (kSharedX || kSharedY) fetch_share(upcoming, k > k_lo ? k - 1 : k_lo);
        const bool inside = tw + lane_off < L;  // this lane's chunk lies in the row (tiles are whole chunks)
        const bool ragged = tw + TILE > L;      // the whole wave: only the row's last tile can end early
        float dtok[J][E];
#pragma unroll
        for (int j = 0; j < J; ++j) {
#pragma unroll
            for (int i = 0; i < E; ++i) dtok[j][i] = 0.0f;
        }
        auto slot_step = [&](const Slot& cur, Slot& next_slot, int32_t mi) __attribute__((always_inline)) {
            ahead(kf, mf);
            place_now = place_next;
            place_next = place_of(kf, mf);
            fetch_slot(next_slot, kf, mf);
            if (mi >= mcount) {  // the padding step of an odd count
#pragma unroll
                for (int j = 0; j < RING; ++j) fetch_row(rows[j], place_next, j);
                return;
            }
            [[maybe_unused]] Rms rms_now;
            if constexpr (LAYER == 2 && MODE != 2) fetch_rms(rms_now, k, mi);

            // per slot: gates (1 where there is no step: identity), coefficients (0 there: no gradient)
            float g[E], co[E], cs[E];
            Elem<T>::unpack(cur.g, g);
            if constexpr (LAYER != 0) {
                spread<E>(cur.co, co);
                spread<E>(cur.cs, cs);
            }
            if (ragged) {
#pragma unroll
                for (int i = 0; i < E; ++i) {
                    g[i] = inside ? g[i] : 1.0f;
                    if constexpr (LAYER != 0) {
                        co[i] = inside ? co[i] : 0.0f;
                        cs[i] = inside ? cs[i] : 0.0f;
                    }
                }
            }
            [[maybe_unused]] float one_minus_g[E];  // the token gradient's factor, once per slot
#pragma unroll
            for (int i = 0; i < E; ++i) one_minus_g[i] = 1.0f - g[i];
            float a = g[E - 1];
#pragma unroll
            for (int i = E - 2; i >= 0; --i) a *= g[i];
            const GateLevels levels = scan_gates(a);
            if constexpr (MODE == 2) {  // the segment's gate product so far (one value for the whole wave)
                if (lane == 0) gate_products[w * Mw + mi] *= levels.ta;
            }
            // (first tile: the chain of remade states starts at the saved h[0], whatever enters: the
            // first step of lane 63, which owns the start of the row, counts as gate 0, token h[0])
            const bool first_step = k == 0 && lane == 63;
            GateLevelsDown down;
            if constexpr (REMAKE) down = scan_gates_down(first_step ? 0.0f : a);

            // The slot's gate gradient over this group of d is sum_d (h[t-1] - x[t]) * delta[t]. With
            // the states taken back from the normalised ones, h[t-1] = rms[t-1] * n[t-1] and rms
            // belongs to the slot: sum_d n[t-1] * delta[t] is built up (`with_state`), the factor
            // applied once, after the rows; sum_d x[t] * delta[t] separately (`with_token`).
            float with_state[E], with_token[E];
#pragma unroll
            for (int i = 0; i < E; ++i) with_state[i] = with_token[i] = 0.0f;
            float* carry_of = mycarry + mi * J;

            {
#pragma unroll
                for (int j = 0; j < J; ++j) {
                    // (unpacked before the loads of the slot after this one reuse the registers)
                    float G[E], h[E], x[E];
                    Row& held = rows[j % RING];
                    Elem<T>::unpack(held.a, G);
                    // what stands before the tile in the row: a state, or a normalised one (the factor
                    // follows with the slot); at k == 0 the initial state itself, or nothing
                    const float hb = (k > 0 || h0 != nullptr) ? Elem<T>::widen(held.hb) : 0.0f;
                    [[maybe_unused]] const float h_first = Elem<T>::widen(held.h_first);
                    if constexpr (LAYER == 2) {
#pragma unroll
                        for (int i = 0; i < E; ++i) h[i] = G[i];  // G[] holds the normalised state
                    } else if constexpr (!REMAKE) {
                        Elem<T>::unpack(held.h, h);
                    }
                    if (j + RING < J) fetch_row(held, place_now, j + RING);  // further on in this slot
                    else fetch_row(held, place_next, j + RING - J);         // the first rows of the step after
                    // the whole wave: a row past the last d adds nothing. (The count goes through an empty asm so
                    // that the comparison is made here, one scalar compare, and not kept from before the loops as
                    // a lane mask per row: sixteen scalar registers the kernel does not have.)
                    int32_t rows_valid = rows_here;
                    asm volatile("" : "+s"(rows_valid));
                    if (j >= rows_valid) continue;

                    float carry = carry_of[j];
                    if constexpr (LAYER != 0) {
                        float y[E];
                        Elem<T>::unpack(shared_xy[((parity * J + j) * 2 + 1) * 64 + lane], y);
#pragma unroll
                        for (int i = 0; i < E; ++i) G[i] = __builtin_fmaf(-cs[i], G[i], co[i] * y[i]);
                    } else if (ragged) {
#pragma unroll
                        for (int i = 0; i < E; ++i) G[i] = inside ? G[i] : 0.0f;
                    }
                    if constexpr (kSharedX) Elem<T>::unpack(shared_xy[((parity * J + j) * 2 + 0) * 64 + lane], x);
                    float hprev[E];  // the state before each of the chunk's steps
                    if constexpr (REMAKE) {
                        float u[E];
#pragma unroll
                        for (int i = 0; i < E; ++i) u[i] = __builtin_fmaf(-g[i], x[i], x[i]);  // as the forward kernel forms it
                        if (first_step) u[0] = h_first;
                        float fb = u[0];
#pragma unroll
                        for (int i = 1; i < E; ++i) fb = __builtin_fmaf(g[i], fb, u[i]);
                        hprev[0] = state_entering_lane_down(fb, down, hb, lane);
                        hprev[1] = first_step ? u[0] : __builtin_fmaf(g[0], hprev[0], u[0]);
#pragma unroll
                        for (int i = 2; i < E; ++i) hprev[i] = __builtin_fmaf(g[i - 1], hprev[i - 1], u[i - 1]);
                    }

                    // the chunk as one step on what arrives from later steps: c_out = a * c_in + bb
                    float bb = g[E - 1] * G[E - 1];
#pragma unroll
                    for (int i = E - 2; i >= 0; --i) bb = g[i] * (bb + G[i]);
                    scan_values(bb, levels);
                    const float eb = dpp<kWaveShr1>(0.0f, bb);
                    const float tb = lane63(bb);
                    if constexpr (!REMAKE) {
                        hprev[0] = dpp<kWaveShl1>(hb, h[E - 1]);
#pragma unroll
                        for (int i = 1; i < E; ++i) hprev[i] = h[i - 1];
                    }

                    float c = __builtin_fmaf(levels.ea, carry, eb);
                    carry = __builtin_fmaf(levels.ta, carry, tb);
                    if (lane == 0) carry_of[j] = carry;
                    if constexpr (MODE != 2) {
#pragma unroll
                        for (int i = E - 1; i >= 0; --i) {
                            const float delta = G[i] + c;
                            c = g[i] * delta;
                            // token gradient (1 - g) * delta
                            if constexpr (PLAIN) dtok[j][i] += delta;
                            else dtok[j][i] = __builtin_fmaf(one_minus_g[i], delta, dtok[j][i]);
                            with_state[i] = __builtin_fmaf(hprev[i], delta, with_state[i]);
                            if constexpr (!PLAIN) with_token[i] = __builtin_fmaf(x[i], delta, with_token[i]);
                        }
                    }
                }
            }
            if constexpr (MODE == 2) return;  // pass one: the carries are all it is after

            // the slot's gate gradient, summed over this group of d
            float dgate[E];
            if constexpr (LAYER == 2) {
                // rms at the step before each element: the chunk's own values moved up by one, the
                // first from the lane that owns the chunk before (lane 63: from before the tile; at
                // k == 0 what stands there is the initial state itself: factor 1)
                float rr[E];
                spread<E>(rms_now.rr, rr);
                const float before = dpp<kWaveShl1>(k > 0 ? rms_now.hbr : 1.0f, rr[E - 1]);
#pragma unroll
                for (int i = 0; i < E; ++i)
                    dgate[i] = __builtin_fmaf(i > 0 ? rr[i > 0 ? i - 1 : 0] : before, with_state[i], -with_token[i]);
            } else {
#pragma unroll
                for (int i = 0; i < E; ++i) dgate[i] = with_state[i] - with_token[i];
            }
            float* __restrict__ ptile = gate_partial + ((b * M + m0 + mi) * NG + grp) * L + tw;
            if constexpr (E == 4) {
                if (inside) {
                    const u32x4 v = {f2u(dgate[0]), f2u(dgate[1]), f2u(dgate[2]), f2u(dgate[3])};
                    __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(ptile + lane_off));
                }
            } else {
                // A lane holds 8 consecutive floats, 32 bytes: stored as they are, each of the two store
                // instructions would write 16 of every 32 bytes over 2 KiB. Through LDS (private to the wave,
                // whose LDS operations complete in order) every instruction writes 1 KiB without gaps.
                static_assert(E == 4 || E == 8, "chunks of 4 or 8 elements");
                float* mine = staging + w * TILE;
                *reinterpret_cast<float4*>(mine + lane_off) = make_float4(dgate[0], dgate[1], dgate[2], dgate[3]);
                *reinterpret_cast<float4*>(mine + lane_off + 4) = make_float4(dgate[4], dgate[5], dgate[6], dgate[7]);
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                const int32_t valid = L - tw < TILE ? (int32_t)(L - tw) : TILE;  // whole chunks
#pragma unroll
                for (int half = 0; half < 2; ++half) {
                    const int32_t at = half * (TILE / 2) + lane * 4;
                    const float4 v = *reinterpret_cast<const float4*>(mine + at);
                    if (at < valid) {
                        const u32x4 u = {f2u(v.x), f2u(v.y), f2u(v.z), f2u(v.w)};
                        __builtin_nontemporal_store(u, reinterpret_cast<u32x4*>(ptile + at));
                    }
                }
            }
        };
        for (int32_t mi = 0; mi < mpad; mi += 2) {
            slot_step(slot_a, slot_b, mi);
            slot_step(slot_b, slot_a, mi + 1);
        }

        // the shared rows of the tile before: in place once the barriers below have been passed
        // (its buffer was last read two tiles ago)
        if constexpr (kSharedX || kSharedY) publish_share(upcoming, parity ^ 1);

        if constexpr (MODE == 2) {  // pass one has no token gradient to hand on: the barrier of the shared rows only
            __syncthreads();
            parity ^= 1;
            continue;
        }
        // the token gradients of the tile go down the waves; the last wave stores the sums
        float* buf = handover + parity * (J * TILE);
#pragma unroll
        for (int ww = 0; ww < NW; ++ww) {
            if (w == ww) {
#pragma unroll
                for (int j = 0; j < J; ++j) {
#pragma unroll
                    for (int q4 = 0; q4 < E / 4; ++q4) {
                        float4* cell = reinterpret_cast<float4*>(buf + ((j * (E / 4) + q4) * 64 + lane) * 4);
                        if (ww > 0) {
                            const float4 v = *cell;
                            dtok[j][4 * q4] += v.x; dtok[j][4 * q4 + 1] += v.y;
                            dtok[j][4 * q4 + 2] += v.z; dtok[j][4 * q4 + 3] += v.w;
                        }
                        if (ww < NW - 1)
                            *cell = make_float4(dtok[j][4 * q4], dtok[j][4 * q4 + 1], dtok[j][4 * q4 + 2],
                                                dtok[j][4 * q4 + 3]);
                    }
                    if (ww == NW - 1 && d0 + j < D) {
                        if (token_partial == nullptr) {
                            store_chunk<T, true>(token_grad + (b * D + d0 + j) * L, tw + lane_off, L, Elem<T>::pack(dtok[j]));
                        } else if (tw + lane_off < L) {  // (tiles are whole chunks)
                            float* __restrict__ dst =
                                token_partial + ((b_tok * D + d0 + j) * split + (b - b_tok * split)) * L + tw + lane_off;
#pragma unroll
                            for (int q4 = 0; q4 < E / 4; ++q4) {
                                const u32x4 v = {f2u(dtok[j][4 * q4]), f2u(dtok[j][4 * q4 + 1]), f2u(dtok[j][4 * q4 + 2]),
                                                 f2u(dtok[j][4 * q4 + 3])};
                                __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(dst + 4 * q4));
                            }
                        }
                    }
                }
            }
            if (ww < NW - 1) __syncthreads();
        }
        parity ^= 1;
    }

    if constexpr (MODE == 2) {
        // the segment's step pair for every row of this wave: (gate product of the slot, what left the segment)
        __builtin_amdgcn_wave_barrier();  // lane 0's writes of the carries and products precede the reads below
        for (int32_t base = 0; base < mcount * J; base += 64) {
            const int32_t idx = base + lane;
            const int32_t mi = idx / J, j = idx - mi * J;
            if (idx >= mcount * J || d0 + j >= D) continue;
            const int64_t row = (b * M + m0 + mi) * D + d0 + j;
            seg_pairs[row * nseg + seg] = make_float2(gate_products[w * Mw + mi], mycarry[idx]);
        }
        return;
    }
    if (h0_grad && k_lo == 0) {  // (a cut row: the block of its first segment)
        __builtin_amdgcn_wave_barrier();  // lane 0's carry writes precede the reads below
        for (int32_t base = 0; base < mcount * J; base += 64) {
            const int32_t idx = base + lane;
            const int32_t mi = idx / J, j = idx - mi * J;
            if (idx >= mcount * J || d0 + j >= D) continue;
            float v[E] = {mycarry[idx]};
            const u32x4 packed = Elem<T>::pack(v);
            const int64_t row = (b * M + m0 + mi) * D + d0 + j;
            if constexpr (sizeof(T) == 4) reinterpret_cast<uint32_t*>(h0_grad)[row] = packed.x;
            else reinterpret_cast<uint16_t*>(h0_grad)[row] = (uint16_t)(packed.x & 0xffffu);
        }
    }
}

// out[r, t] = sum over g of partial[r, g, t], rounded once to T: the pass that follows the kernel above
// when the caller wants d_gates itself (reference fm/scan/fm_scan.py:76, there a torch.sum over a
// (B, M, D, L) tensor). A thread takes V consecutive t (V = 4: 16-byte loads) of one r.
template <typename T, int V>
__global__ __launch_bounds__(256) void sum_groups_kernel(const float* __restrict__ partial, T* __restrict__ out,
                                                         int64_t rows, int32_t G, int64_t L) {
    const int64_t per_row = (L + V - 1) / V;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * per_row) return;
    const int64_t r = i / per_row, t = (i - r * per_row) * V;
    const float* __restrict__ p = partial + r * G * L + t;
    float acc[V];
#pragma unroll
    for (int v = 0; v < V; ++v) acc[v] = 0.0f;
#pragma unroll 8
    for (int32_t g = 0; g < G; ++g) {  // in the order of the groups: run-to-run identical
        if constexpr (V == 4) {
            const float4 x = *reinterpret_cast<const float4*>(p + (int64_t)g * L);
            acc[0] += x.x; acc[1] += x.y; acc[2] += x.z; acc[3] += x.w;
        } else {
            acc[0] += p[(int64_t)g * L];
        }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) out[r * L + t + v] = (T)acc[v];
}

}  // namespace fmscan
