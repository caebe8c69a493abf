// Device-side building blocks of the gfx950 scan kernels: 16-byte packed I/O,
// dtype <-> fp32 conversion, and the 64-lane wavefront scan of the recurrence
// operator. Everything here is written for CDNA4 wave64 directly.
#pragma once

#include <type_traits>

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fmscan {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }

// ---- loads of one address by the whole wave ---------------------------------------
// A 4-byte load whose address is the same in every lane becomes a scalar load, and scalar
// loads complete out of order on a counter they share with LDS traffic: the first wait for
// an LDS read then also waits for every scalar load in flight, however far ahead of its use
// it was issued. Where such a load is a prefetch (the one saved state before a tile, a
// tile or more ahead, a miss in every cache), that wait is a trip to HBM per tile.
// Indexing with a zero the compiler cannot see through keeps the load a vector load: those
// return in order on a counter of their own, which the kernels count.
__device__ __forceinline__ uint32_t opaque_zero() {
    uint32_t z;
    asm volatile("v_mov_b32 %0, 0" : "=v"(z));
    return z;
}
template <typename V>
__device__ __forceinline__ V load_by_wave(const V* p, uint32_t zero) {
    // (a byte offset: uniform base + 32-bit lane offset is an addressing mode of the load itself)
    return *reinterpret_cast<const V*>(reinterpret_cast<const char*>(p) + zero);
}

// All vector loads and stores issued so far have completed. For use just before a loop that
// prefetches: the compiler puts one wait at the loop's head for both ways into it, and sizes it
// for the way that needs the longer wait. From the code before the loop, where the loads the
// first pass needs are the youngest in flight, that is a wait for everything; inside the loop
// it then waits for everything too, on every pass, the prefetch and the stores of the pass
// before included. With nothing in flight on entry the count at the head is the one the loop
// itself needs. (s_waitcnt vmcnt(0); the other counters at their maxima: not waited for.)
__device__ __forceinline__ void wait_for_loads() { __builtin_amdgcn_s_waitcnt(0x0f70); }

// ---- 16 bytes <-> E fp32 values -------------------------------------------------
// One lane always moves 16 bytes per tensor per tile: 4 fp32 or 8 fp16/bf16
// consecutive sequence positions. Narrow types are widened to fp32 on load and
// rounded to nearest-even on store (the reference casts the same way,
// fm/scan/fm_scan.cuh:14-40).
template <typename T> struct Elem;

// 16 bytes at the alignment of one element: the GPU takes such an access as one instruction
typedef u32x4 u32x4_at4 __attribute__((aligned(4)));
typedef u32x4 u32x4_at2 __attribute__((aligned(2)));

template <> struct Elem<float> {
    using LooseVec = u32x4_at4;
    static constexpr int E = 4;
    static constexpr uint32_t kOnes = 0x3f800000u;  // 1.0f
    static __device__ __forceinline__ void unpack(u32x4 r, float (&f)[4]) {
        f[0] = u2f(r.x); f[1] = u2f(r.y); f[2] = u2f(r.z); f[3] = u2f(r.w);
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[4]) {
        u32x4 r; r.x = f2u(f[0]); r.y = f2u(f[1]); r.z = f2u(f[2]); r.w = f2u(f[3]);
        return r;
    }
    static __device__ __forceinline__ float widen(float v) { return v; }
};

template <> struct Elem<__bf16> {
    using LooseVec = u32x4_at2;
    static constexpr int E = 8;
    static constexpr uint32_t kOnes = 0x3f803f80u;  // two bf16 1.0
    static __device__ __forceinline__ void unpack(u32x4 r, float (&f)[8]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = u2f(r[j] << 16);
            f[2 * j + 1] = u2f(r[j] & 0xffff0000u);
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[8]) {
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f32x2 v = {f[2 * j], f[2 * j + 1]};
            bf16x2 b = __builtin_convertvector(v, bf16x2);  // v_cvt_pk_bf16_f32, RNE
            r[j] = __builtin_bit_cast(uint32_t, b);
        }
        return r;
    }
    static __device__ __forceinline__ float widen(__bf16 v) { return (float)v; }
};

template <> struct Elem<_Float16> {
    using LooseVec = u32x4_at2;
    static constexpr int E = 8;
    static constexpr uint32_t kOnes = 0x3c003c00u;  // two fp16 1.0
    static __device__ __forceinline__ void unpack(u32x4 r, float (&f)[8]) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint32_t word = r[j];  // a copy: bit_cast straight from the vector element reads element 0
            f16x2 h = __builtin_bit_cast(f16x2, word);
            f[2 * j] = (float)h.x;
            f[2 * j + 1] = (float)h.y;
        }
    }
    static __device__ __forceinline__ u32x4 pack(const float (&f)[8]) {
        u32x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f32x2 v = {f[2 * j], f[2 * j + 1]};
            f16x2 h = __builtin_convertvector(v, f16x2);  // RNE
            r[j] = __builtin_bit_cast(uint32_t, h);
        }
        return r;
    }
    static __device__ __forceinline__ float widen(_Float16 v) { return (float)v; }
};

// Chunk = the E consecutive elements one lane owns in a tile, starting at
// sequence position t0 of a row. VEC: the row base and L*sizeof(T) are 16-byte
// multiples, so a chunk is either wholly inside [0, L) or wholly outside and
// moves as one 16-byte access. !VEC: a chunk wholly inside moves as one access at the
// alignment of an element, the ragged one at the end of a row as element accesses with a
// bound check each; `fill` is the 32-bit pattern for positions at or beyond L. ONCE marks data that
// no other row reads again: it is loaded with the non-temporal hint so that it does
// not displace anything from the caches on its way through (measured: worth about a
// tenth of the bandwidth on 1 GiB tensors). Stores always carry the hint.
// ALIGNED = false: p is aligned as an element is, not to 16 bytes (still one access).
template <typename T, bool ALIGNED> struct Vec16 { using type = u32x4; };
template <typename T> struct Vec16<T, false> { using type = typename Elem<T>::LooseVec; };

template <typename T, bool ONCE, bool ALIGNED = true>
__device__ __forceinline__ u32x4 load16(const T* __restrict__ p) {
    using V = typename Vec16<T, ALIGNED>::type;
    if constexpr (ONCE) return __builtin_nontemporal_load(reinterpret_cast<const V*>(p));
    else return *reinterpret_cast<const V*>(p);
}

// The VEC form never branches around its load: a chunk outside [0, L) reads the last
// chunk of the row instead and is replaced by `fill` afterwards. A load that is only
// sometimes issued makes the compiler wait for every outstanding load before each use
// (it can no longer count how many newer ones are in flight).
template <typename T, bool VEC, bool ONCE>
__device__ __forceinline__ u32x4 load_chunk(const T* __restrict__ row, int64_t t0, int64_t L,
                                            uint32_t fill) {
    constexpr int E = Elem<T>::E;
    u32x4 r = {fill, fill, fill, fill};
    if constexpr (VEC) {
        const bool inside = t0 < L;
        const u32x4 v = load16<T, ONCE>(row + (inside ? t0 : L - E));
        r = inside ? v : r;
    } else {
        if (t0 + E <= L) {  // a whole chunk: one access at the alignment of an element
            r = load16<T, ONCE, false>(row + t0);
        } else if (t0 < L) {  // the ragged end of a row
            if constexpr (sizeof(T) == 4) {
                const uint32_t* p = reinterpret_cast<const uint32_t*>(row);
#pragma unroll
                for (int i = 0; i < E; ++i)
                    if (t0 + i < L) r[i] = p[t0 + i];
            } else {
                const uint16_t* p = reinterpret_cast<const uint16_t*>(row);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    uint32_t lo = fill & 0xffffu, hi = fill >> 16;
                    if (t0 + 2 * j < L) lo = p[t0 + 2 * j];
                    if (t0 + 2 * j + 1 < L) hi = p[t0 + 2 * j + 1];
                    r[j] = lo | (hi << 16);
                }
            }
        }
    }
    return r;
}

template <typename T, bool ALIGNED = true>
__device__ __forceinline__ void store16(T* __restrict__ p, u32x4 r) {
    using V = typename Vec16<T, ALIGNED>::type;
    __builtin_nontemporal_store(r, reinterpret_cast<V*>(p));
}

template <typename T, bool VEC>
__device__ __forceinline__ void store_chunk(T* __restrict__ row, int64_t t0, int64_t L, u32x4 r) {
    constexpr int E = Elem<T>::E;
    if (t0 >= L) return;
    if constexpr (VEC) {
        __builtin_nontemporal_store(r, reinterpret_cast<u32x4*>(row + t0));
    } else {
        if (t0 + E <= L) {
            store16<T, false>(row + t0, r);
        } else if constexpr (sizeof(T) == 4) {
            uint32_t* p = reinterpret_cast<uint32_t*>(row);
#pragma unroll
            for (int i = 0; i < E; ++i)
                if (t0 + i < L) p[t0 + i] = r[i];
        } else {
            uint16_t* p = reinterpret_cast<uint16_t*>(row);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (t0 + 2 * j < L) p[t0 + 2 * j] = (uint16_t)(r[j] & 0xffffu);
                if (t0 + 2 * j + 1 < L) p[t0 + 2 * j + 1] = (uint16_t)(r[j] >> 16);
            }
        }
    }
}

// ---- wavefront scan ---------------------------------------------------------------
// DPP lane permutes (data-parallel primitives: the permute happens in the VALU
// operand path, no LDS traffic). A lane whose source lane does not exist, or
// that the row mask switches off, receives `old`.
constexpr int kWaveShl1 = 0x130;  // lane i <- lane i+1
constexpr int kWaveShr1 = 0x138;  // lane i <- lane i-1

template <int CTRL, int ROW_MASK = 0xf>
__device__ __forceinline__ float dpp(float old, float v) {
    return u2f((uint32_t)__builtin_amdgcn_update_dpp((int)f2u(old), (int)f2u(v), CTRL, ROW_MASK,
                                                      0xf, false));
}

// The recurrence step "h -> a*h + b" composes as (a1,b1) then (a2,b2) =
// (a1*a2, b1*a2 + b2) (the combine at reference fm/scan/fm_scan.cuh:139-140).
// On entry lane l holds the pair of its own chunk; on exit it holds the
// composition of chunks 0..l: four shifted steps inside each 16-lane row, then
// the row totals are broadcast into rows 1,3 and finally into rows 2,3.
// One wave scan = six steps; each is two VALU instructions that take their first source
// through DPP: b += b[src] * a, then a *= a[src]. A lane whose source lane does not
// exist or whose row is masked off is left untouched, which is exactly "combine only if
// there is something to the left" (the `laneId >= delta` test at reference
// fm/scan/fm_scan.cuh:138). Written as one asm block because the compiler keeps the
// permute as a separate move with an explicit identity (three times the instructions).
// s_nop: a VGPR written by a VALU instruction may be read through DPP two wait states
// later at the earliest; inside the block the instruction in between provides one.
__device__ __forceinline__ void wave_scan_inclusive(float& a, float& b) {
    asm volatile(
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(a), "+v"(b));
}

// The same scan in the other lane direction, for step pairs whose time order runs from lane
// 63 down to lane 0 (the backward kernels lay a tile out that way and still need states that
// run forward in time). DPP has no row broadcast towards lower lanes, so this comes in two
// parts. First every row of 16 lanes scans itself: on exit lane l holds the composition of
// the chunks of lanes (l | 15) down to l.
__device__ __forceinline__ void row_scan_inclusive_down(float& a, float& b) {
    asm volatile(
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shl:1 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shl:2 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shl:4 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 0\n\t"
        "v_fmac_f32_dpp %1, %1, %0 row_shl:8 row_mask:0xf bank_mask:0xf\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(a), "+v"(b));
}

constexpr int kRowShl1 = 0x101;  // lane i <- lane i+1 inside its row of 16

__device__ __forceinline__ float lane_value(float v, int lane) {
    return u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(v), lane));
}

// Second part: the state that enters every lane's chunk when `entry` (the same in all lanes)
// enters lane 63's. (a, b) are the row-scanned pairs of row_scan_inclusive_down. The totals of
// rows 3, 2, 1 sit in lanes 48, 32, 16; three chained steps on wave-uniform values carry the
// state from row to row, and inside a row a lane applies the pairs of the lanes above it.
__device__ __forceinline__ float state_entering_lane_down(float a, float b, float entry, int lane) {
    const float e3 = entry;
    const float e2 = __builtin_fmaf(lane_value(a, 48), e3, lane_value(b, 48));
    const float e1 = __builtin_fmaf(lane_value(a, 32), e2, lane_value(b, 32));
    const float e0 = __builtin_fmaf(lane_value(a, 16), e1, lane_value(b, 16));
    const int row = lane >> 4;
    const float e = row == 3 ? e3 : (row == 2 ? e2 : (row == 1 ? e1 : e0));
    const float xa = dpp<kRowShl1>(1.0f, a);  // the lanes above, inside the row
    const float xb = dpp<kRowShl1>(0.0f, b);
    return __builtin_fmaf(xa, e, xb);
}

__device__ __forceinline__ float lane63(float v) {
    return u2f((uint32_t)__builtin_amdgcn_readlane((int)f2u(v), 63));
}

// ---- wave scan with the gates' part done once ------------------------------------------
// Rows that share their gates (the rows of one memory slot m) share the `a` halves of
// all their step pairs and everything the wave scan does to them. scan_gates runs that half
// once per slot and keeps what each of the six levels needs (the value of `a` before the
// level); scan_values then scans the `b` half of a row with one instruction per level.
struct GateLevels {
    float before[6];  // a in this lane before level 1..6
    float ea;         // product of the gates of all chunks before this lane's (1 in lane 0)
    float ta;         // product over the whole tile
};

__device__ __forceinline__ GateLevels scan_gates(float a) {
    GateLevels g;
    asm volatile(
        "s_nop 1\n\t"
        "v_mov_b32 %1, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %2, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %3, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %4, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %5, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %6, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(a), "=&v"(g.before[0]), "=&v"(g.before[1]), "=&v"(g.before[2]), "=&v"(g.before[3]),
          "=&v"(g.before[4]), "=&v"(g.before[5]));
    g.ea = dpp<kWaveShr1>(1.0f, a);
    g.ta = lane63(a);
    return g;
}

__device__ __forceinline__ void scan_values(float& b, const GateLevels& g) {
    asm volatile(
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %1 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %2 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %3 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %4 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %5 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %6 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(b)
        : "v"(g.before[0]), "v"(g.before[1]), "v"(g.before[2]), "v"(g.before[3]), "v"(g.before[4]),
          "v"(g.before[5]));
}

// E consecutive floats at p (16-byte aligned)
template <int E>
struct FloatChunk {
    float4 v[E / 4];
};
template <int E>
__device__ __forceinline__ FloatChunk<E> load_float_chunk(const float* __restrict__ p) {
    FloatChunk<E> c;
#pragma unroll
    for (int i = 0; i < E / 4; ++i) c.v[i] = reinterpret_cast<const float4*>(p)[i];
    return c;
}
template <int E>
__device__ __forceinline__ void spread(const FloatChunk<E>& c, float (&f)[E]) {
#pragma unroll
    for (int i = 0; i < E / 4; ++i) {
        f[4 * i] = c.v[i].x; f[4 * i + 1] = c.v[i].y; f[4 * i + 2] = c.v[i].z; f[4 * i + 3] = c.v[i].w;
    }
}

// The same split for the scan that runs down the lanes (row_scan_inclusive_down,
// state_entering_lane_down): the gate half once for all rows that share their gates.
struct GateLevelsDown {
    float before[4];        // a in this lane before the four levels inside a row of 16 lanes
    float xa;               // product of the gates of the lanes above, inside the row (1 in its lane 15)
    float a48, a32, a16;    // products over the whole rows 3, 2, 1
};

__device__ __forceinline__ GateLevelsDown scan_gates_down(float a) {
    GateLevelsDown g;
    asm volatile(
        "s_nop 1\n\t"
        "v_mov_b32 %1, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %2, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %3, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_mov_b32 %4, %0\n\t"
        "v_mul_f32_dpp %0, %0, %0 row_shl:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(a), "=&v"(g.before[0]), "=&v"(g.before[1]), "=&v"(g.before[2]), "=&v"(g.before[3]));
    g.xa = dpp<kRowShl1>(1.0f, a);
    g.a48 = lane_value(a, 48);
    g.a32 = lane_value(a, 32);
    g.a16 = lane_value(a, 16);
    return g;
}

// b half of a row's step pairs -> the state that enters every lane's chunk when `entry` (the
// same in all lanes) enters lane 63's
__device__ __forceinline__ float state_entering_lane_down(float b, const GateLevelsDown& g, float entry, int lane) {
    asm volatile(
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %1 row_shl:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %2 row_shl:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %3 row_shl:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_fmac_f32_dpp %0, %0, %4 row_shl:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(b)
        : "v"(g.before[0]), "v"(g.before[1]), "v"(g.before[2]), "v"(g.before[3]));
    const float e3 = entry;
    const float e2 = __builtin_fmaf(g.a48, e3, lane_value(b, 48));
    const float e1 = __builtin_fmaf(g.a32, e2, lane_value(b, 32));
    const float e0 = __builtin_fmaf(g.a16, e1, lane_value(b, 16));
    const int row = lane >> 4;
    const float e = row == 3 ? e3 : (row == 2 ? e2 : (row == 1 ? e1 : e0));
    return __builtin_fmaf(g.xa, e, dpp<kRowShl1>(0.0f, b));
}

}  // namespace fmscan
