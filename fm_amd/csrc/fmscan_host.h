// Host-side pieces shared by the translation units of libfmscan_hip.so: error text,
// argument checks, the choice of kernel variant, and the tags that turn run-time choices
// into template arguments. Declarations and the contract of every entry point:
// include/fmscan.h.
#pragma once

#include "../../include/fmscan.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <initializer_list>

namespace fmscan {
namespace host {

// Text of the last rejected call on this thread (fmscan_last_error); defined in fmscan_core.hip.
extern thread_local char g_err[512];

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

struct Range {
    const char* name;
    const void* p;
    int64_t bytes;
};
inline bool overlap(const Range& a, const Range& b) {
    if (!a.p || !b.p) return false;
    const uintptr_t a0 = (uintptr_t)a.p, b0 = (uintptr_t)b.p;
    return a0 < b0 + (uintptr_t)b.bytes && b0 < a0 + (uintptr_t)a.bytes;
}

struct Problem {
    int64_t B, M, D, L, rows;
    int esize;
    unsigned waves;          // requested waves per row, 0 = auto
    unsigned blocks_per_cu;  // requested cap on resident blocks per CU, 0 = auto
    unsigned depth;          // requested prefetch depth in tiles, 0 = auto
    unsigned segments;       // requested segments per row, 0 = auto
    bool plain;
};

constexpr unsigned kKnownFlags = FMSCAN_FLAG_PLAIN | FMSCAN_FLAG_WAVES_MASK | FMSCAN_FLAG_BLOCKS_MASK |
                                 FMSCAN_FLAG_DEPTH_MASK | FMSCAN_FLAG_SEGMENTS_MASK;

inline int parse(int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags, Problem* pb) {
    if (B < 1 || M < 1 || D < 1 || L < 1)
        return fail(FMSCAN_E_SHAPE, "fmscan: B, M, D, L must be >= 1 (got %lld, %lld, %lld, %lld)",
                    (long long)B, (long long)M, (long long)D, (long long)L);
    if (M > INT32_MAX || D > INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "fmscan: M and D must fit 32 bits");
    if (dtype != FMSCAN_DTYPE_F32 && dtype != FMSCAN_DTYPE_F16 && dtype != FMSCAN_DTYPE_BF16)
        return fail(FMSCAN_E_DTYPE, "fmscan: dtype %d is not float32 (0), float16 (1) or bfloat16 (2)",
                    dtype);
    if (flags & ~kKnownFlags)
        return fail(FMSCAN_E_FLAGS, "fmscan: unknown flag bits 0x%x", flags & ~kKnownFlags);
    const unsigned waves = (flags & FMSCAN_FLAG_WAVES_MASK) >> FMSCAN_FLAG_WAVES_SHIFT;
    if (waves != 0 && waves != 1 && waves != 2 && waves != 4 && waves != 8)
        return fail(FMSCAN_E_FLAGS, "fmscan: waves per row must be 0 (auto), 1, 2, 4 or 8 (got %u)",
                    waves);
    const unsigned depth = (flags & FMSCAN_FLAG_DEPTH_MASK) >> FMSCAN_FLAG_DEPTH_SHIFT;
    if (depth != 0 && depth != 2 && depth != 4)
        return fail(FMSCAN_E_FLAGS, "fmscan: prefetch depth must be 0 (auto), 2 or 4 (got %u)", depth);
    // rows*L elements must be addressable and the grid must fit 31 bits
    const __int128 rows = (__int128)B * M * D;
    if (rows > (__int128)INT32_MAX || rows * L > ((__int128)1 << 46))
        return fail(FMSCAN_E_SHAPE, "fmscan: B*M*D = rows must be < 2^31 and rows*L <= 2^46");
    pb->B = B; pb->M = M; pb->D = D; pb->L = L;
    pb->rows = (int64_t)rows;
    pb->esize = dtype == FMSCAN_DTYPE_F32 ? 4 : 2;
    pb->waves = waves;
    pb->blocks_per_cu = (flags & FMSCAN_FLAG_BLOCKS_MASK) >> FMSCAN_FLAG_BLOCKS_SHIFT;
    pb->depth = depth;
    pb->segments = (flags & FMSCAN_FLAG_SEGMENTS_MASK) >> FMSCAN_FLAG_SEGMENTS_SHIFT;
    pb->plain = (flags & FMSCAN_FLAG_PLAIN) != 0;
    return 0;
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

inline int launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "fmscan: %s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// A kernel may ask for more dynamic LDS than the default limit only after the limit has been
// raised for it. The limit is an upper bound, so it is raised once per (kernel, device) to
// (nearly) all the LDS a compute unit has and never lowered: whatever a launch then asks for is within
// it, and calls from several threads cannot undercut each other. `armed` belongs to one
// kernel instantiation: bit d is set once the limit has been raised on device d (devices
// beyond 63 raise it on every call). Returns 0 or a positive hipError_t with the text set.
constexpr unsigned kLdsPerCU = 160u * 1024u;
constexpr unsigned kMaxDynamicLds = kLdsPerCU - 2048u;  // 2 KiB stay free for the kernels' static LDS
inline int raise_lds_limit(const void* kern, std::atomic<uint64_t>& armed, const char* who) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail((int)e, "%s: hipGetDevice failed: %s", who, hipGetErrorString(e));
    const uint64_t bit = dev < 64 ? (1ull << dev) : 0ull;
    if (bit && (armed.load(std::memory_order_acquire) & bit)) return 0;
    e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMaxDynamicLds);
    if (e != hipSuccess) {
        (void)hipGetLastError();
        return fail((int)e, "%s: cannot raise the kernel's dynamic LDS limit to %u bytes: %s", who, kMaxDynamicLds,
                    hipGetErrorString(e));
    }
    if (bit) armed.fetch_or(bit, std::memory_order_release);
    return 0;
}

// Each block of the streaming kernels asks for a share of the 160 KiB of LDS of a compute
// unit that it never touches: at most `blocks_per_cu` blocks then fit a unit at a time,
// which bounds the number of rows that stream concurrently.
inline unsigned lds_share(unsigned blocks_per_cu) {
    return (kMaxDynamicLds / blocks_per_cu) & ~1023u;
}

// Waves per row, resident blocks per compute unit, prefetch depth and segments per row
// when the caller leaves the choice to the library. The table comes from sweeps on an
// MI355X over rows x row length x element type, forward and backward apart, every
// combination of waves (1, 2, 4, 8), cap (1, 2, 4, 8) and depth (2, 4) a caller can ask for
// (`python bench.py --grid` prints the choice against the best of them). What decides is
// the length of a row in bytes and, for rows of 32 to 64 KiB, how many rows there are:
//   up to 4 KiB     a wave per row, four rows per block, 4 to 8 blocks per compute unit;
//   8 to 16 KiB     2 to 4 waves per row;
//   32 to 64 KiB    with 32768 rows or more a wave per row and few rows open at a time (one or two
//                   blocks per compute unit), with fewer rows 8 waves side by side;
//   128 KiB up      8 waves per row, one block per compute unit, four tiles in flight (16 waves
//                   in backward, which only the library chooses: 0.501 -> 0.478 ms at 4096 rows of
//                   65536; forward gains nothing from them).
// One to two waves per SIMD is where HBM efficiency peaks; more resident rows lower it. With so few
// rows that even eight waves per row leave compute units idle (fewer than 32 rows), and a
// workspace to hold the segment pairs, rows are cut into segments (two passes).
struct Tuning {
    unsigned waves, blocks_per_cu, depth;
    int32_t nseg;       // segments per row (1 = the row is scanned in one piece)
    int64_t seg_tiles;  // tiles per segment
};
constexpr int64_t kSplitBelowRows = 32;     // rows below which cutting rows pays (measured)
constexpr int64_t kSplitTargetSlots = 2048;  // segments in flight the cut aims for
constexpr int64_t kSplitMinTiles = 4;       // a segment is at least this many tiles
constexpr int64_t kMaxSegments = 255;

inline void plan_segments(const Problem& pb, Tuning& t, bool may_split) {
    const int64_t tile1 = (16 / pb.esize) * 64;
    const int64_t tiles1 = (pb.L + tile1 - 1) / tile1;
    t.nseg = 1;
    t.seg_tiles = tiles1;
    if (!may_split) return;
    int64_t want = pb.segments;
    if (!want) {
        if (pb.rows >= kSplitBelowRows || pb.waves) return;
        want = (kSplitTargetSlots + pb.rows - 1) / pb.rows;
        const int64_t most = tiles1 / kSplitMinTiles;
        if (want > most) want = most;
    }
    if (want > tiles1) want = tiles1;
    if (want > kMaxSegments) want = kMaxSegments;
    if (want < 2) return;
    const int64_t seg_tiles = (tiles1 + want - 1) / want;
    const int64_t nseg = (tiles1 + seg_tiles - 1) / seg_tiles;
    if (nseg < 2) return;
    // a cut row is scanned by single waves: enough slots exist without sharing a row
    t.waves = 1;
    t.seg_tiles = seg_tiles;
    t.nseg = (int32_t)nseg;
}

inline Tuning choose(const Problem& pb, bool backward, bool may_split) {
    Tuning t;
    const int64_t tile1 = (16 / pb.esize) * 64;          // elements one wave covers per tile
    const int64_t tiles1 = (pb.L + tile1 - 1) / tile1;   // tiles per row for one wave = KiB per row
    // Gates shared by D rows and tokens shared by M rows come from the caches: the kernel
    // then mostly writes (forward) and the limit on concurrent rows no longer applies.
    // Measured on (B, M, D, L) = (32,32,128,2048), (1,32,2048,8192), (2,32,512,16384), (4,32,1024,4096).
    const bool shared_inputs = pb.M > 1 || pb.D > 1;
    const bool many_rows = pb.rows >= 32768;
    unsigned w, bpc, depth;
    if (shared_inputs) {
        const bool long_rows = tiles1 >= 64, few_rows = pb.rows < 16384 && tiles1 >= 8;
        if (pb.rows >= 16384) w = 1;
        else if (long_rows) w = backward ? 16 : 8;
        else if (few_rows) w = 4;
        else w = 1;
        // rows taken out of memory order (tokens of a batch element beyond an L2, see slot_of_block):
        // fewer of them open at a time
        const bool regrouped = pb.M > 1 && pb.D * pb.L * pb.esize > (4 << 20);
        bpc = regrouped ? 4 : 8;
        depth = 2;
    } else if (!backward) {
        if (tiles1 <= 2) { w = 1; bpc = 8; depth = 2; }
        else if (tiles1 <= 4) { w = 1; bpc = 4; depth = 2; }
        else if (tiles1 <= 8) { w = 2; bpc = 8; depth = 2; }
        else if (tiles1 <= 16) { w = 4; bpc = 4; depth = 2; }
        else if (tiles1 <= 32) { w = many_rows ? 1 : 8; bpc = 2; depth = 2; }
        else if (tiles1 <= 64) { w = many_rows ? 1 : 8; bpc = 1; depth = many_rows ? 4 : 2; }
        else { w = 8; bpc = 1; depth = 4; }
    } else {
        if (tiles1 <= 4) { w = 1; bpc = 4; depth = 2; }
        else if (tiles1 <= 8) { w = 4; bpc = 8; depth = 2; }
        else if (tiles1 <= 16) { w = 4; bpc = 4; depth = 2; }
        else if (tiles1 <= 32) { w = pb.rows >= 16384 ? 1 : 8; bpc = pb.rows >= 16384 ? 2 : 4; depth = 2; }
        else if (tiles1 <= 64) { w = many_rows ? 2 : 8; bpc = many_rows ? 2 : 1; depth = 2; }
        else { w = 16; bpc = 1; depth = 2; }  // 16 waves leave 128 registers each: no deeper prefetch
    }
    if (pb.waves) {
        w = pb.waves;
    } else {
        while (w > 1 && tiles1 < (int64_t)w) w /= 2;                                        // row shorter than a tile
        while (w < 8 && w != 16 && pb.rows * w < 1024 && tiles1 >= 2 * (int64_t)w) w *= 2;  // very few rows
    }
    t.waves = w;
    plan_segments(pb, t, may_split);
    w = t.waves;
    if (t.nseg > 1) {  // a cut row is scanned by single waves, as short rows are
        bpc = (t.seg_tiles >= 8) ? 2 : 4;
        depth = 2;
    }
    t.blocks_per_cu = pb.blocks_per_cu ? pb.blocks_per_cu : bpc;
    t.depth = pb.depth ? pb.depth : depth;
    if (w == 16) t.depth = 2;  // deeper does not fit the registers of a 16-wave block
    return t;
}

inline size_t pairs_bytes(const Problem& pb, const Tuning& t) {
    return t.nseg > 1 ? (size_t)pb.rows * (size_t)t.nseg * sizeof(float2) : 0;
}

// Settles the plan for one call: rows are cut only when the workspace can hold the pairs.
// Returns 0, FMSCAN_E_WORKSPACE when the caller asked for a cut that does not fit, or
// FMSCAN_E_SHAPE when rows * segments does not fit a grid.
inline int settle(const Problem& pb, bool backward, const void* workspace, size_t workspace_bytes, const char* who,
                  Tuning* t) {
    *t = choose(pb, backward, workspace != nullptr);
    if (t->nseg > 1 && (pairs_bytes(pb, *t) > workspace_bytes || ((uintptr_t)workspace & 7u))) {
        if (pb.segments > 1)
            return fail(FMSCAN_E_WORKSPACE, "%s: %u segments per row need an 8-byte aligned workspace of "
                        "%zu bytes (got %zu)", who, pb.segments, pairs_bytes(pb, *t), workspace_bytes);
        *t = choose(pb, backward, false);
    } else if (pb.segments > 1 && !workspace) {
        return fail(FMSCAN_E_WORKSPACE, "%s: %u segments per row need a workspace", who, pb.segments);
    }
    // one block per slot at most (one per four slots with a wave per row): the grid is 31 bits
    if ((__int128)pb.rows * t->nseg > (__int128)INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: rows * segments = %lld * %d must be < 2^31", who, (long long)pb.rows,
                    (int)t->nseg);
    return 0;
}

// Short rows (at most 64 chunks of 16 bytes, 1 KiB) go to the kernels that put several
// rows into a wave (fmscan_packed.h), unless the caller asks for a kernel variant by flag: measured on
// 2^27 elements of bfloat16 with M = D = 1, fraction of 8 TB/s forward (3 streams) / backward (6 streams),
// one row per wave -> packed: L = 32: 0.07 / 0.06 -> 0.82 / 0.75; 64: 0.13 / 0.11 -> 0.77 / 0.72;
// 128: 0.24 / 0.22 -> 0.78 / 0.73; 256: 0.43 / 0.41 -> 0.81 / 0.76; 512: 0.73 / 0.70 -> 0.82 / 0.77.
inline bool packs_rows(const Problem& pb, bool vec, bool backward) {
    (void)vec;  // rows that are not whole aligned vectors are packed too
    if (pb.L * pb.esize > 1024 || pb.waves || pb.blocks_per_cu || pb.depth || pb.segments > 1) return false;
    // The packed backward kernel reads the saved states, which the general one makes again from the gates
    // and tokens: with 4-byte elements and rows of more than 32 chunks the general kernel is as fast or
    // faster (ms, float32: (128,32,128,256) 0.349 against 0.380, (524288,1,1,256) 0.516 against 0.541).
    if (backward && pb.esize == 4 && pb.L * pb.esize > 512) return false;
    return true;
}
// log2 of the lanes a row takes: the power of two at or above its number of 16-byte chunks
inline int32_t packed_lanes_log2(const Problem& pb) {
    const int64_t chunks = (pb.L * pb.esize + 15) / 16;
    int32_t k = 0;
    while ((1 << k) < chunks) ++k;
    return k;
}
// blocks of four waves that cover all rows, 64 >> lanes_log2 rows per wave
inline unsigned packed_blocks(const Problem& pb, int32_t lanes_log2) {
    const int64_t per_wave = 64 >> lanes_log2;
    const int64_t waves = (pb.rows + per_wave - 1) / per_wave;
    return (unsigned)((waves + 3) / 4);
}

// The kernels of the layer and of the backward scan with the sums inside that put several rows into a wave
// (fmscan_packed.h) give a wave a slot, or a batch element and a tile of rows, for the whole of its loop:
// they are taken from this many waves on. Measured on the backward kernel with the sums inside (bf16, us, the
// general routes against the packed kernel): (B,M,D,L) = (64,32,128,64), 1024 waves, 98 against 52;
// (128,32,128,64) 187 / 62; (256,16,64,32), 1024 waves, 105 / 31; (128,16,64,32), 512 waves, 56 / 32;
// (32,32,128,64), 512 waves, 53 / 49; (16,32,128,128), 512 waves, 44 / 49; with 256 waves 43-47 either way.
#ifndef FMSCAN_PACKED_MIN_WAVES
#define FMSCAN_PACKED_MIN_WAVES 512
#endif
constexpr int64_t kPackedMinWaves = FMSCAN_PACKED_MIN_WAVES;
// The read-out's kernels and the dot have less to do per wave and general forms that hold up longer: four
// times as many (us, general / packed, bf16: read-out (B,M,D,L) = (32,32,128,64), 512 waves, 15 / 18,
// (128,32,128,64), 2048 waves, 30 / 22, (64,32,128,128), 2048 waves, 18 / 22, (128,32,128,128) 34 / 25;
// dot (16,32,128,64), 512 waves, 8 / 11, (32,32,128,64) 14 / 12, (64,32,128,128), 2048 waves, 27 / 22;
// scan + norm (16,32,128,64), 512 waves, 16 / 9, (16,32,128,128) 15 / 15, (8,32,128,128), 256 waves, 8 / 15).
constexpr int64_t kPackedMinWavesReadout = 4 * kPackedMinWaves;

// Expands run-time choices into template arguments: F is a generic lambda called with tags.
template <typename T> struct TypeTag { using type = T; };
template <int V> struct IntTag { static constexpr int value = V; };
template <bool V> struct BoolTag { static constexpr bool value = V; };

template <typename F>
void with_dtype(int dtype, F&& f) {
    if (dtype == FMSCAN_DTYPE_F32) f(TypeTag<float>{});
    else if (dtype == FMSCAN_DTYPE_F16) f(TypeTag<_Float16>{});
    else f(TypeTag<__bf16>{});
}

template <typename F>
void with_bool(bool v, F&& f) {
    if (v) f(BoolTag<true>{});
    else f(BoolTag<false>{});
}

// dtype, waves per row (with the rows per block that go with it), prefetch depth, plain,
// vector access, fold -> f(tt, wt, rt, dt, pt, vt, ft). Only what choose() and the flags can ask
// for is instantiated: depths 2 and 4, and 16 waves per row for the backward kernel alone
// (WITH16), the only one choose() gives them to.
template <bool WITH16, typename F>
void dispatch(int dtype, const Tuning& t, bool plain, bool vec, bool fold, F&& f) {
    with_dtype(dtype, [&](auto tt) {
        auto with_waves = [&](auto wt, auto rt) {
            auto with_depth = [&](auto dt, auto vt, auto ft) {
                if (plain) f(tt, wt, rt, dt, BoolTag<true>{}, vt, ft);
                else f(tt, wt, rt, dt, BoolTag<false>{}, vt, ft);
            };
            if (!vec) {  // rows off the 16-byte grid: the slower path gets one variant
                with_depth(IntTag<2>{}, BoolTag<false>{}, BoolTag<false>{});
                return;
            }
            auto with_fold = [&](auto dt) {
                if (fold) with_depth(dt, BoolTag<true>{}, BoolTag<true>{});
                else with_depth(dt, BoolTag<true>{}, BoolTag<false>{});
            };
            if (t.depth == 2) with_fold(IntTag<2>{});
            else with_fold(IntTag<4>{});
        };
        switch (t.waves) {
            case 1: with_waves(IntTag<1>{}, IntTag<4>{}); break;  // 4 independent rows per block
            case 2: with_waves(IntTag<2>{}, IntTag<1>{}); break;
            case 4: with_waves(IntTag<4>{}, IntTag<1>{}); break;
            case 16:
                if constexpr (WITH16) {
                    with_waves(IntTag<16>{}, IntTag<1>{});
                    break;
                }
                [[fallthrough]];
            default: with_waves(IntTag<8>{}, IntTag<1>{}); break;
        }
    });
}

}  // namespace host
}  // namespace fmscan
