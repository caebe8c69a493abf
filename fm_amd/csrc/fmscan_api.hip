// Host side of libfmscan_hip.so: argument checks, choice of kernel variant,
// launch. Declarations and the contract of every entry point: include/fmscan.h.
#include "../../include/fmscan.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "fmscan_kernels.h"
#include "fmscan_readout.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
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
bool overlap(const Range& a, const Range& b) {
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

int parse(int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags, Problem* pb) {
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
    if (depth != 0 && (depth < 2 || depth > 4))
        return fail(FMSCAN_E_FLAGS, "fmscan: prefetch depth must be 0 (auto), 2, 3 or 4 (got %u)", depth);
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

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

int launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "fmscan: %s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// One block per R slots (a slot is a row, or a segment of a row). Each block also asks
// for a share of the 160 KiB of LDS of a compute unit that it never touches: at most
// `blocks_per_cu` blocks then fit a unit at a time, which bounds the number of rows
// that stream concurrently.
struct Grid {
    unsigned blocks, lds;
};
// `last_set` belongs to one kernel instantiation: (device, bytes) of its last attribute call,
// so that the attribute is only set again when the cap or the device changes.
Grid throttled_grid(const void* kern, std::atomic<uint64_t>& last_set, int64_t slots, int R,
                    unsigned blocks_per_cu) {
    Grid g;
    g.blocks = (unsigned)((slots + R - 1) / R);
    g.lds = ((160u * 1024u - 2048u) / blocks_per_cu) & ~1023u;
    int dev = 0;
    (void)hipGetDevice(&dev);
    const uint64_t key = ((uint64_t)dev << 32) | g.lds;
    if (last_set.load(std::memory_order_relaxed) != key) {
        if (hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)g.lds) != hipSuccess) {
            (void)hipGetLastError();
            g.lds = 0;
        } else {
            last_set.store(key, std::memory_order_relaxed);
        }
    }
    return g;
}

// Waves per row, resident blocks per compute unit, prefetch depth and segments per row
// when the caller leaves the choice to the library. The table comes from sweeps on an
// MI355X over the benchmark shapes (rows x L): 131072 x 2048, 32768 x 16384, 4096 x 65536
// in 16-bit types and 8192 x 4096 in float32, forward and backward separately. What it
// encodes: one or two waves per row stream best when there are many rows of moderate
// length; long rows want eight waves side by side so that fewer rows are open at a
// time; with few rows a block per row keeps every compute unit busy. One to two waves
// per SIMD is where HBM efficiency peaks; more resident rows lower it. With so few rows
// that even eight waves per row leave compute units idle (fewer than 32 rows), and a
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

void plan_segments(const Problem& pb, Tuning& t, bool may_split) {
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

Tuning choose(const Problem& pb, bool backward, bool may_split) {
    Tuning t;
    const int64_t tile1 = (16 / pb.esize) * 64;          // elements one wave covers per tile
    const int64_t tiles1 = (pb.L + tile1 - 1) / tile1;   // tiles per row for one wave
    // Gates shared by D rows and tokens shared by M rows come from the caches: the kernel
    // then mostly writes (forward) and the limit on concurrent rows no longer applies.
    // Measured on (B, M, D, L) = (32,32,128,2048), (1,32,2048,8192), (2,32,512,16384).
    const bool shared_inputs = pb.M > 1 || pb.D > 1;
    const bool long_rows = tiles1 >= 64, few_rows = pb.rows < 16384 && tiles1 >= 8;
    unsigned w = pb.waves;
    if (!w) {
        if (shared_inputs && pb.rows >= 16384) w = 1;
        else if (long_rows) w = 8;
        else if (few_rows) w = 4;
        else if (tiles1 >= 16) w = backward ? 1 : 2;
        else if (tiles1 >= 8) w = backward ? 2 : 1;
        else w = 1;
        while (w > 1 && tiles1 < (int64_t)w) w /= 2;                               // row shorter than a tile
        while (w < 8 && pb.rows * w < 1024 && tiles1 >= 2 * (int64_t)w) w *= 2;     // very few rows
    }
    t.waves = w;
    plan_segments(pb, t, may_split);
    w = t.waves;
    const int64_t tiles_per_slot = t.nseg > 1 ? t.seg_tiles : tiles1;
    unsigned bpc, depth;
    if (shared_inputs) { bpc = 8; depth = 2; }
    else if (w == 8) { bpc = backward ? 2 : 1; depth = 4; }
    else if (w == 4) { bpc = 4; depth = backward ? 4 : 2; }
    else if (w == 2) { bpc = 4; depth = 2; }
    else if (tiles_per_slot >= 16) { bpc = backward ? 1 : 2; depth = 2; }
    else if (tiles_per_slot >= 8) { bpc = 2; depth = 2; }
    else { bpc = 4; depth = 2; }
    t.blocks_per_cu = pb.blocks_per_cu ? pb.blocks_per_cu : bpc;
    t.depth = pb.depth ? pb.depth : depth;
    return t;
}

size_t pairs_bytes(const Problem& pb, const Tuning& t) {
    return t.nseg > 1 ? (size_t)pb.rows * (size_t)t.nseg * sizeof(float2) : 0;
}

// Settles the plan for one call: rows are cut only when the workspace can hold the pairs.
// Returns 0, or FMSCAN_E_WORKSPACE when the caller asked for a cut that does not fit.
int settle(const Problem& pb, bool backward, const void* workspace, size_t workspace_bytes, const char* who,
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
    return 0;
}

template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
void launch_fwd(const Problem& pb, const Tuning& t, const void* g, const void* x, const void* h0,
                void* out, const float2* pairs, hipStream_t s) {
    auto kern = fmscan::scan_forward_kernel<T, W, R, P, PLAIN, VEC, FOLD>;
    static std::atomic<uint64_t> last_set{~0ull};
    const Grid grid = throttled_grid((const void*)kern, last_set, pb.rows * t.nseg, R, t.blocks_per_cu);
    kern<<<grid.blocks, 64 * W * R, grid.lds, s>>>((const T*)g, (const T*)x, (const T*)h0, (T*)out,
                                                   pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L,
                                                   t.nseg, t.seg_tiles, pairs);
}

template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
void launch_bwd(const Problem& pb, const Tuning& t, const void* g, const void* G, const void* fpg,
                void* dx, const void* h, const void* x, void* dg, const void* h0, void* dh0,
                const float2* pairs, hipStream_t s) {
    auto kern = fmscan::scan_backward_kernel<T, W, R, P, PLAIN, VEC, FOLD>;
    static std::atomic<uint64_t> last_set{~0ull};
    const Grid grid = throttled_grid((const void*)kern, last_set, pb.rows * t.nseg, R, t.blocks_per_cu);
    kern<<<grid.blocks, 64 * W * R, grid.lds, s>>>(
        (const T*)g, (const T*)G, (const T*)fpg, (T*)dx, (const T*)h, (const T*)x, (T*)dg,
        (const T*)h0, (T*)dh0, pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L, t.nseg, t.seg_tiles, pairs);
}

// Expands the run-time choices (dtype, waves per row, prefetch depth, plain, vector
// access, fold) into the kernel template arguments. F is a generic lambda called with tags.
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
void dispatch(int dtype, const Tuning& t, bool plain, bool vec, bool fold, F&& f) {
    with_dtype(dtype, [&](auto tt) {
        auto with_waves = [&](auto wt, auto rt) {
            auto with_depth = [&](auto dt, auto vt, auto ft) {
                if (plain) f(tt, wt, rt, dt, BoolTag<true>{}, vt, ft);
                else f(tt, wt, rt, dt, BoolTag<false>{}, vt, ft);
            };
            if (!vec) {  // element access: the slow path gets one variant
                with_depth(IntTag<2>{}, BoolTag<false>{}, BoolTag<false>{});
                return;
            }
            auto with_fold = [&](auto dt) {
                if (fold) with_depth(dt, BoolTag<true>{}, BoolTag<true>{});
                else with_depth(dt, BoolTag<true>{}, BoolTag<false>{});
            };
            switch (t.depth) {
                case 2: with_fold(IntTag<2>{}); break;
                case 3: with_fold(IntTag<3>{}); break;
                default: with_fold(IntTag<4>{}); break;
            }
        };
        switch (t.waves) {
            case 1: with_waves(IntTag<1>{}, IntTag<4>{}); break;  // 4 independent rows per block
            case 2: with_waves(IntTag<2>{}, IntTag<1>{}); break;
            case 4: with_waves(IntTag<4>{}, IntTag<1>{}); break;
            default: with_waves(IntTag<8>{}, IntTag<1>{}); break;
        }
    });
}

// Pass one of a segmented scan: one wave per segment, four segments per block.
template <bool BACKWARD>
void launch_aggregate(int dtype, const Problem& pb, const Tuning& t, bool vec, const void* g,
                      const void* other, float2* pairs, hipStream_t s) {
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        auto go = [&](auto pt, auto vt) {
            constexpr int R = 4, P = 3;
            auto kern =
                fmscan::scan_aggregate_kernel<T, R, P, decltype(pt)::value, decltype(vt)::value, BACKWARD>;
            const unsigned blocks = (unsigned)((pb.rows * t.nseg + R - 1) / R);
            kern<<<blocks, 64 * R, 0, s>>>((const T*)g, (const T*)other, pairs, pb.rows, (int32_t)pb.M,
                                          (int32_t)pb.D, pb.L, t.nseg, t.seg_tiles);
        };
        const bool plain = pb.plain && !BACKWARD;  // the backward pairs are the same in both forms
        if (plain) {
            if (vec) go(BoolTag<true>{}, BoolTag<true>{});
            else go(BoolTag<true>{}, BoolTag<false>{});
        } else {
            if (vec) go(BoolTag<false>{}, BoolTag<true>{});
            else go(BoolTag<false>{}, BoolTag<false>{});
        }
    });
}

constexpr int kReducedGroup = 8;  // consecutive d one block of the reduced backward kernel sums over
constexpr int kReducedChunk = 4;  // tiles of a row visited before moving to the next m
constexpr int kLayerChunk = 2;    // ... in the form that makes the states' gradient on the spot
constexpr int kReducedDepth = 1;  // visits whose loads are in flight ahead of the one worked on

}  // namespace

extern "C" {

int fmscan_abi_version(void) { return FMSCAN_ABI_VERSION; }

const char* fmscan_last_error(void) { return g_err; }

size_t fmscan_workspace_bytes(int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags) {
    Problem pb;
    if (parse(B, M, D, L, dtype, flags, &pb)) return 0;
    return pairs_bytes(pb, choose(pb, false, true));  // the cut is the same in both directions
}

int fmscan_forward(const void* gates, const void* tokens, const void* initial_state, void* out,
                   int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                   void* workspace, size_t workspace_bytes, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags, &pb)) return rc;
    if (!gates || !tokens || !out)
        return fail(FMSCAN_E_NULL, "fmscan_forward: gates, tokens and out must not be NULL");
    const Range o{"out", out, pb.rows * L * pb.esize};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {"tokens", tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize},
                         {"workspace", workspace, (int64_t)workspace_bytes}};
    for (const Range& in : ins)
        if (overlap(o, in))
            return fail(FMSCAN_E_ALIAS, "fmscan_forward: out overlaps %s", in.name);

    const bool vec = (L * pb.esize) % 16 == 0 && aligned16(gates) && aligned16(tokens) && aligned16(out);
    Tuning tune;
    if (int rc = settle(pb, false, workspace, workspace_bytes, "fmscan_forward", &tune)) return rc;
    float2* pairs = tune.nseg > 1 ? (float2*)workspace : nullptr;
    if (pairs) {
        launch_aggregate<false>(dtype, pb, tune, vec, gates, tokens, pairs, (hipStream_t)stream);
        if (int rc = launched("forward (segment pass)")) return rc;
    }
    const bool fold = M == 1 && D == 1;
    dispatch(dtype, tune, pb.plain, vec, fold, [&](auto tt, auto wt, auto rt, auto dt, auto pt, auto vt, auto ft) {
        using T = typename decltype(tt)::type;
        launch_fwd<T, decltype(wt)::value, decltype(rt)::value, decltype(dt)::value, decltype(pt)::value,
                   decltype(vt)::value, decltype(ft)::value>(pb, tune, gates, tokens, initial_state, out,
                                                             pairs, (hipStream_t)stream);
    });
    return launched("forward");
}

int fmscan_backward(const void* gates, const void* out_grad, const void* first_prop_grad,
                    void* token_grad_out, const void* cached_output, const void* input_tokens,
                    void* gate_grad_out, const void* initial_state, void* initial_state_grad,
                    int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                    void* workspace, size_t workspace_bytes, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags, &pb)) return rc;
    if (!gates || !out_grad || !token_grad_out || !cached_output || !gate_grad_out)
        return fail(FMSCAN_E_NULL,
                    "fmscan_backward: gates, out_grad, token_grad_out, cached_output and "
                    "gate_grad_out must not be NULL");
    if (!pb.plain && !input_tokens)
        return fail(FMSCAN_E_NULL, "fmscan_backward: input_tokens must not be NULL without FMSCAN_FLAG_PLAIN");
    const int64_t full = pb.rows * L * pb.esize;
    const Range outs[] = {{"token_grad_out", token_grad_out, full},
                          {"gate_grad_out", gate_grad_out, full},
                          {"initial_state_grad", initial_state_grad, pb.rows * pb.esize},
                          {"workspace", workspace, (int64_t)workspace_bytes}};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {"out_grad", out_grad, full},
                         {"first_prop_grad", first_prop_grad, pb.rows * pb.esize},
                         {"cached_output", cached_output, full},
                         {"input_tokens", pb.plain ? nullptr : input_tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in))
                return fail(FMSCAN_E_ALIAS, "fmscan_backward: %s overlaps %s", o.name, in.name);
    for (int i = 0; i < 4; ++i)
        for (int j = i + 1; j < 4; ++j)
            if (overlap(outs[i], outs[j]))
                return fail(FMSCAN_E_ALIAS, "fmscan_backward: %s overlaps %s", outs[i].name, outs[j].name);

    // NULL initial_state reproduces the reference kernel: h[-1] := first_prop_grad.
    const void* h_init = initial_state ? initial_state : first_prop_grad;

    const bool vec = (L * pb.esize) % 16 == 0 && aligned16(gates) && aligned16(out_grad) &&
                     aligned16(token_grad_out) && aligned16(cached_output) &&
                     (pb.plain || aligned16(input_tokens)) && aligned16(gate_grad_out);
    Tuning tune;
    if (int rc = settle(pb, true, workspace, workspace_bytes, "fmscan_backward", &tune)) return rc;
    float2* pairs = tune.nseg > 1 ? (float2*)workspace : nullptr;
    if (pairs) {
        launch_aggregate<true>(dtype, pb, tune, vec, gates, out_grad, pairs, (hipStream_t)stream);
        if (int rc = launched("backward (segment pass)")) return rc;
    }
    const bool fold = M == 1 && D == 1;
    dispatch(dtype, tune, pb.plain, vec, fold, [&](auto tt, auto wt, auto rt, auto dt, auto pt, auto vt, auto ft) {
        using T = typename decltype(tt)::type;
        launch_bwd<T, decltype(wt)::value, decltype(rt)::value, decltype(dt)::value, decltype(pt)::value,
                   decltype(vt)::value, decltype(ft)::value>(pb, tune, gates, out_grad, first_prop_grad,
                                                             token_grad_out, cached_output, input_tokens,
                                                             gate_grad_out, h_init, initial_state_grad,
                                                             pairs, (hipStream_t)stream);
    });
    return launched("backward");
}

int64_t fmscan_reduced_groups(int64_t D) { return D < 1 ? 0 : (D + kReducedGroup - 1) / kReducedGroup; }

// Shared by fmscan_backward_reduced and fmscan_backward_layer (coef_out != NULL): in the second
// form `out_grad` carries the normalised states and the gradient of the states is made in the kernel.
static int backward_reduced(const char* who, const void* gates, const void* out_grad, const void* first_prop_grad,
                            void* token_grad, const void* cached_output, const void* input_tokens,
                            float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                            const void* coef_out, const void* coef_self, const void* layer_out_grad,
                            const void* rms, int64_t B, int64_t M, int64_t D, int64_t L, int dtype,
                            unsigned flags, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags & FMSCAN_FLAG_PLAIN, &pb)) return rc;
    if (flags & ~FMSCAN_FLAG_PLAIN)
        return fail(FMSCAN_E_FLAGS, "%s: only FMSCAN_FLAG_PLAIN is understood here", who);
    const bool layer = coef_out != nullptr;
    const bool recover = layer && !cached_output;  // the states come back from states_n * rms
    if (!gates || !out_grad || !token_grad || (!cached_output && !recover) || !gate_grad_partial)
        return fail(FMSCAN_E_NULL, "%s: gates, %s, token_grad, cached_output and gate_grad_partial must not "
                    "be NULL", who, coef_out ? "states_n" : "out_grad");
    if (recover && !rms)
        return fail(FMSCAN_E_NULL, "%s: without cached_output the states are states_n * rms: rms must "
                    "not be NULL", who);
    if (layer && (!coef_self || !layer_out_grad))
        return fail(FMSCAN_E_NULL, "%s: coef_self and out_grad must not be NULL", who);
    if (!pb.plain && !input_tokens)
        return fail(FMSCAN_E_NULL, "%s: input_tokens must not be NULL without FMSCAN_FLAG_PLAIN", who);
    if (B > INT32_MAX / fmscan_reduced_groups(D))
        return fail(FMSCAN_E_SHAPE, "%s: B * ceil(D/%d) must be < 2^31", who, kReducedGroup);
    const int64_t full = pb.rows * L * pb.esize;
    const int64_t groups = fmscan_reduced_groups(D);
    const Range outs[] = {{"token_grad", token_grad, B * D * L * pb.esize},
                          {"gate_grad_partial", gate_grad_partial, B * M * groups * L * 4},
                          {"initial_state_grad", initial_state_grad, pb.rows * pb.esize}};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {layer ? "states_n" : "out_grad", out_grad, full},
                         {"first_prop_grad", first_prop_grad, pb.rows * pb.esize},
                         {"cached_output", cached_output, full},
                         {"input_tokens", pb.plain ? nullptr : input_tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize},
                         {"coef_out", coef_out, B * M * L * pb.esize},
                         {"coef_self", layer ? coef_self : nullptr, B * M * L * pb.esize},
                         {"out_grad", layer ? layer_out_grad : nullptr, B * D * L * pb.esize},
                         {"rms", recover ? rms : nullptr, B * M * L * pb.esize}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, o.name, in.name);
    for (int i = 0; i < 3; ++i)
        for (int j = i + 1; j < 3; ++j)
            if (overlap(outs[i], outs[j]))
                return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, outs[i].name, outs[j].name);
    const bool vec = (L * pb.esize) % 16 == 0 && aligned16(gates) && aligned16(out_grad) &&
                     aligned16(token_grad) && aligned16(cached_output) && (!recover || aligned16(rms)) &&
                     (pb.plain || aligned16(input_tokens)) && aligned16(gate_grad_partial) &&
                     (!layer || (aligned16(coef_out) && aligned16(coef_self) && aligned16(layer_out_grad)));
    if (!vec)
        return fail(FMSCAN_E_UNALIGNED, "%s: pointers and L * sizeof(element) must be multiples of 16 bytes", who);
    const size_t tile = (size_t)(16 / pb.esize) * 64;
    const size_t lds = (2 * kReducedGroup * tile + (size_t)kReducedGroup * (size_t)M) * sizeof(float);
    if (lds > 160u * 1024u)
        return fail(FMSCAN_E_SHAPE, "%s: M = %lld needs %zu bytes of LDS (limit 163840)", who, (long long)M, lds);
    if ((L + (int64_t)tile - 1) / (int64_t)tile + kReducedChunk > INT32_MAX / M)
        return fail(FMSCAN_E_SHAPE, "%s: M * ceil(L / %zu) must be < 2^31", who, tile);
    const void* h_init = initial_state ? initial_state : first_prop_grad;
    const unsigned grid = (unsigned)(B * groups);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        auto go = [&](auto pt, auto lt, auto ct) {
            auto kern = fmscan::scan_backward_reduced_kernel<T, kReducedGroup, decltype(ct)::value, kReducedDepth,
                                                             decltype(pt)::value, decltype(lt)::value>;  // lt: 0 plain call, 1 layer, 2 layer + recovered states
            if (lds > 48u * 1024u)
                (void)hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            kern<<<grid, 64 * kReducedGroup, lds, (hipStream_t)stream>>>(
                (const T*)gates, (const T*)out_grad, (const T*)first_prop_grad, (T*)token_grad,
                (const T*)cached_output, (const T*)input_tokens, gate_grad_partial, (const T*)h_init,
                (T*)initial_state_grad, (const T*)coef_out, (const T*)coef_self, (const T*)layer_out_grad,
                (const T*)(recover ? rms : nullptr), (int32_t)M, (int32_t)D, L);
        };
        auto with_plain = [&](auto lt, auto ct) {
            if (pb.plain) go(BoolTag<true>{}, lt, ct);
            else go(BoolTag<false>{}, lt, ct);
        };
        // the layer forms hold three more loads per ring entry: two tiles per visit instead of four
        if (recover) with_plain(IntTag<2>{}, IntTag<kLayerChunk>{});
        else if (layer) with_plain(IntTag<1>{}, IntTag<kLayerChunk>{});
        else with_plain(IntTag<0>{}, IntTag<kReducedChunk>{});
    });
    return launched(who);
}

int fmscan_backward_reduced(const void* gates, const void* out_grad, const void* first_prop_grad,
                            void* token_grad, const void* cached_output, const void* input_tokens,
                            float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                            int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                            void* stream) {
    return backward_reduced("fmscan_backward_reduced", gates, out_grad, first_prop_grad, token_grad, cached_output,
                            input_tokens, gate_grad_partial, initial_state, initial_state_grad, nullptr, nullptr,
                            nullptr, nullptr, B, M, D, L, dtype, flags, stream);
}

int fmscan_backward_layer(const void* gates, const void* states_n, const void* coef_out, const void* coef_self,
                          const void* out_grad, const void* first_prop_grad, void* token_grad,
                          const void* cached_output, const void* rms, const void* input_tokens,
                          float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                          int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags, void* stream) {
    if (!coef_out) return fail(FMSCAN_E_NULL, "fmscan_backward_layer: coef_out must not be NULL");
    return backward_reduced("fmscan_backward_layer", gates, states_n, first_prop_grad, token_grad, cached_output,
                            input_tokens, gate_grad_partial, initial_state, initial_state_grad, coef_out, coef_self,
                            out_grad, rms, B, M, D, L, dtype, flags, stream);
}

}  // extern "C"

// ---- read-out of the Factorization-Memory layer -----------------------------------------

namespace {

constexpr int kRowDotWaves = 8;  // waves of a block that share the D rows of a slot
constexpr int kReadoutRows = 4;  // consecutive d per wave in the read-out kernels

struct ReadoutShape {
    int64_t B, M, D, L;
    int esize;
    int32_t tiles;
};

int parse_readout(const char* who, int64_t B, int64_t M, int64_t D, int64_t L, int dtype, ReadoutShape* rs) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, 0, &pb)) return rc;
    const int64_t tile = (16 / pb.esize) * 64;
    const int64_t tiles = (L + tile - 1) / tile;
    if (D >= (1 << 20) || (__int128)B * M * tiles > (__int128)INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: D must be < 2^20 and B * M * ceil(L / %lld) < 2^31", who, (long long)tile);
    rs->B = B; rs->M = M; rs->D = D; rs->L = L;
    rs->esize = pb.esize;
    rs->tiles = (int32_t)tiles;
    return 0;
}

bool vector_path(const ReadoutShape& rs, std::initializer_list<const void*> pointers) {
    if ((rs.L * rs.esize) % 16 != 0) return false;
    for (const void* p : pointers)
        if (p && !aligned16(p)) return false;
    return true;
}

// As for the scan kernels: an untouched slice of dynamic LDS per block bounds how many blocks
// (rows that stream at once) a compute unit holds.
constexpr unsigned kReadoutBlocksPerCU = 4;  // measured on the layer shapes of bench.py
template <typename K>
unsigned capped_lds(K kern, std::atomic<uint64_t>& last_set) {
    if (kReadoutBlocksPerCU == 0) return 0;
    return throttled_grid((const void*)kern, last_set, 1, 1, kReadoutBlocksPerCU).lds;
}

template <typename F>
void with_bool(bool v, F&& f) {
    if (v) f(BoolTag<true>{});
    else f(BoolTag<false>{});
}

}  // namespace

extern "C" {

int fmscan_readout_inv_rms(const void* states, float* inv_rms, int64_t B, int64_t M, int64_t D, int64_t L,
                           int dtype, float eps, void* stream) {
    ReadoutShape rs;
    if (int rc = parse_readout("fmscan_readout_inv_rms", B, M, D, L, dtype, &rs)) return rc;
    if (!states || !inv_rms) return fail(FMSCAN_E_NULL, "fmscan_readout_inv_rms: states and inv_rms must not be NULL");
    if (!(eps >= 0.0f)) return fail(FMSCAN_E_SHAPE, "fmscan_readout_inv_rms: eps must be >= 0");
    if (overlap({"inv_rms", inv_rms, B * M * L * 4}, {"states", states, B * M * D * L * rs.esize}))
        return fail(FMSCAN_E_ALIAS, "fmscan_readout_inv_rms: inv_rms overlaps states");
    const bool vec = vector_path(rs, {states});
    const unsigned grid = (unsigned)(B * M * rs.tiles);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(vec, [&](auto vt) {
            fmscan::rowdot_kernel<T, kRowDotWaves, fmscan::RowDot::kSumSq, false, decltype(vt)::value>
                <<<grid, 64 * kRowDotWaves, 0, (hipStream_t)stream>>>((const T*)states, nullptr, nullptr, inv_rms,
                                                                      nullptr, nullptr, nullptr, nullptr, nullptr,
                                                                      nullptr, (int32_t)M, (int32_t)D, L, rs.tiles, eps);
        });
    });
    return launched("read-out (inverse rms)");
}

int fmscan_readout_forward(const void* states, const float* inv_rms, const void* read, void* states_out,
                           void* output, int64_t B, int64_t M, int64_t D, int64_t L, int dtype, void* stream) {
    ReadoutShape rs;
    if (int rc = parse_readout("fmscan_readout_forward", B, M, D, L, dtype, &rs)) return rc;
    if (!states || !read || !output)
        return fail(FMSCAN_E_NULL, "fmscan_readout_forward: states, read and output must not be NULL");
    if (inv_rms && !states_out)
        return fail(FMSCAN_E_NULL, "fmscan_readout_forward: states_out must not be NULL with inv_rms");
    const int64_t full = B * M * D * L * rs.esize;
    const Range out_r = {"output", output, B * D * L * rs.esize};
    const Range sn_r = {"states_out", inv_rms ? states_out : nullptr, full};
    const Range ins[] = {{"states", states, full}, {"inv_rms", inv_rms, B * M * L * 4},
                         {"read", read, B * M * L * rs.esize}};
    for (const Range& in : ins) {
        if (overlap(out_r, in)) return fail(FMSCAN_E_ALIAS, "fmscan_readout_forward: output overlaps %s", in.name);
        // states_out == states (in place) is allowed: every element is read before it is written
        if (overlap(sn_r, in) && !(in.p == states && states_out == states))
            return fail(FMSCAN_E_ALIAS, "fmscan_readout_forward: states_out overlaps %s", in.name);
    }
    if (overlap(out_r, sn_r)) return fail(FMSCAN_E_ALIAS, "fmscan_readout_forward: output overlaps states_out");
    const bool vec = vector_path(rs, {states, inv_rms, read, inv_rms ? states_out : nullptr, output});
    const dim3 grid((unsigned)(B * rs.tiles), (unsigned)((D + 4 * kReadoutRows - 1) / (4 * kReadoutRows)));
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(inv_rms != nullptr, [&](auto nt) {
            with_bool(vec, [&](auto vt) {
                auto kern = fmscan::readout_forward_kernel<T, kReadoutRows, decltype(nt)::value, decltype(vt)::value>;
                static std::atomic<uint64_t> last_set{~0ull};
                kern<<<grid, 256, capped_lds(kern, last_set), (hipStream_t)stream>>>(
                    (const T*)states, inv_rms, (const T*)read, (T*)states_out, (T*)output, (int32_t)M, (int32_t)D,
                    L, rs.tiles);
            });
        });
    });
    return launched("read-out (forward)");
}

int fmscan_readout_dot(const void* states_n, const void* out_grad, const void* ext_grad, float* q, float* qe,
                       const float* inv_rms, const void* read, void* coef_out, void* coef_self, void* rms_out,
                       int64_t B, int64_t M, int64_t D, int64_t L, int dtype, void* stream) {
    ReadoutShape rs;
    if (int rc = parse_readout("fmscan_readout_dot", B, M, D, L, dtype, &rs)) return rc;
    if (!states_n || !out_grad || !q)
        return fail(FMSCAN_E_NULL, "fmscan_readout_dot: states_n, out_grad and q must not be NULL");
    if (ext_grad && !qe) return fail(FMSCAN_E_NULL, "fmscan_readout_dot: qe must not be NULL with ext_grad");
    if ((coef_out || coef_self) && (!coef_out || !coef_self || !read))
        return fail(FMSCAN_E_NULL, "fmscan_readout_dot: coef_out, coef_self and read go together");
    if (rms_out && !inv_rms) return fail(FMSCAN_E_NULL, "fmscan_readout_dot: rms_out needs inv_rms");
    const int64_t full = B * M * D * L * rs.esize, slot = B * M * L;
    const Range outs[] = {{"q", q, slot * 4}, {"qe", ext_grad ? qe : nullptr, slot * 4},
                          {"coef_out", coef_out, slot * rs.esize}, {"coef_self", coef_self, slot * rs.esize},
                          {"rms_out", rms_out, slot * rs.esize}};
    const Range ins[] = {{"states_n", states_n, full}, {"out_grad", out_grad, B * D * L * rs.esize},
                         {"ext_grad", ext_grad, full}, {"inv_rms", (coef_out || rms_out) ? inv_rms : nullptr, slot * 4},
                         {"read", coef_out ? read : nullptr, slot * rs.esize}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "fmscan_readout_dot: %s overlaps %s", o.name, in.name);
    for (int i = 0; i < 5; ++i)
        for (int j = i + 1; j < 5; ++j)
            if (overlap(outs[i], outs[j]))
                return fail(FMSCAN_E_ALIAS, "fmscan_readout_dot: %s overlaps %s", outs[i].name, outs[j].name);
    const bool vec = vector_path(rs, {states_n, out_grad, ext_grad});
    const unsigned grid = (unsigned)(B * M * rs.tiles);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(ext_grad != nullptr, [&](auto et) {
            with_bool(vec, [&](auto vt) {
                fmscan::rowdot_kernel<T, kRowDotWaves, fmscan::RowDot::kDot, decltype(et)::value, decltype(vt)::value>
                    <<<grid, 64 * kRowDotWaves, 0, (hipStream_t)stream>>>(
                        (const T*)states_n, (const T*)out_grad, (const T*)ext_grad, q, qe, inv_rms, (const T*)read,
                        (T*)coef_out, (T*)coef_self, (T*)rms_out, (int32_t)M, (int32_t)D, L, rs.tiles, 0.0f);
            });
        });
    });
    return launched("read-out (dot)");
}

int fmscan_readout_backward(const void* states_n, const float* inv_rms, const void* read, const void* out_grad,
                            const void* ext_grad, const float* q, const float* qe, void* state_grad, int64_t B,
                            int64_t M, int64_t D, int64_t L, int dtype, void* stream) {
    ReadoutShape rs;
    if (int rc = parse_readout("fmscan_readout_backward", B, M, D, L, dtype, &rs)) return rc;
    if (!read || !out_grad || !state_grad)
        return fail(FMSCAN_E_NULL, "fmscan_readout_backward: read, out_grad and state_grad must not be NULL");
    const bool norm = inv_rms != nullptr;
    if (norm && (!states_n || !q))
        return fail(FMSCAN_E_NULL, "fmscan_readout_backward: states_n and q must not be NULL with inv_rms");
    if (norm && ext_grad && !qe)
        return fail(FMSCAN_E_NULL, "fmscan_readout_backward: qe must not be NULL with inv_rms and ext_grad");
    const int64_t full = B * M * D * L * rs.esize;
    const Range out_r = {"state_grad", state_grad, full};
    const Range ins[] = {{"states_n", norm ? states_n : nullptr, full}, {"inv_rms", inv_rms, B * M * L * 4},
                         {"read", read, B * M * L * rs.esize}, {"out_grad", out_grad, B * D * L * rs.esize},
                         {"ext_grad", ext_grad, full}, {"q", norm ? q : nullptr, B * M * L * 4},
                         {"qe", norm && ext_grad ? qe : nullptr, B * M * L * 4}};
    for (const Range& in : ins) {
        // state_grad == ext_grad (in place) is allowed: every element is read before it is written
        if (overlap(out_r, in) && !(in.p == ext_grad && state_grad == ext_grad))
            return fail(FMSCAN_E_ALIAS, "fmscan_readout_backward: state_grad overlaps %s", in.name);
    }
    const bool vec = vector_path(rs, {norm ? states_n : nullptr, inv_rms, read, out_grad, ext_grad,
                                      norm ? (const void*)q : nullptr, norm && ext_grad ? (const void*)qe : nullptr,
                                      state_grad});
    const dim3 grid((unsigned)(B * rs.tiles), (unsigned)((D + 4 * kReadoutRows - 1) / (4 * kReadoutRows)));
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(norm, [&](auto nt) {
            with_bool(ext_grad != nullptr, [&](auto et) {
                with_bool(vec, [&](auto vt) {
                    auto kern = fmscan::readout_backward_kernel<T, kReadoutRows, decltype(nt)::value,
                                                                decltype(et)::value, decltype(vt)::value>;
                    static std::atomic<uint64_t> last_set{~0ull};
                    kern<<<grid, 256, capped_lds(kern, last_set), (hipStream_t)stream>>>(
                        (const T*)states_n, inv_rms, (const T*)read, (const T*)out_grad, (const T*)ext_grad, q, qe,
                        (T*)state_grad, (int32_t)M, (int32_t)D, L, rs.tiles);
                });
            });
        });
    });
    return launched("read-out (backward)");
}

int fmscan_layer_prepare(const void* alpha, const void* update_scale, const void* output_scale, void* gates,
                         void* read, int64_t B, int64_t L, int64_t M, int dtype, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, 1, L, dtype, 0, &pb)) return rc;
    if (!alpha || !update_scale || !output_scale || !gates || !read)
        return fail(FMSCAN_E_NULL, "fmscan_layer_prepare: no argument may be NULL");
    const int64_t tiles_t = (L + 63) / 64, tiles_m = (M + 63) / 64;
    if ((__int128)B * tiles_t * tiles_m > (__int128)INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "fmscan_layer_prepare: too many tiles for one launch");
    const int64_t big = B * L * M * pb.esize, small = B * L * pb.esize;
    const Range outs[] = {{"gates", gates, big}, {"read", read, big}};
    const Range ins[] = {{"alpha", alpha, big}, {"update_scale", update_scale, small},
                         {"output_scale", output_scale, small}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "fmscan_layer_prepare: %s overlaps %s", o.name, in.name);
    if (overlap(outs[0], outs[1])) return fail(FMSCAN_E_ALIAS, "fmscan_layer_prepare: gates overlaps read");
    const unsigned grid = (unsigned)(B * tiles_t * tiles_m);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        fmscan::layer_prepare_kernel<T><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const T*)alpha, (const T*)update_scale, (const T*)output_scale, (T*)gates, (T*)read, L, M,
            (int32_t)tiles_t, (int32_t)tiles_m);
    });
    return launched("layer (prepare)");
}

int fmscan_layer_finish(const float* gate_grad_partial, int64_t G, const float* read_grad, const void* alpha,
                        const void* update_scale, const void* output_scale, void* alpha_grad,
                        void* update_scale_grad, void* output_scale_grad, int64_t B, int64_t L, int64_t M,
                        int dtype, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, 1, L, dtype, 0, &pb)) return rc;
    if (G < 1 || G > INT32_MAX) return fail(FMSCAN_E_SHAPE, "fmscan_layer_finish: G must be >= 1");
    if (!gate_grad_partial || !read_grad || !alpha || !update_scale || !output_scale || !alpha_grad ||
        !update_scale_grad || !output_scale_grad)
        return fail(FMSCAN_E_NULL, "fmscan_layer_finish: no argument may be NULL");
    const int64_t tiles_t = (L + 63) / 64;
    if ((__int128)B * tiles_t > (__int128)INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "fmscan_layer_finish: too many tiles for one launch");
    const int64_t big = B * L * M * pb.esize, small = B * L * pb.esize;
    const Range outs[] = {{"alpha_grad", alpha_grad, big}, {"update_scale_grad", update_scale_grad, small},
                          {"output_scale_grad", output_scale_grad, small}};
    const Range ins[] = {{"gate_grad_partial", gate_grad_partial, B * M * G * L * 4},
                         {"read_grad", read_grad, B * M * L * 4}, {"alpha", alpha, big},
                         {"update_scale", update_scale, small}, {"output_scale", output_scale, small}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "fmscan_layer_finish: %s overlaps %s", o.name, in.name);
    for (int i = 0; i < 3; ++i)
        for (int j = i + 1; j < 3; ++j)
            if (overlap(outs[i], outs[j]))
                return fail(FMSCAN_E_ALIAS, "fmscan_layer_finish: %s overlaps %s", outs[i].name, outs[j].name);
    const unsigned grid = (unsigned)(B * tiles_t);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        fmscan::layer_finish_kernel<T><<<grid, 256, 0, (hipStream_t)stream>>>(
            gate_grad_partial, (int32_t)G, read_grad, (const T*)alpha, (const T*)update_scale,
            (const T*)output_scale, (T*)alpha_grad, (T*)update_scale_grad, (T*)output_scale_grad, L, M,
            (int32_t)tiles_t);
    });
    return launched("layer (finish)");
}

int fmscan_swap_last_two(const void* src, void* dst, int64_t B, int64_t R, int64_t C, int element_size,
                         void* stream) {
    if (!src || !dst) return fail(FMSCAN_E_NULL, "fmscan_swap_last_two: src and dst must not be NULL");
    if (B < 1 || R < 1 || C < 1) return fail(FMSCAN_E_SHAPE, "fmscan_swap_last_two: B, R, C must be >= 1");
    if (element_size != 2 && element_size != 4)
        return fail(FMSCAN_E_DTYPE, "fmscan_swap_last_two: element size must be 2 or 4 bytes (got %d)", element_size);
    const int64_t tiles_r = (R + 63) / 64, tiles_c = (C + 63) / 64;
    if (tiles_r > INT32_MAX || tiles_c > INT32_MAX || (__int128)B * tiles_r * tiles_c > (__int128)INT32_MAX ||
        (__int128)B * R * C > ((__int128)1 << 46))
        return fail(FMSCAN_E_SHAPE, "fmscan_swap_last_two: too many tiles for one launch");
    const int64_t bytes = B * R * C * element_size;
    if (overlap({"dst", dst, bytes}, {"src", src, bytes}))
        return fail(FMSCAN_E_ALIAS, "fmscan_swap_last_two: dst overlaps src");
    const unsigned grid = (unsigned)(B * tiles_r * tiles_c);
    if (element_size == 2 && R % 2 == 0 && C % 2 == 0 && ((uintptr_t)src & 3u) == 0 && ((uintptr_t)dst & 3u) == 0)
        fmscan::swap_last_two_pairs_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, (uint16_t*)dst, R, C, (int32_t)tiles_c, (int32_t)tiles_r);
    else if (element_size == 2)
        fmscan::swap_last_two_kernel<uint16_t><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, (uint16_t*)dst, R, C, (int32_t)tiles_c, (int32_t)tiles_r);
    else
        fmscan::swap_last_two_kernel<uint32_t><<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint32_t*)src, (uint32_t*)dst, R, C, (int32_t)tiles_c, (int32_t)tiles_r);
    return launched("swap of the last two axes");
}

}  // extern "C"
