// Host side of libfmscan_hip.so: argument checks, choice of kernel variant,
// launch. Declarations and the contract of every entry point: include/fmscan.h.
#include "../../include/fmscan.h"

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>

#include "fmscan_kernels.h"

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
    unsigned waves;  // requested waves per row, 0 = auto
    unsigned blocks_per_cu;  // requested cap on resident blocks per CU, 0 = auto
    unsigned depth;          // requested prefetch depth in tiles, 0 = auto
    bool plain;
};

int parse(int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags, Problem* pb) {
    if (B < 1 || M < 1 || D < 1 || L < 1)
        return fail(FMSCAN_E_SHAPE, "fmscan: B, M, D, L must be >= 1 (got %lld, %lld, %lld, %lld)",
                    (long long)B, (long long)M, (long long)D, (long long)L);
    if (M > INT32_MAX || D > INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "fmscan: M and D must fit 32 bits");
    if (dtype != FMSCAN_DTYPE_F32 && dtype != FMSCAN_DTYPE_F16 && dtype != FMSCAN_DTYPE_BF16)
        return fail(FMSCAN_E_DTYPE, "fmscan: dtype %d is not float32 (0), float16 (1) or bfloat16 (2)",
                    dtype);
    if (flags & ~(FMSCAN_FLAG_PLAIN | FMSCAN_FLAG_WAVES_MASK | FMSCAN_FLAG_BLOCKS_MASK |
                  FMSCAN_FLAG_DEPTH_MASK))
        return fail(FMSCAN_E_FLAGS, "fmscan: unknown flag bits 0x%x", flags);
    const unsigned waves = (flags & FMSCAN_FLAG_WAVES_MASK) >> FMSCAN_FLAG_WAVES_SHIFT;
    if (waves != 0 && waves != 1 && waves != 2 && waves != 4 && waves != 8)
        return fail(FMSCAN_E_FLAGS, "fmscan: waves per row must be 0 (auto), 1, 2, 4 or 8 (got %u)",
                    waves);
    // rows*L elements must be addressable and the grid must fit 31 bits
    const __int128 rows = (__int128)B * M * D;
    if (rows > (__int128)INT32_MAX || rows * L > ((__int128)1 << 46))
        return fail(FMSCAN_E_SHAPE, "fmscan: B*M*D = rows must be < 2^31 and rows*L <= 2^46");
    pb->B = B; pb->M = M; pb->D = D; pb->L = L;
    pb->rows = (int64_t)rows;
    pb->esize = dtype == FMSCAN_DTYPE_F32 ? 4 : 2;
    pb->waves = waves;
    pb->blocks_per_cu = (flags & FMSCAN_FLAG_BLOCKS_MASK) >> FMSCAN_FLAG_BLOCKS_SHIFT;
    pb->depth = (flags & FMSCAN_FLAG_DEPTH_MASK) >> FMSCAN_FLAG_DEPTH_SHIFT;
    if (pb->depth != 0 && (pb->depth < 2 || pb->depth > 4))
        return fail(FMSCAN_E_FLAGS, "fmscan: prefetch depth must be 0 (auto), 2, 3 or 4 (got %u)", pb->depth);
    pb->plain = (flags & FMSCAN_FLAG_PLAIN) != 0;
    return 0;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

int launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "fmscan: %s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

// One block per R rows. Each block also asks for a share of the 160 KiB of LDS of a
// compute unit that it never touches: at most `blocks_per_cu` blocks then fit a unit
// at a time, which bounds the number of rows that stream concurrently.
struct Grid {
    unsigned blocks, lds;
};
Grid throttled_grid(const void* kern, int64_t rows, int R, unsigned blocks_per_cu) {
    Grid g;
    g.blocks = (unsigned)((rows + R - 1) / R);
    g.lds = ((160u * 1024u - 2048u) / blocks_per_cu) & ~1023u;
    static std::atomic<uint64_t> last_set{~0ull};  // (kernel, device, bytes) of the last attribute call
    int dev = 0;
    (void)hipGetDevice(&dev);
    const uint64_t key = ((uint64_t)(uintptr_t)kern << 24) ^ ((uint64_t)dev << 20) ^ g.lds;
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

// Waves per row, resident blocks per compute unit and prefetch depth when the caller
// leaves the choice to the library. The table comes from sweeps on an MI355X over the
// benchmark shapes (rows x L): 131072 x 2048, 32768 x 16384, 4096 x 65536 in 16-bit types
// and 8192 x 4096 in float32. What it encodes: a wave per row streams best when there are
// many rows of moderate length; long rows want several waves side by side so that fewer
// rows are open at a time; with few rows a block per row keeps every compute unit busy.
// About two waves per SIMD is where HBM efficiency peaks; more resident rows lower it.
struct Tuning {
    unsigned waves, blocks_per_cu, depth;
};
Tuning choose(const Problem& pb) {
    Tuning t;
    const int64_t tile1 = (16 / pb.esize) * 64;               // elements one wave covers per tile
    const int64_t tiles1 = (pb.L + tile1 - 1) / tile1;        // tiles per row for one wave
    unsigned w = pb.waves;
    if (!w) {
        if (tiles1 >= 64) w = 4;
        else if (pb.rows < 16384 && tiles1 >= 8) w = 8;
        else w = 1;
        while (w > 1 && tiles1 < (int64_t)w) w /= 2;                                     // row shorter than a tile
        while (w < 8 && pb.rows * w < 1024 && tiles1 >= 2 * (int64_t)w) w *= 2;           // very few rows
    }
    t.waves = w;
    if (pb.blocks_per_cu) t.blocks_per_cu = pb.blocks_per_cu;
    else if (w == 1) t.blocks_per_cu = tiles1 >= 16 ? 2 : 4;
    else if (w == 4) t.blocks_per_cu = 2;
    else t.blocks_per_cu = 4;
    if (pb.depth) t.depth = pb.depth;
    else if (w == 1) t.depth = tiles1 >= 16 ? 3 : 4;
    else if (w == 4) t.depth = 4;
    else t.depth = 3;
    return t;
}

template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
void launch_fwd(const Problem& pb, unsigned bpc, const void* g, const void* x, const void* h0, void* out,
                hipStream_t s) {
    auto kern = fmscan::scan_forward_kernel<T, W, R, P, PLAIN, VEC, FOLD>;
    const Grid grid = throttled_grid((const void*)kern, pb.rows, R, bpc);
    kern<<<grid.blocks, 64 * W * R, grid.lds, s>>>(
        (const T*)g, (const T*)x, (const T*)h0, (T*)out, pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L);
}

template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
void launch_bwd(const Problem& pb, unsigned bpc, const void* g, const void* G, const void* fpg, void* dx,
                const void* h, const void* x, void* dg, const void* h0, hipStream_t s) {
    auto kern = fmscan::scan_backward_kernel<T, W, R, P, PLAIN, VEC, FOLD>;
    const Grid grid = throttled_grid((const void*)kern, pb.rows, R, bpc);
    kern<<<grid.blocks, 64 * W * R, grid.lds, s>>>(
        (const T*)g, (const T*)G, (const T*)fpg, (T*)dx, (const T*)h, (const T*)x, (T*)dg,
        (const T*)h0, pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L);
}

// Expands the run-time choices (dtype, waves per row, prefetch depth, plain, vector
// access) into the kernel template arguments. F is a generic lambda called with tags.
template <typename T> struct TypeTag { using type = T; };
template <int V> struct IntTag { static constexpr int value = V; };
template <bool V> struct BoolTag { static constexpr bool value = V; };

template <typename F>
void dispatch(int dtype, const Tuning& t, bool plain, bool vec, bool fold, F&& f) {
    auto with_type = [&](auto tt) {
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
    };
    if (dtype == FMSCAN_DTYPE_F32) with_type(TypeTag<float>{});
    else if (dtype == FMSCAN_DTYPE_F16) with_type(TypeTag<_Float16>{});
    else with_type(TypeTag<__bf16>{});
}

}  // namespace

extern "C" {

int fmscan_abi_version(void) { return FMSCAN_ABI_VERSION; }

const char* fmscan_last_error(void) { return g_err; }

int fmscan_forward(const void* gates, const void* tokens, const void* initial_state, void* out,
                   int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                   void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags, &pb)) return rc;
    if (!gates || !tokens || !out)
        return fail(FMSCAN_E_NULL, "fmscan_forward: gates, tokens and out must not be NULL");
    const Range o{"out", out, pb.rows * L * pb.esize};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {"tokens", tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize}};
    for (const Range& in : ins)
        if (overlap(o, in))
            return fail(FMSCAN_E_ALIAS, "fmscan_forward: out overlaps %s", in.name);

    const bool vec = (L * pb.esize) % 16 == 0 && aligned16(gates) && aligned16(tokens) && aligned16(out);
    const Tuning tune = choose(pb);
    const bool fold = M == 1 && D == 1;
    dispatch(dtype, tune, pb.plain, vec, fold, [&](auto tt, auto wt, auto rt, auto dt, auto pt, auto vt, auto ft) {
        using T = typename decltype(tt)::type;
        launch_fwd<T, decltype(wt)::value, decltype(rt)::value, decltype(dt)::value, decltype(pt)::value,
                   decltype(vt)::value, decltype(ft)::value>(pb, tune.blocks_per_cu, gates, tokens,
                                                             initial_state, out, (hipStream_t)stream);
    });
    return launched("forward");
}

int fmscan_backward(const void* gates, const void* out_grad, const void* first_prop_grad,
                    void* token_grad_out, const void* cached_output, const void* input_tokens,
                    void* gate_grad_out, const void* initial_state, int64_t B, int64_t M, int64_t D,
                    int64_t L, int dtype, unsigned flags, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags, &pb)) return rc;
    if (!gates || !out_grad || !token_grad_out || !cached_output || !gate_grad_out)
        return fail(FMSCAN_E_NULL,
                    "fmscan_backward: gates, out_grad, token_grad_out, cached_output and "
                    "gate_grad_out must not be NULL");
    if (!pb.plain && !input_tokens)
        return fail(FMSCAN_E_NULL, "fmscan_backward: input_tokens must not be NULL without FMSCAN_FLAG_PLAIN");
    const int64_t full = pb.rows * L * pb.esize;
    const Range outs[] = {{"token_grad_out", token_grad_out, full}, {"gate_grad_out", gate_grad_out, full}};
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
    if (overlap(outs[0], outs[1]))
        return fail(FMSCAN_E_ALIAS, "fmscan_backward: token_grad_out overlaps gate_grad_out");

    // NULL initial_state reproduces the reference kernel: h[-1] := first_prop_grad.
    const void* h_init = initial_state ? initial_state : first_prop_grad;

    const bool vec = (L * pb.esize) % 16 == 0 && aligned16(gates) && aligned16(out_grad) &&
                     aligned16(token_grad_out) && aligned16(cached_output) &&
                     (pb.plain || aligned16(input_tokens)) && aligned16(gate_grad_out);
    const Tuning tune = choose(pb);
    const bool fold = M == 1 && D == 1;
    dispatch(dtype, tune, pb.plain, vec, fold, [&](auto tt, auto wt, auto rt, auto dt, auto pt, auto vt, auto ft) {
        using T = typename decltype(tt)::type;
        launch_bwd<T, decltype(wt)::value, decltype(rt)::value, decltype(dt)::value, decltype(pt)::value,
                   decltype(vt)::value, decltype(ft)::value>(pb, tune.blocks_per_cu, gates, out_grad,
                                                             first_prop_grad, token_grad_out, cached_output,
                                                             input_tokens, gate_grad_out, h_init,
                                                             (hipStream_t)stream);
    });
    return launched("backward");
}

}  // extern "C"
