// Host side of libfmscan_hip.so: argument checks, choice of kernel variant,
// launch. Declarations and the contract of every entry point: include/fmscan.h.
#include "../../include/fmscan.h"

#include <hip/hip_runtime.h>

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
    if (flags & ~(FMSCAN_FLAG_PLAIN | FMSCAN_FLAG_WAVES_MASK))
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
    pb->plain = (flags & FMSCAN_FLAG_PLAIN) != 0;
    return 0;
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// Waves per row when the caller leaves the choice to the library. A wave walks
// its row alone unless there are too few rows to fill the chip that way
// (256 CUs x 4 SIMDs x several waves) and the row is long enough to share.
unsigned choose_waves(const Problem& pb) {
    if (pb.waves) return pb.waves;
    const int64_t tile1 = (16 / pb.esize) * 64;  // elements one wave covers per tile
    unsigned w = 1;
    while (w < 8 && pb.rows * w < 8192 && pb.L >= (int64_t)tile1 * w * 2) w *= 2;
    return w;
}

int launched(const char* what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail((int)e, "fmscan: %s launch failed: %s", what, hipGetErrorString(e));
    return 0;
}

template <typename T, int W, int R, bool PLAIN, bool VEC>
void launch_fwd(const Problem& pb, const void* g, const void* x, const void* h0, void* out,
                hipStream_t s) {
    const unsigned grid = (unsigned)((pb.rows + R - 1) / R);
    fmscan::scan_forward_kernel<T, W, R, PLAIN, VEC><<<grid, 64 * W * R, 0, s>>>(
        (const T*)g, (const T*)x, (const T*)h0, (T*)out, pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L);
}

template <typename T, int W, int R, bool PLAIN, bool VEC>
void launch_bwd(const Problem& pb, const void* g, const void* G, const void* fpg, void* dx,
                const void* h, const void* x, void* dg, const void* h0, hipStream_t s) {
    const unsigned grid = (unsigned)((pb.rows + R - 1) / R);
    fmscan::scan_backward_kernel<T, W, R, PLAIN, VEC><<<grid, 64 * W * R, 0, s>>>(
        (const T*)g, (const T*)G, (const T*)fpg, (T*)dx, (const T*)h, (const T*)x, (T*)dg,
        (const T*)h0, pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L);
}

// Expands the run-time choices (dtype, waves per row, plain, vector access) into
// the kernel template arguments. F is a generic lambda called with tag values.
template <typename T> struct TypeTag { using type = T; };
template <int V> struct IntTag { static constexpr int value = V; };
template <bool V> struct BoolTag { static constexpr bool value = V; };

template <typename F>
void dispatch(int dtype, unsigned waves, bool plain, bool vec, F&& f) {
    auto with_type = [&](auto tt) {
        auto with_waves = [&](auto wt, auto rt) {
            if (plain) {
                if (vec) f(tt, wt, rt, BoolTag<true>{}, BoolTag<true>{});
                else f(tt, wt, rt, BoolTag<true>{}, BoolTag<false>{});
            } else {
                if (vec) f(tt, wt, rt, BoolTag<false>{}, BoolTag<true>{});
                else f(tt, wt, rt, BoolTag<false>{}, BoolTag<false>{});
            }
        };
        switch (waves) {
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
    const unsigned waves = choose_waves(pb);
    dispatch(dtype, waves, pb.plain, vec, [&](auto tt, auto wt, auto rt, auto pt, auto vt) {
        using T = typename decltype(tt)::type;
        launch_fwd<T, decltype(wt)::value, decltype(rt)::value, decltype(pt)::value,
                   decltype(vt)::value>(pb, gates, tokens, initial_state, out, (hipStream_t)stream);
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
    const unsigned waves = choose_waves(pb);
    dispatch(dtype, waves, pb.plain, vec, [&](auto tt, auto wt, auto rt, auto pt, auto vt) {
        using T = typename decltype(tt)::type;
        launch_bwd<T, decltype(wt)::value, decltype(rt)::value, decltype(pt)::value,
                   decltype(vt)::value>(pb, gates, out_grad, first_prop_grad, token_grad_out,
                                        cached_output, input_tokens, gate_grad_out, h_init,
                                        (hipStream_t)stream);
    });
    return launched("backward");
}

}  // extern "C"
