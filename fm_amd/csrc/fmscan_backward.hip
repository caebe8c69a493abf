// fmscan_backward: argument checks, choice of kernel variant, launch.
// Contract: include/fmscan.h.
#include "fmscan_host.h"
#include "fmscan_kernels.h"
#include "fmscan_packed.h"

using namespace fmscan::host;

namespace {

template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
int launch_bwd(const Problem& pb, const Tuning& t, const void* g, const void* G, const void* fpg,
               void* dx, const void* h, const void* x, void* dg, const void* h0, void* dh0,
               const float2* pairs, hipStream_t s) {
    auto kern = fmscan::scan_backward_kernel<T, W, R, P, PLAIN, VEC, FOLD>;
    static std::atomic<uint64_t> armed{0};
    if (int rc = raise_lds_limit((const void*)kern, armed, "fmscan_backward")) return rc;
    const unsigned blocks = (unsigned)((pb.rows * t.nseg + R - 1) / R);
    kern<<<blocks, 64 * W * R, lds_share(t.blocks_per_cu), s>>>(
        (const T*)g, (const T*)G, (const T*)fpg, (T*)dx, (const T*)h, (const T*)x, (T*)dg,
        (const T*)h0, (T*)dh0, pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L, t.nseg, t.seg_tiles, pairs);
    return 0;
}

// Pass one of a segmented scan: one wave per segment, four segments per block. The
// backward pairs (g, g * G) are the same with and without the (1 - g) input scaling.
void launch_aggregate(int dtype, const Problem& pb, const Tuning& t, bool vec, const void* g,
                      const void* other, float2* pairs, hipStream_t s) {
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(vec, [&](auto vt) {
            constexpr int R = 4, P = 3;
            auto kern = fmscan::scan_aggregate_kernel<T, R, P, false, decltype(vt)::value, true>;
            const unsigned blocks = (unsigned)((pb.rows * t.nseg + R - 1) / R);
            kern<<<blocks, 64 * R, 0, s>>>((const T*)g, (const T*)other, pairs, pb.rows, (int32_t)pb.M,
                                          (int32_t)pb.D, pb.L, t.nseg, t.seg_tiles);
        });
    });
}

}  // namespace

extern "C" {

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
    const bool fold = M == 1 && D == 1;
    if (packs_rows(pb, vec, true)) {  // short rows: several per wave
        const int32_t lanes_log2 = packed_lanes_log2(pb);
        with_dtype(dtype, [&](auto tt) {
            using T = typename decltype(tt)::type;
            with_bool(pb.plain, [&](auto pt) {
                with_bool(vec, [&](auto vt) { with_bool(fold, [&](auto ft) {
                    fmscan::scan_backward_packed_kernel<T, decltype(pt)::value, decltype(vt)::value, decltype(ft)::value>
                        <<<packed_blocks(pb, lanes_log2), 256, 0, (hipStream_t)stream>>>(
                            (const T*)gates, (const T*)out_grad, (const T*)first_prop_grad, (T*)token_grad_out,
                            (const T*)cached_output, (const T*)input_tokens, (T*)gate_grad_out, (const T*)h_init,
                            (T*)initial_state_grad, pb.rows, (int32_t)pb.M, (int32_t)pb.D, (int32_t)pb.L, lanes_log2);
                }); });
            });
        });
        return launched("backward");
    }
    Tuning tune;
    if (int rc = settle(pb, true, workspace, workspace_bytes, "fmscan_backward", &tune)) return rc;
    float2* pairs = tune.nseg > 1 ? (float2*)workspace : nullptr;
    if (pairs) {
        launch_aggregate(dtype, pb, tune, vec, gates, out_grad, pairs, (hipStream_t)stream);
        if (int rc = launched("backward (segment pass)")) return rc;
    }
    int rc = 0;
    dispatch<true>(dtype, tune, pb.plain, vec, fold, [&](auto tt, auto wt, auto rt, auto dt, auto pt, auto vt, auto ft) {
        using T = typename decltype(tt)::type;
        rc = launch_bwd<T, decltype(wt)::value, decltype(rt)::value, decltype(dt)::value, decltype(pt)::value,
                   decltype(vt)::value, decltype(ft)::value>(pb, tune, gates, out_grad, first_prop_grad,
                                                             token_grad_out, cached_output, input_tokens,
                                                             gate_grad_out, h_init, initial_state_grad,
                                                             pairs, (hipStream_t)stream);
    });
    if (rc) return rc;
    return launched("backward");
}

}  // extern "C"
