// fmscan_backward_reduced and fmscan_backward_layer: the backward scan with the sums over
// D and M inside. Contract: include/fmscan.h.
#include "fmscan_host.h"
#include "fmscan_reduced.h"
#include "fmscan_packed.h"

using namespace fmscan::host;

namespace {

constexpr int kReducedWaves = 4;  // waves of a block: they split the M memory slots between them

// Consecutive d that one block of the reduced backward kernel sums over: 8 where that still leaves two
// blocks (eight waves, all the kernel's registers allow) for each of the 256 compute units, halving the
// partials and the work per slot that does not depend on the row; 4 otherwise, for twice the blocks.
int reduced_group(int64_t B, int64_t D) { return (__int128)B * ((D + 7) / 8) >= 512 ? 8 : 4; }

// Into how many blocks the M slots of a batch element are dealt (1: not at all) so that the blocks reach
// the 512 that fill the GPU. First choice: with groups of 8 rows, the smallest divisor of M that brings the
// (b, group of 8 d) pairs there and leaves every wave two slots (M / split >= 2 * kReducedWaves); measured
// in the layer form (bf16, us, unsplit -> split): (16,32,128,2048) 127 -> 101 (2), (8,32,128,8192) 298 -> 212
// (4), (4,64,128,4096) 261 -> 108 (8), (8,16,256,4096) 122 -> 108 (2). Else with groups of 4 rows: the
// smallest divisor that brings the (b, group of 4 d) pairs there, every wave keeping a slot.
int64_t reduced_split(int64_t B, int64_t M, int64_t D) {
    const __int128 pairs8 = (__int128)B * ((D + 7) / 8);
    if (pairs8 >= 512) return 1;
    const int64_t want8 = (int64_t)((512 + pairs8 - 1) / pairs8);
    for (int64_t s = 2; s <= M / (2 * kReducedWaves); ++s)
        if (M % s == 0 && s >= want8) return s;
    const __int128 pairs = (__int128)B * ((D + 3) / 4);
    if (pairs >= 512 || M < 2 * kReducedWaves) return 1;
    const int64_t want = (int64_t)((512 + pairs - 1) / pairs);
    int64_t best = 1;
    for (int64_t s = 2; s <= M / kReducedWaves; ++s) {
        if (M % s != 0) continue;
        best = s;
        if (s >= want) break;
    }
    return best;
}

}  // namespace

extern "C" {

int64_t fmscan_reduced_groups(int64_t B, int64_t D) {
    if (B < 1 || D < 1) return 0;
    const int64_t group = reduced_group(B, D);
    return (D + group - 1) / group;
}

// Shared by fmscan_backward_reduced and fmscan_backward_layer (coef_out != NULL): in the second
// form `out_grad` carries the normalised states and the gradient of the states is made in the kernel.
// split > 1: the slots of a batch element dealt to `split` blocks; the token gradient then goes to
// token_partial (float32) and token_grad is not written.
static int backward_reduced(const char* who, const void* gates, const void* out_grad, const void* first_prop_grad,
                            void* token_grad, const void* cached_output, const void* input_tokens,
                            float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                            const float* coef_out, const float* coef_self, const void* layer_out_grad,
                            const float* rms, int64_t B, int64_t M, int64_t D, int64_t L, int dtype,
                            unsigned flags, void* stream, float* token_partial = nullptr, int64_t split = 1,
                            bool split_call = false, int64_t segments = 1, void* workspace = nullptr,
                            size_t workspace_bytes = 0) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags & FMSCAN_FLAG_PLAIN, &pb)) return rc;
    if (flags & ~FMSCAN_FLAG_PLAIN)
        return fail(FMSCAN_E_FLAGS, "%s: only FMSCAN_FLAG_PLAIN is understood here", who);
    if (split < 1 || M % split != 0 || split > INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: split = %lld must be >= 1 and divide M = %lld", who, (long long)split,
                    (long long)M);
    if ((split > 1 || split_call) != (token_partial != nullptr))
        return fail(FMSCAN_E_NULL, "%s: token_grad_partial must not be NULL", who);
    const bool layer = coef_out != nullptr;
    const bool recover = layer && !cached_output;  // the states come back from states_n * rms
    if (!gates || !out_grad || (!token_grad && !token_partial) || (!cached_output && !recover) || !gate_grad_partial)
        return fail(FMSCAN_E_NULL, "%s: gates, %s, token_grad, cached_output and gate_grad_partial must not "
                    "be NULL", who, coef_out ? "states_n" : "out_grad");
    if (recover && !rms)
        return fail(FMSCAN_E_NULL, "%s: without cached_output the states are states_n * rms: rms must "
                    "not be NULL", who);
    if (layer && (!coef_self || !layer_out_grad))
        return fail(FMSCAN_E_NULL, "%s: coef_self and out_grad must not be NULL", who);
    if (!pb.plain && !input_tokens)
        return fail(FMSCAN_E_NULL, "%s: input_tokens must not be NULL without FMSCAN_FLAG_PLAIN", who);
    // what the kernel is told: B * split batch elements of M / split slots (the same memory)
    const int64_t Bk = B * split, Mk = M / split;
    const int group = reduced_group(Bk, D);
    const int64_t groups = fmscan_reduced_groups(Bk, D);
    if (Bk > INT32_MAX / groups) return fail(FMSCAN_E_SHAPE, "%s: B * split * ceil(D/%d) must be < 2^31", who, group);
    const int64_t full = pb.rows * L * pb.esize;
    const Range outs[] = {token_partial ? Range{"token_grad_partial", token_partial, B * D * split * L * 4}
                                    : Range{"token_grad", token_grad, B * D * L * pb.esize},
                          {"gate_grad_partial", gate_grad_partial, B * M * groups * L * 4},
                          {"initial_state_grad", initial_state_grad, pb.rows * pb.esize}};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {layer ? "states_n" : "out_grad", out_grad, full},
                         {"first_prop_grad", first_prop_grad, pb.rows * pb.esize},
                         {"cached_output", cached_output, full},
                         {"input_tokens", pb.plain ? nullptr : input_tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize},
                         {"coef_out", coef_out, B * M * L * 4},
                         {"coef_self", layer ? coef_self : nullptr, B * M * L * 4},
                         {"out_grad", layer ? layer_out_grad : nullptr, B * D * L * pb.esize},
                         {"rms", recover ? rms : nullptr, B * M * L * 4}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, o.name, in.name);
    for (int i = 0; i < 3; ++i)
        for (int j = i + 1; j < 3; ++j)
            if (overlap(outs[i], outs[j]))
                return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, outs[i].name, outs[j].name);
    const bool vec = (L * pb.esize) % 16 == 0 && aligned16(gates) && aligned16(out_grad) &&
                     aligned16(token_grad) && aligned16(token_partial) && aligned16(cached_output) &&
                     (!recover || aligned16(rms)) &&
                     (pb.plain || aligned16(input_tokens)) && aligned16(gate_grad_partial) &&
                     (!layer || (aligned16(coef_out) && aligned16(coef_self) && aligned16(layer_out_grad)));
    if (!vec)
        return fail(FMSCAN_E_UNALIGNED, "%s: pointers and L * sizeof(element) must be multiples of 16 bytes", who);
    const size_t tile = (size_t)(16 / pb.esize) * 64;
    const int64_t Mw = (Mk + kReducedWaves - 1) / kReducedWaves;  // slots per wave
    const size_t lds = (2 * group * tile + 2 * (size_t)group * 2 * 64 * 4 + (size_t)kReducedWaves * (size_t)Mw * group +
                        (size_t)kReducedWaves * tile + (size_t)kReducedWaves * (size_t)Mw) * sizeof(float);
    if (lds > kMaxDynamicLds)
        return fail(FMSCAN_E_SHAPE, "%s: M = %lld needs %zu bytes of LDS (limit %u)", who, (long long)M, lds,
                    kMaxDynamicLds);
    if ((L + (int64_t)tile - 1) / (int64_t)tile > INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: ceil(L / %zu) must be < 2^31", who, tile);
    const void* h_init = initial_state ? initial_state : first_prop_grad;
    // the cut: as many segments as asked for, each a whole number of tiles, none empty (layer forms,
    // Factorization-Memory form only); two passes, the segments' step pairs between them in the workspace
    const int64_t ntiles = (L + (int64_t)tile - 1) / (int64_t)tile;
    if (segments < 1 || segments > 255 || segments > ntiles)
        return fail(FMSCAN_E_SHAPE, "%s: segments = %lld must be between 1 and min(255, ceil(L / %zu) = %lld)", who,
                    (long long)segments, tile, (long long)ntiles);
    int32_t nseg = 1, seg_tiles = (int32_t)ntiles;
    float2* pairs = nullptr;
    if (segments > 1) {
        if (pb.plain)
            return fail(FMSCAN_E_FLAGS, "%s: rows are cut without FMSCAN_FLAG_PLAIN only", who);
        seg_tiles = (int32_t)((ntiles + segments - 1) / segments);
        nseg = (int32_t)((ntiles + seg_tiles - 1) / seg_tiles);
        const __int128 need = (__int128)pb.rows * nseg * (int64_t)sizeof(float2);
        if (!workspace || ((uintptr_t)workspace & 7u) || (__int128)workspace_bytes < need)
            return fail(FMSCAN_E_WORKSPACE, "%s: %d segments need an 8-byte aligned workspace of %lld bytes (got %zu)",
                        who, nseg, (long long)need, workspace_bytes);
        if ((__int128)Bk * groups * nseg > (__int128)INT32_MAX)
            return fail(FMSCAN_E_SHAPE, "%s: B * split * ceil(D/%d) * segments must be < 2^31", who, group);
        const Range ws{"workspace", workspace, (int64_t)need};
        for (const Range& o : outs)
            if (overlap(ws, o)) return fail(FMSCAN_E_ALIAS, "%s: workspace overlaps %s", who, o.name);
        for (const Range& in : ins)
            if (overlap(ws, in)) return fail(FMSCAN_E_ALIAS, "%s: workspace overlaps %s", who, in.name);
        pairs = (float2*)workspace;
    }
    const unsigned grid = (unsigned)(Bk * groups * nseg);
    int rc = 0;
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        auto go = [&](auto jt, auto pt, auto lt, auto mode) {
            auto kern = fmscan::scan_backward_reduced_kernel<T, decltype(jt)::value, kReducedWaves, decltype(pt)::value,
                                                             decltype(lt)::value,  // lt: 0 plain call, 1 layer, 2 layer + recovered states
                                                             decltype(mode)::value>;  // 0 whole rows, 1 a segment, 2 the segments' step pairs
            static std::atomic<uint64_t> armed{0};
            if ((rc = raise_lds_limit((const void*)kern, armed, who)) != 0) return;
            kern<<<grid, 64 * kReducedWaves, lds, (hipStream_t)stream>>>(
                (const T*)gates, (const T*)out_grad, (const T*)first_prop_grad, (T*)token_grad,
                (const T*)cached_output, (const T*)input_tokens, gate_grad_partial, (const T*)h_init,
                (T*)initial_state_grad, coef_out, coef_self, (const T*)layer_out_grad,
                recover ? rms : nullptr, (int32_t)Mk, (int32_t)D, L, (int32_t)Mw, token_partial, (int32_t)split, nseg,
                seg_tiles, pairs);
        };
        auto with_plain = [&](auto lt) {
            if (nseg > 1) {  // (not plain: checked above)
                if (group == 8) {
                    go(IntTag<8>{}, BoolTag<false>{}, lt, IntTag<2>{});
                    if (!rc) go(IntTag<8>{}, BoolTag<false>{}, lt, IntTag<1>{});
                } else {
                    go(IntTag<4>{}, BoolTag<false>{}, lt, IntTag<2>{});
                    if (!rc) go(IntTag<4>{}, BoolTag<false>{}, lt, IntTag<1>{});
                }
                return;
            }
            if (group == 8) {
                if (pb.plain) go(IntTag<8>{}, BoolTag<true>{}, lt, IntTag<0>{});
                else go(IntTag<8>{}, BoolTag<false>{}, lt, IntTag<0>{});
            } else {
                if (pb.plain) go(IntTag<4>{}, BoolTag<true>{}, lt, IntTag<0>{});
                else go(IntTag<4>{}, BoolTag<false>{}, lt, IntTag<0>{});
            }
        };
        if (recover) with_plain(IntTag<2>{});
        else if (layer) with_plain(IntTag<1>{});
        else with_plain(IntTag<0>{});
    });
    if (rc) return rc;
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

int fmscan_backward_layer(const void* gates, const void* states_n, const float* coef_out, const float* coef_self,
                          const void* out_grad, const void* first_prop_grad, void* token_grad,
                          const void* cached_output, const float* rms, const void* input_tokens,
                          float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                          int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags, void* stream) {
    if (!coef_out) return fail(FMSCAN_E_NULL, "fmscan_backward_layer: coef_out must not be NULL");
    return backward_reduced("fmscan_backward_layer", gates, states_n, first_prop_grad, token_grad, cached_output,
                            input_tokens, gate_grad_partial, initial_state, initial_state_grad, coef_out, coef_self,
                            out_grad, rms, B, M, D, L, dtype, flags, stream);
}

int64_t fmscan_reduced_split(int64_t B, int64_t M, int64_t D) {
    if (B < 1 || M < 1 || D < 1) return 0;
    return reduced_split(B, M, D);
}

int fmscan_reduced_plan(int64_t B, int64_t M, int64_t D, int64_t L, int dtype, int64_t* split,
                               int64_t* segments) {
    if (!split || !segments) return fail(FMSCAN_E_NULL, "fmscan_reduced_plan: split and segments must not be NULL");
    *split = *segments = 0;
    if (B < 1 || M < 1 || D < 1 || L < 1)
        return fail(FMSCAN_E_SHAPE, "fmscan_reduced_plan: B, M, D, L must be >= 1");
    if (dtype != FMSCAN_DTYPE_F32 && dtype != FMSCAN_DTYPE_F16 && dtype != FMSCAN_DTYPE_BF16)
        return fail(FMSCAN_E_DTYPE, "fmscan_reduced_plan: unknown dtype %d", dtype);
    *split = reduced_split(B, M, D);
    *segments = 1;
    // From 64 (b, group of 4 d) pairs on, dealing the slots out reaches the 512 blocks without a second
    // read of the states, and was as fast or faster than any cut (bf16, us, split x segments:
    // (2,32,128,16384) 8x1 194, 1x8 184; (4,32,128,8192) 4x1 135, 1x8 180). Below, rows are cut first, into
    // up to 16 segments of four tiles or more, and the slots dealt out for what is still missing:
    // (1,32,128,32768) 8x1 287, 1x16 186; (1,16,64,65536) 4x1 514, 1x16 144, 2x16 121.
    const __int128 pairs = (__int128)B * ((D + 3) / 4);
    const int64_t tile = dtype == FMSCAN_DTYPE_F32 ? 256 : 512, ntiles = (L + tile - 1) / tile;
    const int64_t most = ntiles / 4 < 16 ? ntiles / 4 : 16;
    if (pairs >= 64 || most < 2) return 0;
    const int64_t want = (int64_t)((512 + pairs - 1) / pairs);
    *segments = want < most ? want : most;
    const int64_t rest = (int64_t)((512 + pairs * *segments - 1) / (pairs * *segments));
    *split = 1;
    for (int64_t s = 2; rest > 1 && s <= M / kReducedWaves; ++s) {
        if (M % s != 0) continue;
        *split = s;
        if (s >= rest) break;
    }
    return 0;
}

int fmscan_reduced_pays(int64_t B, int64_t M, int64_t D, int64_t L, int dtype) {
    if (B < 1 || M < 2 || D < 2 || L < 1) return 0;
    // Rows of at most 256 bytes leave three quarters of this kernel's lanes idle; fmscan_backward_reduced_packed
    // (where fmscan_reduced_packed_groups is not 0) and fmscan_backward put several such rows into a wave
    // (bf16, ms, this kernel against fmscan_backward and the two sums:
    // (512,32,128,64) 0.73 against 0.30, (256,32,128,128) 0.39 against 0.29, (128,32,128,256) 0.21 against 0.28).
    const int64_t row_bytes = L * (dtype == FMSCAN_DTYPE_F32 ? 4 : 2);
    if (row_bytes <= 256) return 0;
    int64_t split = 0, segments = 0;
    if (fmscan_reduced_plan(B, M, D, L, dtype, &split, &segments) != 0) return 0;
    // Measured against fmscan_backward followed by the two sums (bf16, ms): 512 blocks after split and cut
    // (2,32,128,16384) 0.24 against 0.27, (4,32,128,8192) 0.18 against 0.27; 256 blocks (1,32,128,32768)
    // 0.35 against 0.33; 64 blocks (1,16,64,65536) 0.56 against 0.16, (2,8,64,32768) 0.29 against 0.09.
    return (__int128)B * ((D + 3) / 4) * split * segments >= 256 ? 1 : 0;
}

int fmscan_backward_reduced_split(const void* gates, const void* out_grad, const void* first_prop_grad,
                                  float* token_grad_partial, const void* cached_output, const void* input_tokens,
                                  float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                                  int64_t B, int64_t M, int64_t D, int64_t L, int64_t split, int64_t segments,
                                  void* workspace, size_t workspace_bytes, int dtype, unsigned flags, void* stream) {
    return backward_reduced("fmscan_backward_reduced_split", gates, out_grad, first_prop_grad, nullptr, cached_output,
                            input_tokens, gate_grad_partial, initial_state, initial_state_grad, nullptr, nullptr,
                            nullptr, nullptr, B, M, D, L, dtype, flags, stream, token_grad_partial, split, true, segments,
                            workspace, workspace_bytes);
}

int fmscan_backward_layer_split(const void* gates, const void* states_n, const float* coef_out,
                                const float* coef_self, const void* out_grad, const void* first_prop_grad,
                                float* token_grad_partial, const void* cached_output, const float* rms,
                                const void* input_tokens, float* gate_grad_partial, const void* initial_state,
                                void* initial_state_grad, int64_t B, int64_t M, int64_t D, int64_t L, int64_t split,
                                int64_t segments, void* workspace, size_t workspace_bytes, int dtype, unsigned flags,
                                void* stream) {
    if (!coef_out) return fail(FMSCAN_E_NULL, "fmscan_backward_layer_split: coef_out must not be NULL");
    return backward_reduced("fmscan_backward_layer_split", gates, states_n, first_prop_grad, nullptr, cached_output,
                            input_tokens, gate_grad_partial, initial_state, initial_state_grad, coef_out, coef_self,
                            out_grad, rms, B, M, D, L, dtype, flags, stream, token_grad_partial, split, true, segments,
                            workspace, workspace_bytes);
}

// Rows of at most 256 bytes of whole 16-byte vectors, and enough (b, tile of rows) pairs to fill the GPU:
// the kernel that puts several rows into a wave and walks the slots (fmscan_packed.h). 0: not for this shape.
int64_t fmscan_reduced_packed_groups(int64_t B, int64_t M, int64_t D, int64_t L, int dtype) {
    if (B < 1 || M < 1 || D < 1 || L < 1) return 0;
    if (dtype != FMSCAN_DTYPE_F32 && dtype != FMSCAN_DTYPE_F16 && dtype != FMSCAN_DTYPE_BF16) return 0;
    const int64_t row_bytes = L * (dtype == FMSCAN_DTYPE_F32 ? 4 : 2);
    if (row_bytes > 256 || row_bytes % 16 != 0) return 0;
    int lanes_log2 = 0;
    while ((16 << lanes_log2) < row_bytes) ++lanes_log2;
    const int64_t per_tile = 64 >> lanes_log2;
    const int64_t groups = (D + per_tile - 1) / per_tile;
    // a wave per (b, tile): with few of them the routes that spread over rows are as fast or faster
    if ((__int128)B * groups < kPackedMinWaves) return 0;
    return groups;
}

// Shared by fmscan_backward_reduced_packed and fmscan_backward_layer_packed (coef_out != NULL: `out_grad`
// carries the normalised states and the gradient of the states is made in the kernel).
static int backward_reduced_packed(const char* who, const void* gates, const void* out_grad,
                                   const void* first_prop_grad, void* token_grad, const void* cached_output,
                                   const void* input_tokens, float* gate_grad_partial, const void* initial_state,
                                   void* initial_state_grad, const float* coef_out, const float* coef_self,
                                   const void* layer_out_grad, const float* rms, int64_t B, int64_t M, int64_t D,
                                   int64_t L, int dtype, unsigned flags, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags & FMSCAN_FLAG_PLAIN, &pb)) return rc;
    if (flags & ~FMSCAN_FLAG_PLAIN) return fail(FMSCAN_E_FLAGS, "%s: only FMSCAN_FLAG_PLAIN is understood here", who);
    const bool layer = coef_out != nullptr;
    const bool recover = layer && !cached_output;  // the states come back from states_n * rms
    if (layer && pb.plain) return fail(FMSCAN_E_FLAGS, "%s: the layer's scan has no FMSCAN_FLAG_PLAIN form", who);
    const int64_t groups = fmscan_reduced_packed_groups(B, M, D, L, dtype);
    if (groups < 1)
        return fail(FMSCAN_E_SHAPE, "%s: not for this shape (fmscan_reduced_packed_groups is 0): rows of whole "
                    "16-byte vectors up to 256 bytes, 512 (b, tile of rows) pairs or more", who);
    if (!gates || !out_grad || !token_grad || (!cached_output && !recover) || !gate_grad_partial)
        return fail(FMSCAN_E_NULL, "%s: gates, %s, token_grad, cached_output and gate_grad_partial must not "
                    "be NULL", who, layer ? "states_n" : "out_grad");
    if (recover && !rms)
        return fail(FMSCAN_E_NULL, "%s: without cached_output the states are states_n * rms: rms must not be NULL", who);
    if (layer && (!coef_self || !layer_out_grad))
        return fail(FMSCAN_E_NULL, "%s: coef_self and out_grad must not be NULL", who);
    if (!pb.plain && !input_tokens)
        return fail(FMSCAN_E_NULL, "%s: input_tokens must not be NULL without FMSCAN_FLAG_PLAIN", who);
    if (B > INT32_MAX || (__int128)B * groups > (__int128)INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: B * groups must be < 2^31", who);
    const int64_t full = pb.rows * L * pb.esize;
    const Range outs[] = {{"token_grad", token_grad, B * D * L * pb.esize},
                          {"gate_grad_partial", gate_grad_partial, B * M * groups * L * 4},
                          {"initial_state_grad", initial_state_grad, pb.rows * pb.esize}};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {layer ? "states_n" : "out_grad", out_grad, full},
                         {"first_prop_grad", first_prop_grad, pb.rows * pb.esize},
                         {"cached_output", cached_output, full},
                         {"input_tokens", pb.plain ? nullptr : input_tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize},
                         {"coef_out", coef_out, B * M * L * 4},
                         {"coef_self", layer ? coef_self : nullptr, B * M * L * 4},
                         {"out_grad", layer ? layer_out_grad : nullptr, B * D * L * pb.esize},
                         {"rms", recover ? rms : nullptr, B * M * L * 4}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, o.name, in.name);
    for (int i = 0; i < 3; ++i)
        for (int j = i + 1; j < 3; ++j)
            if (overlap(outs[i], outs[j])) return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, outs[i].name, outs[j].name);
    if (!(aligned16(gates) && aligned16(out_grad) && aligned16(token_grad) && aligned16(cached_output) &&
          (pb.plain || aligned16(input_tokens)) && aligned16(gate_grad_partial) && (!recover || aligned16(rms)) &&
          (!layer || (aligned16(coef_out) && aligned16(coef_self) && aligned16(layer_out_grad)))))
        return fail(FMSCAN_E_UNALIGNED, "%s: pointers must be multiples of 16 bytes", who);
    // NULL initial_state reproduces the reference kernel: h[-1] := first_prop_grad
    const void* h_init = initial_state ? initial_state : first_prop_grad;
    const int32_t lanes_log2 = packed_lanes_log2(pb);
    const unsigned grid = (unsigned)((B * groups + 3) / 4);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        auto go = [&](auto pt, auto lt) {
            fmscan::scan_backward_reduced_packed_kernel<T, decltype(pt)::value, decltype(lt)::value>
                <<<grid, 256, 0, (hipStream_t)stream>>>(
                    (const T*)gates, (const T*)out_grad, (const T*)first_prop_grad, (T*)token_grad,
                    (const T*)cached_output, (const T*)input_tokens, gate_grad_partial, (const T*)h_init,
                    (T*)initial_state_grad, coef_out, coef_self, (const T*)layer_out_grad, recover ? rms : nullptr,
                    (int32_t)B, (int32_t)M, (int32_t)D, (int32_t)L, lanes_log2, (int32_t)groups);
        };
        if (recover) go(BoolTag<false>{}, IntTag<2>{});
        else if (layer) go(BoolTag<false>{}, IntTag<1>{});
        else if (pb.plain) go(BoolTag<true>{}, IntTag<0>{});
        else go(BoolTag<false>{}, IntTag<0>{});
    });
    return launched(who);
}

int fmscan_backward_reduced_packed(const void* gates, const void* out_grad, const void* first_prop_grad,
                                   void* token_grad, const void* cached_output, const void* input_tokens,
                                   float* gate_grad_partial, const void* initial_state, void* initial_state_grad,
                                   int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                                   void* stream) {
    return backward_reduced_packed("fmscan_backward_reduced_packed", gates, out_grad, first_prop_grad, token_grad,
                                   cached_output, input_tokens, gate_grad_partial, initial_state, initial_state_grad,
                                   nullptr, nullptr, nullptr, nullptr, B, M, D, L, dtype, flags, stream);
}

int fmscan_backward_layer_packed(const void* gates, const void* states_n, const float* coef_out,
                                 const float* coef_self, const void* out_grad, const void* first_prop_grad,
                                 void* token_grad, const void* cached_output, const float* rms,
                                 const void* input_tokens, float* gate_grad_partial, const void* initial_state,
                                 void* initial_state_grad, int64_t B, int64_t M, int64_t D, int64_t L, int dtype,
                                 unsigned flags, void* stream) {
    if (!coef_out) return fail(FMSCAN_E_NULL, "fmscan_backward_layer_packed: coef_out must not be NULL");
    return backward_reduced_packed("fmscan_backward_layer_packed", gates, states_n, first_prop_grad, token_grad,
                                   cached_output, input_tokens, gate_grad_partial, initial_state, initial_state_grad,
                                   coef_out, coef_self, out_grad, rms, B, M, D, L, dtype, flags, stream);
}

int fmscan_sum_groups(const float* partial, int64_t G, void* out, int64_t rows, int64_t L, int dtype,
                      void* stream) {
    const char* who = "fmscan_sum_groups";
    if (!partial || !out) return fail(FMSCAN_E_NULL, "%s: partial and out must not be NULL", who);
    if (rows < 1 || L < 1 || G < 1 || G > INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: rows, G, L must be >= 1 and G fit 32 bits (got %lld, %lld, %lld)", who,
                    (long long)rows, (long long)G, (long long)L);
    if (dtype != FMSCAN_DTYPE_F32 && dtype != FMSCAN_DTYPE_F16 && dtype != FMSCAN_DTYPE_BF16)
        return fail(FMSCAN_E_DTYPE, "%s: unknown dtype %d", who, dtype);
    const int esize = dtype == FMSCAN_DTYPE_F32 ? 4 : 2;
    if ((__int128)rows * G * L * 4 > (__int128)INT64_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: rows * G * L is too large", who);
    if (overlap({"out", out, rows * L * esize}, {"partial", partial, rows * G * L * 4}))
        return fail(FMSCAN_E_ALIAS, "%s: out overlaps partial", who);
    const bool vec = L % 4 == 0 && aligned16(partial);
    const __int128 threads = (__int128)rows * (vec ? L / 4 : L);
    if ((threads + 255) / 256 > (__int128)INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: rows * L is too large for one launch", who);
    const unsigned grid = (unsigned)((threads + 255) / 256);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        if (vec)
            fmscan::sum_groups_kernel<T, 4><<<grid, 256, 0, (hipStream_t)stream>>>(partial, (T*)out, rows, (int32_t)G, L);
        else
            fmscan::sum_groups_kernel<T, 1><<<grid, 256, 0, (hipStream_t)stream>>>(partial, (T*)out, rows, (int32_t)G, L);
    });
    return launched(who);
}

}  // extern "C"
