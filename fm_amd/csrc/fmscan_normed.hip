// fmscan_forward_normed, fmscan_forward_sumsq, fmscan_sumsq_finish: the layer's forward scan with the
// RMS norm, or the norm's sums of squares, inside.
// Contract: include/fmscan.h.
#include "fmscan_host.h"
#include "fmscan_normed.h"
#include "fmscan_packed.h"

using namespace fmscan::host;

namespace {

constexpr int64_t kNormedMaxD = 128;  // rows of one slot a block can hold in registers (16 waves x 8 rows)

// How a slot's sequence is cut (nseg == 1: not at all).
struct Cut {
    int32_t nseg, seg_tiles;
    float2* pairs;
};

template <typename T, int J, int NW>
void launch_normed(const void* g, const void* x, const void* h0, void* out, float* inv_rms, int64_t B, int64_t M,
                   int64_t D, int64_t L, float eps, Cut cut, hipStream_t s) {
    if (cut.nseg > 1) {  // pass one: every segment of every row to its step pair, a wave per segment
        constexpr int R = 4, P = 3;
        const int64_t slots = B * M * D * cut.nseg;
        fmscan::scan_aggregate_kernel<T, R, P, false, true, false><<<(unsigned)((slots + R - 1) / R), 64 * R, 0, s>>>(
            (const T*)g, (const T*)x, cut.pairs, B * M * D, (int32_t)M, (int32_t)D, L, cut.nseg, (int64_t)cut.seg_tiles);
    }
    fmscan::scan_forward_normed_kernel<T, J, NW><<<(unsigned)(B * M * cut.nseg), 64 * NW, 0, s>>>(
        (const T*)g, (const T*)x, (const T*)h0, (T*)out, inv_rms, (int32_t)M, (int32_t)D, L, eps, 1, cut.nseg,
        cut.seg_tiles, cut.pairs);
}

// Segments for a slot's sequence so that B * M * segments blocks reach one per compute unit, none shorter
// than four tiles; 1 when the slots alone do, or the rows are too short to cut.
Cut plan_cut(int64_t B, int64_t M, int64_t L, int esize) {
    const int64_t tile = (16 / esize) * 64, ntiles = (L + tile - 1) / tile;
    Cut c{1, (int32_t)(ntiles < INT32_MAX ? ntiles : INT32_MAX), nullptr};
    const __int128 slots = (__int128)B * M;
    if (slots >= 256 || ntiles < 8 || ntiles >= INT32_MAX) return c;
    int64_t want = (int64_t)((256 + slots - 1) / slots);
    if (want > ntiles / 4) want = ntiles / 4;
    if (want > 64) want = 64;
    const int64_t seg_tiles = (ntiles + want - 1) / want;
    c.seg_tiles = (int32_t)seg_tiles;
    c.nseg = (int32_t)((ntiles + seg_tiles - 1) / seg_tiles);
    return c;
}

constexpr int kSumsqRows = 8, kSumsqWaves = 16;  // rows per wave and waves per block of the partial-sum form


}  // namespace

extern "C" {

int64_t fmscan_forward_normed_max_d(void) { return kNormedMaxD; }

int fmscan_forward_normed_pays(int64_t B, int64_t M, int64_t D) {
    if (B < 1 || M < 1 || D < 1) return 0;
    // A block of these kernels is a slot (or 128 rows of one) for the whole length of the sequence: below 64
    // blocks three quarters of the GPU stand idle, and fmscan_forward (a block per four rows, rows cut into
    // segments when there are few) followed by the norm's and the read-out's own kernels is faster although
    // it moves twice the bytes (measured: (B,L,M,D) = (1,32768,32,128) 0.43 against 0.28 ms, (1,65536,16,64)
    // 0.46 against 0.18; (2,16384,32,128) 0.28 either way; (4,8192,32,128) 0.20 against 0.27).
    return (__int128)B * M * ((D + kNormedMaxD - 1) / kNormedMaxD) >= 64 ? 1 : 0;
}

// fmscan_forward_normed (segments == 1) and fmscan_forward_normed_cut.
static int forward_normed(const char* who, const void* gates, const void* tokens, const void* initial_state,
                          void* states_n, float* inv_rms, int64_t B, int64_t M, int64_t D, int64_t L, int dtype,
                          float eps, int64_t segments, void* workspace, size_t workspace_bytes, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, 0, &pb)) return rc;
    if (!gates || !tokens || !states_n || !inv_rms)
        return fail(FMSCAN_E_NULL, "%s: gates, tokens, states_n and inv_rms must not be NULL", who);
    if (!(eps >= 0.0f)) return fail(FMSCAN_E_SHAPE, "%s: eps must be >= 0", who);
    if (D > kNormedMaxD)
        return fail(FMSCAN_E_SHAPE, "%s: D = %lld is beyond the %lld rows a block holds; use fmscan_forward, "
                    "fmscan_readout_inv_rms and fmscan_readout_forward", who, (long long)D, (long long)kNormedMaxD);
    if ((__int128)B * M > (__int128)INT32_MAX) return fail(FMSCAN_E_SHAPE, "%s: B * M must be < 2^31", who);
    const Range outs[] = {{"states_n", states_n, pb.rows * L * pb.esize}, {"inv_rms", inv_rms, B * M * L * 4}};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {"tokens", tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, o.name, in.name);
    if (overlap(outs[0], outs[1])) return fail(FMSCAN_E_ALIAS, "%s: states_n overlaps inv_rms", who);
    if ((L * pb.esize) % 16 != 0 || !aligned16(gates) || !aligned16(tokens) || !aligned16(states_n))
        return fail(FMSCAN_E_UNALIGNED, "%s: pointers and L * sizeof(element) must be multiples of 16 bytes", who);
    // the cut: as many segments as asked for, each a whole number of tiles, none empty
    const int64_t tile = (16 / pb.esize) * 64, ntiles = (L + tile - 1) / tile;
    if (segments < 1 || segments > 255 || segments > ntiles || ntiles >= INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: segments = %lld must be between 1 and min(255, ceil(L / %lld) = %lld)", who,
                    (long long)segments, (long long)tile, (long long)ntiles);
    Cut cut{1, (int32_t)ntiles, nullptr};
    if (segments > 1) {
        cut.seg_tiles = (int32_t)((ntiles + segments - 1) / segments);
        cut.nseg = (int32_t)((ntiles + cut.seg_tiles - 1) / cut.seg_tiles);
        const __int128 need = (__int128)pb.rows * cut.nseg * (int64_t)sizeof(float2);
        if (!workspace || ((uintptr_t)workspace & 7u) || (__int128)workspace_bytes < need)
            return fail(FMSCAN_E_WORKSPACE, "%s: %d segments need an 8-byte aligned workspace of %lld bytes (got %zu)",
                        who, cut.nseg, (long long)need, workspace_bytes);
        if ((__int128)B * M * cut.nseg > (__int128)INT32_MAX || (__int128)pb.rows * cut.nseg > ((__int128)1 << 33))
            return fail(FMSCAN_E_SHAPE, "%s: B * M * D * segments is too large for one launch", who);
        const Range ws{"workspace", workspace, (int64_t)need};
        for (const Range& r : outs)
            if (overlap(ws, r)) return fail(FMSCAN_E_ALIAS, "%s: workspace overlaps %s", who, r.name);
        for (const Range& r : ins)
            if (overlap(ws, r)) return fail(FMSCAN_E_ALIAS, "%s: workspace overlaps %s", who, r.name);
        cut.pairs = (float2*)workspace;
    }
    // Rows of at most 256 bytes, many slots: several rows to a wave, a wave per slot (fmscan_packed.h), where
    // a slot's rows fit the tiles a wave holds; the layer's forward at (B,L,M,D) = (512,64,32,128) bf16: 0.60 -> 0.25 ms.
    if (segments == 1 && L * pb.esize <= 256 && aligned16(inv_rms) && (__int128)B * M >= kPackedMinWaves) {
        const int32_t lanes_log2 = packed_lanes_log2(pb);
        const int64_t per_tile = 64 >> lanes_log2, tiles = (D + per_tile - 1) / per_tile;
        if (tiles <= 32) {
            const int64_t slots = B * M;
            with_dtype(dtype, [&](auto tt) {
                using T = typename decltype(tt)::type;
                auto go = [&](auto nt) {
                    fmscan::scan_forward_normed_packed_kernel<T, decltype(nt)::value>
                        <<<(unsigned)((slots + 3) / 4), 256, 0, (hipStream_t)stream>>>(
                            (const T*)gates, (const T*)tokens, (const T*)initial_state, (T*)states_n, inv_rms, slots,
                            (int32_t)M, (int32_t)D, (int32_t)L, eps, lanes_log2, (int32_t)tiles);
                };
                if (tiles <= 8) go(IntTag<8>{});
                else if (tiles <= 16) go(IntTag<16>{});
                else go(IntTag<32>{});
            });
            return launched(who);
        }
    }
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        hipStream_t s = (hipStream_t)stream;
        if (D <= 32) launch_normed<T, 4, 8>(gates, tokens, initial_state, states_n, inv_rms, B, M, D, L, eps, cut, s);
        else if (D <= 64) launch_normed<T, 4, 16>(gates, tokens, initial_state, states_n, inv_rms, B, M, D, L, eps, cut, s);
        else launch_normed<T, 8, 16>(gates, tokens, initial_state, states_n, inv_rms, B, M, D, L, eps, cut, s);
    });
    return launched(who);
}

}  // extern "C"

extern "C" {

int fmscan_forward_normed(const void* gates, const void* tokens, const void* initial_state, void* states_n,
                          float* inv_rms, int64_t B, int64_t M, int64_t D, int64_t L, int dtype, float eps,
                          void* stream) {
    return forward_normed("fmscan_forward_normed", gates, tokens, initial_state, states_n, inv_rms, B, M, D, L, dtype,
                          eps, 1, nullptr, 0, stream);
}

int64_t fmscan_forward_normed_segments(int64_t B, int64_t M, int64_t D, int64_t L, int dtype) {
    if (B < 1 || M < 1 || D < 1 || L < 1 || D > kNormedMaxD) return 0;
    if (dtype != FMSCAN_DTYPE_F32 && dtype != FMSCAN_DTYPE_F16 && dtype != FMSCAN_DTYPE_BF16) return 0;
    return plan_cut(B, M, L, dtype == FMSCAN_DTYPE_F32 ? 4 : 2).nseg;
}

int fmscan_forward_normed_cut(const void* gates, const void* tokens, const void* initial_state, void* states_n,
                              float* inv_rms, int64_t B, int64_t M, int64_t D, int64_t L, int dtype, float eps,
                              int64_t segments, void* workspace, size_t workspace_bytes, void* stream) {
    return forward_normed("fmscan_forward_normed_cut", gates, tokens, initial_state, states_n, inv_rms, B, M, D, L,
                          dtype, eps, segments, workspace, workspace_bytes, stream);
}

int64_t fmscan_sumsq_groups(int64_t D) {
    const int64_t per_block = (int64_t)kSumsqRows * kSumsqWaves;
    return D < 1 ? 0 : (D + per_block - 1) / per_block;
}

int fmscan_forward_sumsq(const void* gates, const void* tokens, const void* initial_state, void* states,
                         float* sumsq_partial, int64_t B, int64_t M, int64_t D, int64_t L, int dtype, void* stream) {
    const char* who = "fmscan_forward_sumsq";
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, 0, &pb)) return rc;
    if (!gates || !tokens || !states || !sumsq_partial)
        return fail(FMSCAN_E_NULL, "%s: gates, tokens, states and sumsq_partial must not be NULL", who);
    const int64_t groups = fmscan_sumsq_groups(D);
    if ((__int128)B * M * groups > (__int128)INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: B * M * ceil(D / %d) must be < 2^31", who, kSumsqRows * kSumsqWaves);
    const Range outs[] = {{"states", states, pb.rows * L * pb.esize},
                          {"sumsq_partial", sumsq_partial, B * M * groups * L * 4}};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {"tokens", tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize}};
    for (const Range& o : outs)
        for (const Range& in : ins)
            if (overlap(o, in)) return fail(FMSCAN_E_ALIAS, "%s: %s overlaps %s", who, o.name, in.name);
    if (overlap(outs[0], outs[1])) return fail(FMSCAN_E_ALIAS, "%s: states overlaps sumsq_partial", who);
    if ((L * pb.esize) % 16 != 0 || !aligned16(gates) || !aligned16(tokens) || !aligned16(states))
        return fail(FMSCAN_E_UNALIGNED, "%s: pointers and L * sizeof(element) must be multiples of 16 bytes", who);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        fmscan::scan_forward_normed_kernel<T, kSumsqRows, kSumsqWaves, false>
            <<<(unsigned)(B * M * groups), 64 * kSumsqWaves, 0, (hipStream_t)stream>>>(
                (const T*)gates, (const T*)tokens, (const T*)initial_state, (T*)states, sumsq_partial, (int32_t)M,
                (int32_t)D, L, 0.0f, (int32_t)groups, 1, 0, nullptr);
    });
    return launched(who);
}

int fmscan_sumsq_finish(const float* sumsq_partial, int64_t G, float* inv_rms, int64_t B, int64_t M, int64_t D,
                        int64_t L, float eps, void* stream) {
    const char* who = "fmscan_sumsq_finish";
    if (!sumsq_partial || !inv_rms) return fail(FMSCAN_E_NULL, "%s: sumsq_partial and inv_rms must not be NULL", who);
    if (B < 1 || M < 1 || D < 1 || L < 1 || G < 1 || G > INT32_MAX || D > INT32_MAX)
        return fail(FMSCAN_E_SHAPE, "%s: B, M, D, L, G must be >= 1 and G, D fit 32 bits", who);
    if (!(eps >= 0.0f)) return fail(FMSCAN_E_SHAPE, "%s: eps must be >= 0", who);
    const __int128 n = (__int128)B * M * L;
    if ((n + 255) / 256 > (__int128)INT32_MAX) return fail(FMSCAN_E_SHAPE, "%s: B * M * L must be < 2^39", who);
    if (overlap({"inv_rms", inv_rms, (int64_t)n * 4}, {"sumsq_partial", sumsq_partial, (int64_t)n * G * 4}))
        return fail(FMSCAN_E_ALIAS, "%s: inv_rms overlaps sumsq_partial", who);
    fmscan::sumsq_finish_kernel<<<(unsigned)((n + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        sumsq_partial, inv_rms, B * M, (int32_t)G, L, (int32_t)D, eps);
    return launched(who);
}

}  // extern "C"
