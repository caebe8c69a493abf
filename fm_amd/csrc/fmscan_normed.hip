// fmscan_forward_normed, fmscan_forward_sumsq, fmscan_sumsq_finish: the layer's forward scan with the
// RMS norm, or the norm's sums of squares, inside.
// Contract: include/fmscan.h.
#include "fmscan_host.h"
#include "fmscan_normed.h"

using namespace fmscan::host;

namespace {

constexpr int64_t kNormedMaxD = 128;  // rows of one slot a block can hold in registers (16 waves x 8 rows)

template <typename T, int J, int NW>
void launch_normed(const void* g, const void* x, const void* h0, void* out, float* inv_rms, int64_t B, int64_t M,
                   int64_t D, int64_t L, float eps, hipStream_t s) {
    fmscan::scan_forward_normed_kernel<T, J, NW><<<(unsigned)(B * M), 64 * NW, 0, s>>>(
        (const T*)g, (const T*)x, (const T*)h0, (T*)out, inv_rms, (int32_t)M, (int32_t)D, L, eps, 1);
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

int fmscan_forward_normed(const void* gates, const void* tokens, const void* initial_state, void* states_n,
                          float* inv_rms, int64_t B, int64_t M, int64_t D, int64_t L, int dtype, float eps,
                          void* stream) {
    const char* who = "fmscan_forward_normed";
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
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        hipStream_t s = (hipStream_t)stream;
        if (D <= 32) launch_normed<T, 4, 8>(gates, tokens, initial_state, states_n, inv_rms, B, M, D, L, eps, s);
        else if (D <= 64) launch_normed<T, 4, 16>(gates, tokens, initial_state, states_n, inv_rms, B, M, D, L, eps, s);
        else launch_normed<T, 8, 16>(gates, tokens, initial_state, states_n, inv_rms, B, M, D, L, eps, s);
    });
    return launched(who);
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
                (int32_t)D, L, 0.0f, (int32_t)groups);
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
