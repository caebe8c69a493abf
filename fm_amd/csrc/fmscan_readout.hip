// The layer around the scan: RMS norm and read-out with their gradients, the layer's small
// tensors, and the swap of the last two axes. Contract: include/fmscan.h.
#include "fmscan_host.h"
#include "fmscan_readout.h"
#include "fmscan_packed.h"

// Rows up to this many bytes take the packed forms of the read-out's two kernels, which have no sum across
// lanes and so no limit on the lanes of a group (bf16, us, general / packed, forward and backward:
// (256,32,128,192) 85 / 67 and 272 / 208, (256,32,128,256) 96 / 91 and 278 / 239, (128,32,128,512) 89 / 108 and
// 217 / 311).
#ifndef FMSCAN_READOUT_PACKED_BYTES
#define FMSCAN_READOUT_PACKED_BYTES 512
#endif

using namespace fmscan::host;

namespace {

// Waves of a block that share the D rows of a slot in rowdot_kernel: one where the (b, m, tile)
// triples alone fill the GPU (a wave then walks all D rows: no sum across waves, no short-lived
// blocks), more where they are few.
int rowdot_waves(int64_t triples, int64_t D) {
    int waves = 1;
    while (waves < 8 && triples * waves < 4096 && 2 * waves <= D) waves *= 2;
    return waves;
}
template <typename F>
void with_rowdot_waves(int waves, F&& f) {
    switch (waves) {
        case 1: f(std::integral_constant<int, 1>{}); break;
        case 2: f(std::integral_constant<int, 2>{}); break;
        case 4: f(std::integral_constant<int, 4>{}); break;
        default: f(std::integral_constant<int, 8>{}); break;
    }
}
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
constexpr unsigned kReadoutLds = (kMaxDynamicLds / kReadoutBlocksPerCU) & ~1023u;

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
            with_rowdot_waves(rowdot_waves(grid, D), [&](auto wt) {
                constexpr int WV = decltype(wt)::value;
                fmscan::rowdot_kernel<T, WV, fmscan::RowDot::kSumSq, false, decltype(vt)::value>
                    <<<grid, 64 * WV, 0, (hipStream_t)stream>>>((const T*)states, nullptr, nullptr, inv_rms, nullptr,
                                                                nullptr, nullptr, nullptr, nullptr, nullptr,
                                                                (int32_t)M, (int32_t)D, L, rs.tiles, eps);
            });
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
    // Rows of at most 256 bytes without the norm (the layer's read-out of normalised states), enough
    // (b, tile of rows) pairs: several rows to a wave (fmscan_packed.h)
    if (vec && !inv_rms && L * rs.esize <= FMSCAN_READOUT_PACKED_BYTES) {
        int32_t lanes_log2 = 0;
        while ((16 << lanes_log2) < L * rs.esize) ++lanes_log2;
        const int64_t per_tile = 64 >> lanes_log2, groups = (D + per_tile - 1) / per_tile;
        if ((__int128)B * groups >= kPackedMinWavesReadout && (__int128)B * groups <= (__int128)INT32_MAX && B <= INT32_MAX) {
            with_dtype(dtype, [&](auto tt) {
                using T = typename decltype(tt)::type;
                fmscan::readout_forward_packed_kernel<T><<<(unsigned)((B * groups + 3) / 4), 256, 0, (hipStream_t)stream>>>(
                    (const T*)states, (const T*)read, (T*)output, (int32_t)B, (int32_t)M, (int32_t)D, (int32_t)L,
                    lanes_log2, (int32_t)groups);
            });
            return launched("read-out (forward)");
        }
    }
    const dim3 grid((unsigned)(B * rs.tiles), (unsigned)((D + 4 * kReadoutRows - 1) / (4 * kReadoutRows)));
    int rc = 0;
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(inv_rms != nullptr, [&](auto nt) {
            with_bool(vec, [&](auto vt) {
                auto kern = fmscan::readout_forward_kernel<T, kReadoutRows, decltype(nt)::value, decltype(vt)::value>;
                static std::atomic<uint64_t> armed{0};
                if ((rc = raise_lds_limit((const void*)kern, armed, "fmscan_readout_forward")) != 0) return;
                kern<<<grid, 256, kReadoutLds, (hipStream_t)stream>>>(
                    (const T*)states, inv_rms, (const T*)read, (T*)states_out, (T*)output, (int32_t)M, (int32_t)D,
                    L, rs.tiles);
            });
        });
    });
    if (rc) return rc;
    return launched("read-out (forward)");
}

int fmscan_readout_dot(const void* states_n, const void* out_grad, const void* ext_grad, float* q, float* qe,
                       const float* inv_rms, const void* read, float* coef_out, float* coef_self, float* rms_out,
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
                          {"coef_out", coef_out, slot * 4}, {"coef_self", coef_self, slot * 4},
                          {"rms_out", rms_out, slot * 4}};
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
    // Rows of at most 256 bytes, many slots: several rows to a wave, a wave per slot
    if (vec && L * rs.esize <= 256 && (__int128)B * M >= kPackedMinWavesReadout && aligned16(q) && aligned16(qe) && aligned16(inv_rms) &&
        aligned16(read) && aligned16(coef_out) && aligned16(coef_self) && aligned16(rms_out)) {
        int32_t lanes_log2 = 0;
        while ((16 << lanes_log2) < L * rs.esize) ++lanes_log2;
        const int64_t per_tile = 64 >> lanes_log2, tiles = (D + per_tile - 1) / per_tile, slots = B * M;
        with_dtype(dtype, [&](auto tt) {
            using T = typename decltype(tt)::type;
            with_bool(ext_grad != nullptr, [&](auto et) {
                fmscan::readout_dot_packed_kernel<T, decltype(et)::value>
                    <<<(unsigned)((slots + 3) / 4), 256, 0, (hipStream_t)stream>>>(
                        (const T*)states_n, (const T*)out_grad, (const T*)ext_grad, q, qe, inv_rms, (const T*)read,
                        coef_out, coef_self, rms_out, slots, (int32_t)M, (int32_t)D, (int32_t)L, lanes_log2,
                        (int32_t)tiles);
            });
        });
        return launched("read-out (dot)");
    }
    const unsigned grid = (unsigned)(B * M * rs.tiles);
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(ext_grad != nullptr, [&](auto et) {
            with_bool(vec, [&](auto vt) {
                with_rowdot_waves(rowdot_waves(grid, D), [&](auto wt) {
                    constexpr int WV = decltype(wt)::value;
                    fmscan::rowdot_kernel<T, WV, fmscan::RowDot::kDot, decltype(et)::value, decltype(vt)::value>
                        <<<grid, 64 * WV, 0, (hipStream_t)stream>>>(
                            (const T*)states_n, (const T*)out_grad, (const T*)ext_grad, q, qe, inv_rms, (const T*)read,
                            coef_out, coef_self, rms_out, (int32_t)M, (int32_t)D, L, rs.tiles, 0.0f);
                });
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
    // Rows of at most 256 bytes, enough (b, tile of rows) pairs: several rows to a wave (fmscan_packed.h)
    if (vec && L * rs.esize <= FMSCAN_READOUT_PACKED_BYTES) {
        int32_t lanes_log2 = 0;
        while ((16 << lanes_log2) < L * rs.esize) ++lanes_log2;
        const int64_t per_tile = 64 >> lanes_log2, groups = (D + per_tile - 1) / per_tile;
        if ((__int128)B * groups >= kPackedMinWavesReadout && (__int128)B * groups <= (__int128)INT32_MAX && B <= INT32_MAX) {
            with_dtype(dtype, [&](auto tt) {
                using T = typename decltype(tt)::type;
                with_bool(norm, [&](auto nt) {
                    with_bool(ext_grad != nullptr, [&](auto et) {
                        fmscan::readout_backward_packed_kernel<T, decltype(nt)::value, decltype(et)::value>
                            <<<(unsigned)((B * groups + 3) / 4), 256, 0, (hipStream_t)stream>>>(
                                (const T*)states_n, inv_rms, (const T*)read, (const T*)out_grad, (const T*)ext_grad, q, qe,
                                (T*)state_grad, (int32_t)B, (int32_t)M, (int32_t)D, (int32_t)L, lanes_log2,
                                (int32_t)groups);
                    });
                });
            });
            return launched("read-out (backward)");
        }
    }
    const dim3 grid((unsigned)(B * rs.tiles), (unsigned)((D + 4 * kReadoutRows - 1) / (4 * kReadoutRows)));
    int rc = 0;
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(norm, [&](auto nt) {
            with_bool(ext_grad != nullptr, [&](auto et) {
                with_bool(vec, [&](auto vt) {
                    auto kern = fmscan::readout_backward_kernel<T, kReadoutRows, decltype(nt)::value,
                                                                decltype(et)::value, decltype(vt)::value>;
                    static std::atomic<uint64_t> armed{0};
                    if ((rc = raise_lds_limit((const void*)kern, armed, "fmscan_readout_backward")) != 0) return;
                    kern<<<grid, 256, kReadoutLds, (hipStream_t)stream>>>(
                        (const T*)states_n, inv_rms, (const T*)read, (const T*)out_grad, (const T*)ext_grad, q, qe,
                        (T*)state_grad, (int32_t)M, (int32_t)D, L, rs.tiles);
                });
            });
        });
    });
    if (rc) return rc;
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
    if (element_size == 2 && R % 8 == 0 && C % 8 == 0 && aligned16(src) && aligned16(dst))
        fmscan::swap_last_two_wide_kernel<<<grid, 256, 0, (hipStream_t)stream>>>(
            (const uint16_t*)src, (uint16_t*)dst, R, C, (int32_t)tiles_c, (int32_t)tiles_r);
    else if (element_size == 2 && R % 2 == 0 && C % 2 == 0 && ((uintptr_t)src & 3u) == 0 && ((uintptr_t)dst & 3u) == 0)
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
