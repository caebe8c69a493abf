// fmscan_forward and fmscan_forward_static: argument checks, choice of kernel variant, launch.
// Contract: include/fmscan.h.
#include "fmscan_host.h"
#include "fmscan_kernels.h"
#include "fmscan_packed.h"

using namespace fmscan::host;

// The segment pairs of fmscan_forward_static.
// Device memory that belongs to the library: every GPU the library runs on holds its own
// copy of this array (64 KiB) from the first call on it until the process ends. Host code
// must not use the array's name as an address; it asks the runtime for the array's address
// on the current device and hands that to the kernels like any other workspace.
static __device__ __align__(256) float2 scratch[FMSCAN_STATIC_PAIRS];

namespace {

template <typename T, int W, int R, int P, bool PLAIN, bool VEC, bool FOLD>
int launch_fwd(const Problem& pb, const Tuning& t, const void* g, const void* x, const void* h0,
               void* out, const float2* pairs, hipStream_t s) {
    auto kern = fmscan::scan_forward_kernel<T, W, R, P, PLAIN, VEC, FOLD>;
    static std::atomic<uint64_t> armed{0};
    if (int rc = raise_lds_limit((const void*)kern, armed, "fmscan_forward")) return rc;
    const unsigned blocks = (unsigned)((pb.rows * t.nseg + R - 1) / R);
    kern<<<blocks, 64 * W * R, lds_share(t.blocks_per_cu), s>>>((const T*)g, (const T*)x, (const T*)h0, (T*)out,
                                                                pb.rows, (int32_t)pb.M, (int32_t)pb.D, pb.L,
                                                                t.nseg, t.seg_tiles, pairs);
    return 0;
}

// Pass one of a segmented scan: one wave per segment, four segments per block.
void launch_aggregate(int dtype, const Problem& pb, const Tuning& t, bool vec, const void* g,
                      const void* other, float2* pairs, hipStream_t s) {
    with_dtype(dtype, [&](auto tt) {
        using T = typename decltype(tt)::type;
        with_bool(pb.plain, [&](auto pt) {
            with_bool(vec, [&](auto vt) {
                constexpr int R = 4, P = 3;
                auto kern = fmscan::scan_aggregate_kernel<T, R, P, decltype(pt)::value, decltype(vt)::value, false>;
                const unsigned blocks = (unsigned)((pb.rows * t.nseg + R - 1) / R);
                kern<<<blocks, 64 * R, 0, s>>>((const T*)g, (const T*)other, pairs, pb.rows, (int32_t)pb.M,
                                              (int32_t)pb.D, pb.L, t.nseg, t.seg_tiles);
            });
        });
    });
}

// ---- the segment pairs of fmscan_forward_static (the array itself is at the top of the file)
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Address of `scratch` on the device that is current, looked up once per device.
int static_pairs(void** ptr) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess)
        return fail((int)e, "fmscan_forward_static: hipGetDevice failed: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices)
        return fail(FMSCAN_E_SHAPE, "fmscan_forward_static: device %d is beyond the %d this call keeps a "
                    "workspace for", dev, kMaxDevices);
    void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || !p) {
            (void)hipGetLastError();
            return fail(e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol,
                        "fmscan_forward_static: cannot locate the library's workspace on device %d: %s", dev,
                        hipGetErrorString(e));
        }
        g_scratch_ptr[dev].store(p, std::memory_order_release);  // every thread finds the same address
    }
    *ptr = p;
    return 0;
}

// Both forward entry points: `who` names the one that was called.
int forward(const char* who, const void* gates, const void* tokens, const void* initial_state, void* out,
            int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
            void* workspace, size_t workspace_bytes, void* stream) {
    Problem pb;
    if (int rc = parse(B, M, D, L, dtype, flags, &pb)) return rc;
    if (!gates || !tokens || !out)
        return fail(FMSCAN_E_NULL, "%s: gates, tokens and out must not be NULL", who);
    const Range o{"out", out, pb.rows * L * pb.esize};
    const Range ins[] = {{"gates", gates, B * M * L * pb.esize},
                         {"tokens", tokens, B * D * L * pb.esize},
                         {"initial_state", initial_state, pb.rows * pb.esize},
                         {"workspace", workspace, (int64_t)workspace_bytes}};
    for (const Range& in : ins)
        if (overlap(o, in))
            return fail(FMSCAN_E_ALIAS, "%s: out overlaps %s", who, in.name);

    const bool vec = (L * pb.esize) % 16 == 0 && aligned16(gates) && aligned16(tokens) && aligned16(out);
    const bool fold = M == 1 && D == 1;
    if (packs_rows(pb, vec, false)) {  // short rows: several per wave
        const int32_t lanes_log2 = packed_lanes_log2(pb);
        with_dtype(dtype, [&](auto tt) {
            using T = typename decltype(tt)::type;
            with_bool(pb.plain, [&](auto pt) {
                with_bool(vec, [&](auto vt) { with_bool(fold, [&](auto ft) {
                    fmscan::scan_forward_packed_kernel<T, decltype(pt)::value, decltype(vt)::value, decltype(ft)::value>
                        <<<packed_blocks(pb, lanes_log2), 256, 0, (hipStream_t)stream>>>(
                            (const T*)gates, (const T*)tokens, (const T*)initial_state, (T*)out, pb.rows,
                            (int32_t)pb.M, (int32_t)pb.D, (int32_t)pb.L, lanes_log2);
                }); });
            });
        });
        return launched("forward");
    }
    Tuning tune;
    if (int rc = settle(pb, false, workspace, workspace_bytes, who, &tune)) return rc;
    float2* pairs = tune.nseg > 1 ? (float2*)workspace : nullptr;
    if (pairs) {
        launch_aggregate(dtype, pb, tune, vec, gates, tokens, pairs, (hipStream_t)stream);
        if (int rc = launched("forward (segment pass)")) return rc;
    }
    int rc = 0;
    dispatch<false>(dtype, tune, pb.plain, vec, fold, [&](auto tt, auto wt, auto rt, auto dt, auto pt, auto vt, auto ft) {
        using T = typename decltype(tt)::type;
        rc = launch_fwd<T, decltype(wt)::value, decltype(rt)::value, decltype(dt)::value, decltype(pt)::value,
                   decltype(vt)::value, decltype(ft)::value>(pb, tune, gates, tokens, initial_state, out,
                                                             pairs, (hipStream_t)stream);
    });
    if (rc) return rc;
    return launched("forward");
}

}  // namespace

extern "C" {

int fmscan_forward(const void* gates, const void* tokens, const void* initial_state, void* out,
                   int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                   void* workspace, size_t workspace_bytes, void* stream) {
    return forward("fmscan_forward", gates, tokens, initial_state, out, B, M, D, L, dtype, flags, workspace,
                   workspace_bytes, stream);
}

int fmscan_forward_static(const void* gates, const void* tokens, const void* initial_state, void* out,
                          int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags,
                          void* stream) {
    void* ws = nullptr;
    if (int rc = static_pairs(&ws)) return rc;
    return forward("fmscan_forward_static", gates, tokens, initial_state, out, B, M, D, L, dtype, flags, ws,
                   sizeof(float2) * FMSCAN_STATIC_PAIRS, stream);
}

}  // extern "C"
