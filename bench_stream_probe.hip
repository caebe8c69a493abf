// bench_stream_probe.so: a bare streaming kernel for bench.py (which builds it when it is not there),
// not part of the fm_amd package or of libfmscan_hip.so.
//
// It walks memory the way the scan kernels do (rows side by side, 1, 2, 4 or 8 waves on a row, 16 bytes per
// lane and step, the next steps' loads in flight while the current one is stored, non-temporal, an optional
// cap on the blocks a compute unit holds) but does no arithmetic beyond an exclusive-or of what it read:
// `reads` input tensors in, `writes` output tensors out. Swept over those knobs, the best it reaches is what
// this access pattern gets from the memory system with no arithmetic in the way: a second reference point
// for the scan kernels besides the published peak, which no kernel reaches.
// It has no counterpart in the reference.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

// WV waves side by side on a row (a block is one row; with WV == 1 four rows): a step of the block covers
// WV KiB contiguous per tensor. `steps` = row_bytes / (1024 * WV).
template <int R, int W, int DEPTH, int WV>
__global__ __launch_bounds__(WV == 1 ? 256 : 64 * WV) void stream_rows_kernel(const u32x4* __restrict__ in,
                                                                            u32x4* __restrict__ out, int64_t rows,
                                                                            int64_t steps, int64_t tensor_vecs) {
    constexpr int ROWS_PER_BLOCK = WV == 1 ? 4 : 1;
    const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
    const int64_t row = int64_t(blockIdx.x) * ROWS_PER_BLOCK + (WV == 1 ? wave : 0);
    if (row >= rows) return;
    const int w = WV == 1 ? 0 : wave;
    const u32x4* src = in + row * steps * 64 * WV + w * 64 + lane;
    u32x4* dst = out + row * steps * 64 * WV + w * 64 + lane;
    u32x4 held[DEPTH][R];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        const int64_t at = d < steps ? d : steps - 1;
#pragma unroll
        for (int r = 0; r < R; ++r) held[d][r] = __builtin_nontemporal_load(src + r * tensor_vecs + at * 64 * WV);
    }
    for (int64_t t = 0; t < steps; t += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            if (t + d >= steps) break;
            u32x4 v = held[d][0];
#pragma unroll
            for (int r = 1; r < R; ++r) v ^= held[d][r];
            int64_t ahead = t + d + DEPTH;  // clamped: the last steps load the row's last vectors again
            if (ahead >= steps) ahead = steps - 1;
#pragma unroll
            for (int r = 0; r < R; ++r) held[d][r] = __builtin_nontemporal_load(src + r * tensor_vecs + ahead * 64 * WV);
#pragma unroll
            for (int ww = 0; ww < W; ++ww) {
                u32x4 o = v;
                o.x += ww;
                __builtin_nontemporal_store(o, dst + ww * tensor_vecs + (t + d) * 64 * WV);
            }
        }
    }
}

constexpr unsigned kLdsForCaps = 158u * 1024u;  // what the cap on resident blocks divides (the scan kernels' own way)

template <int R, int W, int DEPTH, int WV>
int launch_variant(const void* in, void* out, int64_t rows, int64_t row_bytes, int blocks_per_cu, hipStream_t stream) {
    auto kern = stream_rows_kernel<R, W, DEPTH, WV>;
    unsigned lds = 0;
    if (blocks_per_cu > 0) {  // an untouched slice of LDS per block: at most that many blocks fit a compute unit
        const hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 (int)kLdsForCaps);
        if (e != hipSuccess) return (int)e;
        lds = (kLdsForCaps / (unsigned)blocks_per_cu) & ~1023u;
    }
    constexpr int ROWS_PER_BLOCK = WV == 1 ? 4 : 1;
    const int64_t steps = row_bytes / (1024 * WV);
    const int64_t tensor_vecs = rows * row_bytes / 16;
    const dim3 grid((unsigned)((rows + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK)), block(WV == 1 ? 256 : 64 * WV);
    kern<<<grid, block, lds, stream>>>((const u32x4*)in, (u32x4*)out, rows, steps, tensor_vecs);
    return (int)hipGetLastError();
}

template <int R, int W>
int launch(const void* in, void* out, int64_t rows, int64_t row_bytes, int depth, int waves, int blocks_per_cu,
           hipStream_t s) {
#define FMSCAN_PROBE_CASE(D, WV) \
    if (depth == D && waves == WV) return launch_variant<R, W, D, WV>(in, out, rows, row_bytes, blocks_per_cu, s);
    FMSCAN_PROBE_CASE(2, 1) FMSCAN_PROBE_CASE(4, 1) FMSCAN_PROBE_CASE(2, 2) FMSCAN_PROBE_CASE(4, 2)
    FMSCAN_PROBE_CASE(2, 4) FMSCAN_PROBE_CASE(4, 4) FMSCAN_PROBE_CASE(2, 8) FMSCAN_PROBE_CASE(4, 8)
#undef FMSCAN_PROBE_CASE
    return -1;
}

}  // namespace

// `in` holds `reads` tensors and `out` `writes` tensors of rows * row_bytes bytes each, one after the
// other; both pointers are 16-byte aligned. (reads, writes) is (2, 1), the forward scan's streams, or (3, 2),
// the backward scan's; depth 2 or 4; waves_per_row 1, 2, 4 or 8 (row_bytes a multiple of 1024 * waves_per_row);
// blocks_per_cu 0 (no cap) to 15: the same three knobs the scan kernels have.
// Returns 0, -1 for arguments outside that, or the hipError_t of the launch.
extern "C" int fmscan_probe_stream(const void* in, void* out, int64_t rows, int64_t row_bytes, int reads, int writes,
                                   int depth, int waves_per_row, int blocks_per_cu, void* stream) {
    if (!in || !out || rows <= 0 || rows > (int64_t(1) << 31) || row_bytes <= 0 || (depth != 2 && depth != 4) ||
        (waves_per_row != 1 && waves_per_row != 2 && waves_per_row != 4 && waves_per_row != 8) ||
        row_bytes % (1024 * waves_per_row) != 0 || blocks_per_cu < 0 || blocks_per_cu > 15 ||
        (reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) % 16 != 0)
        return -1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (reads == 2 && writes == 1) return launch<2, 1>(in, out, rows, row_bytes, depth, waves_per_row, blocks_per_cu, s);
    if (reads == 3 && writes == 2) return launch<3, 2>(in, out, rows, row_bytes, depth, waves_per_row, blocks_per_cu, s);
    return -1;
}
