// bench_stream_probe.so: a bare streaming kernel for bench.py (which builds it when it is not there),
// not part of the fm_amd package or of libfmscan_hip.so.
//
// It walks memory the way the scan kernels do (one 64-lane wave per row, 16 bytes per lane and step,
// four rows per block, the next steps' loads in flight while the current one is stored) but does no
// arithmetic beyond an exclusive-or of what it read: `reads` input tensors in, `writes` output tensors
// out. What it reaches is what this access pattern gets from the memory system with no arithmetic in
// the way and no tuning of how many waves a compute unit holds: a second reference point for the scan
// kernels besides the published peak, which no kernel reaches.
// It has no counterpart in the reference.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef unsigned u32x4 __attribute__((ext_vector_type(4)));

template <int R, int W, int DEPTH>
__global__ __launch_bounds__(256) void stream_rows_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out,
                                                          int64_t rows, int64_t steps, int64_t tensor_vecs) {
    const int64_t row = int64_t(blockIdx.x) * 4 + threadIdx.x / 64;
    if (row >= rows) return;
    const int lane = threadIdx.x % 64;
    const u32x4* src = in + row * steps * 64 + lane;
    u32x4* dst = out + row * steps * 64 + lane;
    u32x4 held[DEPTH][R];
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        const int64_t at = d < steps ? d : steps - 1;
#pragma unroll
        for (int r = 0; r < R; ++r) held[d][r] = __builtin_nontemporal_load(src + r * tensor_vecs + at * 64);
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
            for (int r = 0; r < R; ++r) held[d][r] = __builtin_nontemporal_load(src + r * tensor_vecs + ahead * 64);
#pragma unroll
            for (int w = 0; w < W; ++w) {
                u32x4 o = v;
                o.x += w;
                __builtin_nontemporal_store(o, dst + w * tensor_vecs + (t + d) * 64);
            }
        }
    }
}

template <int R, int W>
int launch(const void* in, void* out, int64_t rows, int64_t steps, int depth, hipStream_t stream) {
    const int64_t tensor_vecs = rows * steps * 64;
    const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
    if (depth == 4)
        stream_rows_kernel<R, W, 4><<<grid, block, 0, stream>>>((const u32x4*)in, (u32x4*)out, rows, steps, tensor_vecs);
    else
        stream_rows_kernel<R, W, 2><<<grid, block, 0, stream>>>((const u32x4*)in, (u32x4*)out, rows, steps, tensor_vecs);
    return (int)hipGetLastError();
}

}  // namespace

// `in` holds `reads` tensors and `out` `writes` tensors of rows * row_bytes bytes each, one after the
// other; row_bytes is a multiple of 1024 (one step of a wave), both pointers are 16-byte aligned.
// (reads, writes) is (2, 1), the forward scan's streams, or (3, 2), the backward scan's; depth 2 or 4.
// Returns 0, -1 for arguments outside that, or the hipError_t of the launch.
extern "C" int fmscan_probe_stream(const void* in, void* out, int64_t rows, int64_t row_bytes, int reads, int writes,
                                   int depth, void* stream) {
    if (!in || !out || rows <= 0 || rows > (int64_t(1) << 31) || row_bytes <= 0 || row_bytes % 1024 != 0 ||
        (depth != 2 && depth != 4) || (reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) % 16 != 0)
        return -1;
    const int64_t steps = row_bytes / 1024;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (reads == 2 && writes == 1) return launch<2, 1>(in, out, rows, steps, depth, s);
    if (reads == 3 && writes == 2) return launch<3, 2>(in, out, rows, steps, depth, s);
    return -1;
}
