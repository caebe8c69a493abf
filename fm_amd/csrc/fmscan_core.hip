// libfmscan_hip.so, the pieces every entry point shares: the per-thread error text,
// the interface version, and the two size queries. Contract: include/fmscan.h.
#include "fmscan_host.h"

namespace fmscan {
namespace host {
thread_local char g_err[512] = "";
}  // namespace host
}  // namespace fmscan

using namespace fmscan::host;

#ifndef FMSCAN_BUILD_ID
#define FMSCAN_BUILD_ID "unknown"
#endif

extern "C" {

int fmscan_abi_version(void) { return FMSCAN_ABI_VERSION; }

const char* fmscan_build_id(void) { return FMSCAN_BUILD_ID; }

const char* fmscan_last_error(void) { return g_err; }

size_t fmscan_workspace_bytes(int64_t B, int64_t M, int64_t D, int64_t L, int dtype, unsigned flags) {
    Problem pb;
    if (parse(B, M, D, L, dtype, flags, &pb)) return 0;
    const Tuning t = choose(pb, false, true);  // the cut is the same in both directions
    if ((__int128)pb.rows * t.nseg > (__int128)INT32_MAX) return 0;
    return pairs_bytes(pb, t);
}

}  // extern "C"
