"""Builds libfmscan_hip.so (gfx950) from fm_amd/csrc with hipcc.

The reference JIT-compiles its CUDA source at import time
(fm/scan/fm_scan.py:18-33); here the library is built ahead of time, in-tree,
and loaded with ctypes (`fm_amd._lib`).

    python -m fm_amd.build
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
SRC = PKG / "csrc" / "fmscan_api.hip"
DEPS = [SRC, PKG / "csrc" / "fmscan_kernels.h", PKG / "csrc" / "fmscan_device.h",
        PKG.parent / "include" / "fmscan.h"]
LIB = PKG / "lib" / "libfmscan_hip.so"

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    # keep hipcc from forming packed fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def is_stale() -> bool:
    if not LIB.exists():
        return True
    t = LIB.stat().st_mtime
    return any(d.stat().st_mtime > t for d in DEPS)


def build(verbose: bool = True, extra_flags=()) -> Path:
    """Compiles the library unconditionally and returns its path."""
    LIB.parent.mkdir(parents=True, exist_ok=True)
    tmp = LIB.with_suffix(".so.tmp%d" % os.getpid())
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, "-o", str(tmp), str(SRC)]
    if verbose:
        print("[fm_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only feature flag; that warning is noise
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        tmp.unlink(missing_ok=True)
        raise RuntimeError("hipcc failed (%d):\n%s" % (res.returncode, err))
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(tmp, LIB)
    return LIB


if __name__ == "__main__":
    print(build())
