"""Builds libfmscan_hip.so (gfx950) from fm_amd/csrc with hipcc.

The reference JIT-compiles its CUDA source at import time
(fm/scan/fm_scan.py:18-33); here the library is built ahead of time, in-tree,
and loaded with ctypes (`fm_amd._lib`).

    python -m fm_amd.build

The translation units are compiled side by side and linked into one shared
library. The library carries a hash of the sources it was built from
(`fmscan_build_id()`), so that a library older than its sources is noticed
when it is loaded.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
UNITS = ["fmscan_core.hip", "fmscan_forward.hip", "fmscan_backward.hip", "fmscan_reduced.hip",
         "fmscan_readout.hip", "fmscan_normed.hip"]
HEADERS = ["fmscan_host.h", "fmscan_device.h", "fmscan_kernels.h", "fmscan_reduced.h", "fmscan_readout.h",
           "fmscan_normed.h", "fmscan_packed.h"]
DEPS = [CSRC / n for n in UNITS + HEADERS] + [PKG.parent / "include" / "fmscan.h"]
LIB = PKG / "lib" / "libfmscan_hip.so"
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep hipcc from forming packed fp32 VALU ops out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin)")


def source_id() -> str:
    """Hash of everything the library is built from (sources, headers, flags)."""
    h = hashlib.sha256(" ".join(HIPCC_FLAGS).encode())
    for d in DEPS:
        h.update(d.name.encode())
        h.update(d.read_bytes())
    return h.hexdigest()[:16]


def _run(cmd, verbose):
    if verbose:
        print("[fm_amd.build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the device-only feature flag; that warning is noise
    noise = ("is not a recognized feature for this target", "1 warning generated", "warnings generated")
    err = "\n".join(l for l in res.stderr.splitlines() if not any(n in l for n in noise))
    if res.returncode != 0:
        raise RuntimeError("hipcc failed (%d): %s\n%s" % (res.returncode, " ".join(cmd), err))
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = True, extra_flags=(), jobs: int | None = None) -> Path:
    """Compiles the library unconditionally and returns its path."""
    LIB.parent.mkdir(parents=True, exist_ok=True)
    hipcc = hipcc_path()
    build_id = source_id()
    jobs = jobs or min(len(UNITS), int(os.environ.get("MAX_JOBS", "0")) or os.cpu_count() or 1)
    with tempfile.TemporaryDirectory(prefix="fmscan_build_") as tmpdir:
        objs = [str(Path(tmpdir) / (Path(u).stem + ".o")) for u in UNITS]
        cmds = [[hipcc, *HIPCC_FLAGS, *extra_flags, f'-DFMSCAN_BUILD_ID="{build_id}"', "-c", str(CSRC / u), "-o", o]
                for u, o in zip(UNITS, objs)]
        with ThreadPoolExecutor(max_workers=jobs) as pool:
            list(pool.map(lambda c: _run(c, verbose), cmds))
        tmp = LIB.with_suffix(".so.tmp%d" % os.getpid())
        try:
            _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *objs], verbose)
            os.replace(tmp, LIB)
        finally:
            tmp.unlink(missing_ok=True)
    return LIB


if __name__ == "__main__":
    print(build())
