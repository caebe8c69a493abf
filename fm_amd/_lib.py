"""ctypes binding of libfmscan_hip.so (interface: include/fmscan.h).

There is no other implementation behind these calls: if the library cannot
be loaded the import of `fm_amd.scan.fm_scan` fails, and tensors that are not
on a GPU are rejected.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint, c_void_p

from . import build as _build

ABI_VERSION = 7

DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
FLAG_PLAIN = 0x1
FLAG_WAVES_SHIFT = 8
FLAG_BLOCKS_SHIFT = 12
FLAG_DEPTH_SHIFT = 16
FLAG_SEGMENTS_SHIFT = 20

_lib = None


def _open_current() -> ctypes.CDLL:
    """The built library, rebuilt first when it is missing or older than its sources (its
    build id is a hash of them). Without a compiler an outdated library is an error."""
    try:
        want = _build.source_id()
    except OSError:
        want = None  # the sources are not there (a deployed library): nothing to compare with
    for attempt in (0, 1):
        if _build.LIB.exists():
            lib = ctypes.CDLL(str(_build.LIB))
            try:
                lib.fmscan_build_id.restype = c_char_p
                lib.fmscan_build_id.argtypes = []
                have = lib.fmscan_build_id().decode()
            except AttributeError:
                have = "none"
            if want is None or have == want:
                return lib
            import _ctypes

            _ctypes.dlclose(lib._handle)  # or loading the same path again would return this one
            del lib
            why = f"libfmscan_hip.so was built from other sources (build id {have}, sources {want})"
        else:
            why = "libfmscan_hip.so has not been built"
        if attempt:
            break
        try:
            _build.hipcc_path()
        except RuntimeError:
            raise RuntimeError(why + " and hipcc is not available; build it with `python -m fm_amd.build`")
        # dlopen keeps a loaded file by path: build to the same path, then load it afresh
        _build.build(verbose=False)
    raise RuntimeError(why + " after a rebuild; run `python -m fm_amd.build` and check its output")


def load() -> ctypes.CDLL:
    """Loads the built library (see _open_current) and declares its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    lib = _open_current()
    lib.fmscan_abi_version.restype = c_int
    lib.fmscan_abi_version.argtypes = []
    lib.fmscan_last_error.restype = c_char_p
    lib.fmscan_last_error.argtypes = []
    lib.fmscan_forward.restype = c_int
    lib.fmscan_workspace_bytes.restype = c_size_t
    lib.fmscan_workspace_bytes.argtypes = [c_int64, c_int64, c_int64, c_int64, c_int, c_uint]
    lib.fmscan_forward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p,
                                   c_int64, c_int64, c_int64, c_int64, c_int, c_uint,
                                   c_void_p, c_size_t, c_void_p]
    lib.fmscan_forward_static.restype = c_int
    lib.fmscan_forward_static.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_int64, c_int64, c_int64, c_int64, c_int, c_uint, c_void_p]
    lib.fmscan_backward.restype = c_int
    lib.fmscan_backward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p,
                                    c_int64, c_int64, c_int64, c_int64, c_int, c_uint,
                                    c_void_p, c_size_t, c_void_p]
    lib.fmscan_reduced_groups.restype = c_int64
    lib.fmscan_reduced_groups.argtypes = [c_int64, c_int64]
    lib.fmscan_sum_groups.restype = c_int
    lib.fmscan_sum_groups.argtypes = [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int, c_void_p]
    lib.fmscan_backward_reduced.restype = c_int
    lib.fmscan_backward_reduced.argtypes = [c_void_p] * 9 + [c_int64] * 4 + [c_int, c_uint, c_void_p]
    lib.fmscan_backward_layer.restype = c_int
    lib.fmscan_backward_layer.argtypes = [c_void_p] * 13 + [c_int64] * 4 + [c_int, c_uint, c_void_p]
    lib.fmscan_reduced_split.restype = c_int64
    lib.fmscan_reduced_split.argtypes = [c_int64] * 3
    lib.fmscan_reduced_pays.restype = c_int
    lib.fmscan_reduced_pays.argtypes = [c_int64] * 4 + [c_int]
    lib.fmscan_reduced_packed_groups.restype = c_int64
    lib.fmscan_reduced_packed_groups.argtypes = [c_int64] * 4 + [c_int]
    lib.fmscan_backward_reduced_packed.restype = c_int
    lib.fmscan_backward_reduced_packed.argtypes = [c_void_p] * 9 + [c_int64] * 4 + [c_int, c_uint, c_void_p]
    lib.fmscan_backward_layer_packed.restype = c_int
    lib.fmscan_backward_layer_packed.argtypes = [c_void_p] * 13 + [c_int64] * 4 + [c_int, c_uint, c_void_p]
    lib.fmscan_backward_reduced_split.restype = c_int
    lib.fmscan_backward_reduced_split.argtypes = ([c_void_p] * 9 + [c_int64] * 6 + [c_void_p, c_size_t]
                                                  + [c_int, c_uint, c_void_p])
    lib.fmscan_backward_layer_split.restype = c_int
    lib.fmscan_backward_layer_split.argtypes = ([c_void_p] * 13 + [c_int64] * 6 + [c_void_p, c_size_t]
                                                + [c_int, c_uint, c_void_p])
    lib.fmscan_reduced_plan.restype = c_int
    lib.fmscan_reduced_plan.argtypes = [c_int64] * 4 + [c_int, ctypes.POINTER(c_int64), ctypes.POINTER(c_int64)]
    dims = [c_int64] * 4
    lib.fmscan_readout_inv_rms.restype = c_int
    lib.fmscan_readout_inv_rms.argtypes = [c_void_p] * 2 + dims + [c_int, c_float, c_void_p]
    lib.fmscan_forward_normed_max_d.restype = c_int64
    lib.fmscan_forward_normed_max_d.argtypes = []
    lib.fmscan_forward_normed_pays.restype = c_int
    lib.fmscan_forward_normed_pays.argtypes = [c_int64] * 3
    lib.fmscan_forward_normed_segments.restype = c_int64
    lib.fmscan_forward_normed_segments.argtypes = [c_int64] * 4 + [c_int]
    lib.fmscan_forward_normed_cut.restype = c_int
    lib.fmscan_forward_normed_cut.argtypes = [c_void_p] * 5 + dims + [c_int, c_float, c_int64, c_void_p, c_size_t,
                                              c_void_p]
    lib.fmscan_forward_normed.restype = c_int
    lib.fmscan_forward_normed.argtypes = [c_void_p] * 5 + dims + [c_int, c_float, c_void_p]
    lib.fmscan_sumsq_groups.restype = c_int64
    lib.fmscan_sumsq_groups.argtypes = [c_int64]
    lib.fmscan_forward_sumsq.restype = c_int
    lib.fmscan_forward_sumsq.argtypes = [c_void_p] * 5 + dims + [c_int, c_void_p]
    lib.fmscan_sumsq_finish.restype = c_int
    lib.fmscan_sumsq_finish.argtypes = [c_void_p, c_int64, c_void_p] + dims + [c_float, c_void_p]
    lib.fmscan_readout_forward.restype = c_int
    lib.fmscan_readout_forward.argtypes = [c_void_p] * 5 + dims + [c_int, c_void_p]
    lib.fmscan_readout_dot.restype = c_int
    lib.fmscan_readout_dot.argtypes = [c_void_p] * 10 + dims + [c_int, c_void_p]
    lib.fmscan_layer_prepare.restype = c_int
    lib.fmscan_layer_prepare.argtypes = [c_void_p] * 5 + [c_int64] * 3 + [c_int, c_void_p]
    lib.fmscan_layer_finish.restype = c_int
    lib.fmscan_layer_finish.argtypes = [c_void_p, c_int64] + [c_void_p] * 7 + [c_int64] * 3 + [c_int, c_void_p]
    lib.fmscan_readout_backward.restype = c_int
    lib.fmscan_readout_backward.argtypes = [c_void_p] * 8 + dims + [c_int, c_void_p]
    lib.fmscan_swap_last_two.restype = c_int
    lib.fmscan_swap_last_two.argtypes = [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p]
    got = lib.fmscan_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError(f"libfmscan_hip.so has ABI version {got}, this package needs {ABI_VERSION}; "
                           "rebuild with `python -m fm_amd.build`")
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc != 0:
        msg = load().fmscan_last_error().decode("utf-8", "replace")
        raise RuntimeError(msg or f"libfmscan_hip.so returned {rc}")
