"""ctypes binding of libfmscan_hip.so (interface: include/fmscan.h).

There is no other implementation behind these calls: if the library cannot
be loaded the import of `fm_amd.scan.fm_scan` fails, and tensors that are not
on a GPU are rejected.
"""
from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_uint, c_void_p

from . import build as _build

ABI_VERSION = 3

DTYPE_F32, DTYPE_F16, DTYPE_BF16 = 0, 1, 2
FLAG_PLAIN = 0x1
FLAG_WAVES_SHIFT = 8
FLAG_BLOCKS_SHIFT = 12
FLAG_DEPTH_SHIFT = 16
FLAG_SEGMENTS_SHIFT = 20

_lib = None


def load() -> ctypes.CDLL:
    """Loads the built library; builds it first only when no build exists."""
    global _lib
    if _lib is not None:
        return _lib
    if not _build.LIB.exists():
        _build.build(verbose=False)
    lib = ctypes.CDLL(str(_build.LIB))
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
    lib.fmscan_backward.restype = c_int
    lib.fmscan_backward.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_void_p,
                                    c_int64, c_int64, c_int64, c_int64, c_int, c_uint,
                                    c_void_p, c_size_t, c_void_p]
    lib.fmscan_reduced_groups.restype = c_int64
    lib.fmscan_reduced_groups.argtypes = [c_int64]
    lib.fmscan_backward_reduced.restype = c_int
    lib.fmscan_backward_reduced.argtypes = [c_void_p] * 9 + [c_int64] * 4 + [c_int, c_uint, c_void_p]
    lib.fmscan_backward_layer.restype = c_int
    lib.fmscan_backward_layer.argtypes = [c_void_p] * 13 + [c_int64] * 4 + [c_int, c_uint, c_void_p]
    dims = [c_int64] * 4
    lib.fmscan_readout_inv_rms.restype = c_int
    lib.fmscan_readout_inv_rms.argtypes = [c_void_p] * 2 + dims + [c_int, c_float, c_void_p]
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
