"""ctypes access to oracle/libfmscan_cpu.so (test infrastructure, not product).

`forward_f64` / `backward_f64` are the compiled float64 checker (same results as
oracle/fm_scan_oracle.py, fast enough for millions of elements);
`port_forward` / `port_backward` run the storage-dtype float32-arithmetic port
on torch CPU tensors (float32, float16 or bfloat16): the timed CPU baseline.
Reference lines each C function follows: see the header of fmscan_cpu.c.
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import c_int, c_int64, c_void_p
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "libfmscan_cpu.so"
_lib = None


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-B", "libfmscan_cpu.so"], check=True,
                   capture_output=True, text=True)
    return LIB


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB.exists():
            build()
        lib = ctypes.CDLL(str(LIB))
        lib.fmscan_oracle_forward_f64.restype = None
        lib.fmscan_oracle_forward_f64.argtypes = [c_void_p] * 4 + [c_int64] * 4 + [c_int]
        lib.fmscan_oracle_backward_f64.restype = None
        lib.fmscan_oracle_backward_f64.argtypes = [c_void_p] * 8 + [c_int64] * 4 + [c_int]
        lib.fmscan_cpu_forward.restype = c_int
        lib.fmscan_cpu_forward.argtypes = [c_void_p] * 4 + [c_int64] * 4 + [c_int] * 3
        lib.fmscan_cpu_backward.restype = c_int
        lib.fmscan_cpu_backward.argtypes = [c_void_p] * 8 + [c_int64] * 4 + [c_int] * 3
        lib.fmscan_cpu_max_threads.restype = c_int
        lib.fmscan_cpu_max_threads.argtypes = []
        _lib = lib
    return _lib


def _f64(a):
    if a is None:
        return None
    if hasattr(a, "detach"):
        import torch

        a = a.detach().to("cpu").to(torch.float64).numpy()
    return np.ascontiguousarray(a, dtype=np.float64)


def _p(a):
    return None if a is None else a.ctypes.data


def forward_f64(gates, tokens, initial_state=None, plain=False):
    """float64 states (B, M, D, L) from gates (B, M, L), tokens (B, D, L)."""
    g, x, h0 = _f64(gates), _f64(tokens), _f64(initial_state)
    B, M, L = g.shape
    D = x.shape[1]
    assert x.shape == (B, D, L)
    assert h0 is None or h0.size == B * M * D
    out = np.empty((B, M, D, L), np.float64)
    load().fmscan_oracle_forward_f64(_p(g), _p(x), _p(h0), _p(out), B, M, D, L, int(plain))
    return out


def backward_f64(gates, out_grad, states, tokens, first_prop_grad=None, initial_state=None,
                 plain=False):
    """float64 (token_grad, gate_grad), both (B, M, D, L); arguments as
    fm_scan_oracle.backward_per_row."""
    g, G, h, x = _f64(gates), _f64(out_grad), _f64(states), _f64(tokens)
    fpg, h0 = _f64(first_prop_grad), _f64(initial_state)
    B, M, L = g.shape
    D = x.shape[1]
    assert G.shape == (B, M, D, L) and h.shape == (B, M, D, L) and x.shape == (B, D, L)
    dtok = np.empty((B, M, D, L), np.float64)
    dgate = np.empty((B, M, D, L), np.float64)
    load().fmscan_oracle_backward_f64(_p(g), _p(G), _p(fpg), _p(dtok), _p(h), _p(x), _p(dgate),
                                      _p(h0), B, M, D, L, int(plain))
    return dtok, dgate


def _dtype_code(t):
    import torch

    return {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[t.dtype]


def max_threads() -> int:
    return load().fmscan_cpu_max_threads()


def port_forward(gates, tokens, initial_state, out, plain=False, nthreads=0):
    """Storage-dtype CPU port on contiguous torch CPU tensors; fills and returns `out`."""
    B, M, D, L = out.shape
    for t in (gates, tokens, out):
        assert t.device.type == "cpu" and t.is_contiguous() and t.dtype == gates.dtype
    rc = load().fmscan_cpu_forward(gates.data_ptr(), tokens.data_ptr(),
                                   None if initial_state is None else initial_state.data_ptr(),
                                   out.data_ptr(), B, M, D, L, _dtype_code(gates), int(plain), nthreads)
    assert rc == 0
    return out


def port_backward(gates, out_grad, first_prop_grad, token_grad, states, tokens, gate_grad,
                  initial_state=None, plain=False, nthreads=0):
    B, M, D, L = states.shape
    for t in (gates, out_grad, token_grad, states, tokens, gate_grad):
        assert t.device.type == "cpu" and t.is_contiguous() and t.dtype == gates.dtype
    rc = load().fmscan_cpu_backward(
        gates.data_ptr(), out_grad.data_ptr(),
        None if first_prop_grad is None else first_prop_grad.data_ptr(), token_grad.data_ptr(),
        states.data_ptr(), tokens.data_ptr(), gate_grad.data_ptr(),
        None if initial_state is None else initial_state.data_ptr(),
        B, M, D, L, _dtype_code(gates), int(plain), nthreads)
    assert rc == 0
