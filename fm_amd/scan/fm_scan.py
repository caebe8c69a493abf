"""Factorization-Memory scan on MI355X: the module that stands where the reference's
`fm/scan/fm_scan.py` stands.

Exports, with the reference's names and positional signatures:

    fm_scan_forward(gates, tokens, initial_state, out) -> out        fm_scan.py:9,34 / fm_scan.cuh:344-358
    fm_scan_backward(gates, outGrad, firstPropGrad, tokenGradOut,
                     cached_output, input_tokens, gateGradOut)        fm_scan.py:11-15,35 / fm_scan.cuh:361-381
    FM_Scan (torch.autograd.Function)                                fm_scan.py:37-81
    fm_scan(gates, tokens, initial_state=None)                       fm_scan.py:84-99
    fm_memory(alpha, update_scale, output_scale, inputs, ...)        fm_scan.py:102-133

and, for what fm_memory does with the states after the scan (RMS norm over D and the
read-out over the M slots, fm_scan.py:124-131), `fm_readout` / `FM_Readout`, which run
those steps and their gradients as four kernels instead of PyTorch operations over
(B, M, D, L) tensors.

The two extension functions call libfmscan_hip.so through ctypes with raw device
pointers and the current HIP stream; there is no CPU implementation behind them.
"""
from __future__ import annotations

import ctypes

import torch

from .. import _lib

__all__ = ["fm_scan_forward", "fm_scan_backward", "fm_scan_backward_reduced", "FM_Scan", "fm_scan",
           "fm_readout_forward", "fm_readout_backward", "FM_Readout", "fm_readout", "FM_Layer", "fm_layer",
           "FM_Memory", "fm_memory", "module"]

_DTYPES = {torch.float32: _lib.DTYPE_F32, torch.float16: _lib.DTYPE_F16,
           torch.bfloat16: _lib.DTYPE_BF16}

class _Extension:
    """Stands where the reference's `module` stands (fm_scan.py:18-35, the object load_inline
    returns): `module.fm_scan_forward` and `module.fm_scan_backward` are the two extension
    functions; every other attribute is an entry point of libfmscan_hip.so."""

    def __init__(self, lib):
        self._lib = lib

    def __getattr__(self, name):
        if name in ("fm_scan_forward", "fm_scan_backward"):
            return globals()[name]
        return getattr(self._lib, name)


# the library is loaded when this module is imported, as the reference builds and
# loads its extension at import (fm_scan.py:18-33); a missing library is an error here
_raw = _lib.load()
module = _Extension(_raw)


def _require(cond: bool, what: str) -> None:
    # the reference's TORCH_CHECKs surface as RuntimeError
    if not cond:
        raise RuntimeError(what)


def _dtype_code(t: torch.Tensor) -> int:
    _require(t.dtype in _DTYPES,
             f"Unsupported tensor dtype {t.dtype}: expecting bfloat16, float16 or float32")
    return _DTYPES[t.dtype]


def _on_gpu(name: str, t: torch.Tensor, dev: torch.device) -> None:
    _require(t.is_cuda, f"{name} must be a GPU tensor (got device {t.device}); "
                        "this scan has no CPU implementation")
    _require(t.device == dev, f"{name} is on {t.device}, expected {dev}")


class _on_device:
    """`with torch.cuda.device(dev)` without its cost when `dev` is already current."""

    __slots__ = ("ctx",)

    def __init__(self, dev):
        self.ctx = None if torch.cuda.current_device() == dev.index else torch.cuda.device(dev)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def _flags(plain: bool, waves_per_row: int, blocks_per_cu: int, depth: int, segments: int) -> int:
    return ((_lib.FLAG_PLAIN if plain else 0) | (int(waves_per_row) << _lib.FLAG_WAVES_SHIFT)
            | (int(blocks_per_cu) << _lib.FLAG_BLOCKS_SHIFT) | (int(depth) << _lib.FLAG_DEPTH_SHIFT)
            | (int(segments) << _lib.FLAG_SEGMENTS_SHIFT))


def _workspace(B, M, D, L, code, flags, device):
    """Scratch for the carries between the segments of a cut row (few rows, long L);
    None when the library scans every row in one piece."""
    if B * M * D >= 32 and not (flags >> _lib.FLAG_SEGMENTS_SHIFT):
        return None, 0  # rows are only cut on request or when there are very few of them
    need = _raw.fmscan_workspace_bytes(B, M, D, L, code, flags)
    if not need:
        return None, 0
    return torch.empty(need, dtype=torch.uint8, device=device), need


def fm_scan_forward(gates, tokens, initial_state, out, *, plain=False, waves_per_row=0, blocks_per_cu=0,
                    depth=0, segments=0):
    """Writes the scan states into `out` (B, M, D, L) and returns `out`.

    gates (B, M, L), tokens (B, D, L), initial_state (B, M, D); everything
    contiguous, on one GPU, of one dtype. Sizes are read from `out`, as the
    reference launcher does (fm_scan.cuh:265-269). `plain=True` drops the
    (1 - gate) input scaling (h_t = g_t h_{t-1} + x_t).
    """
    dev = out.device
    for name, t in (("gates", gates), ("tokens", tokens), ("initial_state", initial_state),
                    ("out", out)):
        _on_gpu(name, t, dev)
        _require(t.is_contiguous(), f"{name} must be contiguous")
        _require(t.dtype == gates.dtype, f"{name} has dtype {t.dtype}, gates has {gates.dtype}")
    _require(out.dim() == 4, "out must be (B, M, D, L)")
    B, M, D, L = out.shape
    _require(tuple(gates.shape) == (B, M, L), f"gates must be {(B, M, L)}, got {tuple(gates.shape)}")
    _require(tuple(tokens.shape) == (B, D, L), f"tokens must be {(B, D, L)}, got {tuple(tokens.shape)}")
    _require(initial_state.numel() == B * M * D, f"initial_state must hold {B * M * D} elements")
    code = _dtype_code(gates)
    if out.numel() == 0:
        return out
    flags = _flags(plain, waves_per_row, blocks_per_cu, depth, segments)
    with _on_device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        ws, ws_bytes = _workspace(B, M, D, L, code, flags, dev)
        _lib.check(_raw.fmscan_forward(gates.data_ptr(), tokens.data_ptr(), initial_state.data_ptr(),
                                         out.data_ptr(), B, M, D, L, code, flags,
                                         None if ws is None else ws.data_ptr(), ws_bytes, stream))
    return out


def fm_scan_backward(gates, outGrad, firstPropGrad, tokenGradOut, cached_output, input_tokens,
                     gateGradOut, *, initial_state=None, initial_state_grad=None, plain=False,
                     waves_per_row=0, blocks_per_cu=0, depth=0, segments=0):
    """Reverse scan of `outGrad` (B, M, D, L); fills `tokenGradOut` and `gateGradOut`
    (both (B, M, D, L), one contribution per (m, d) pair) and returns None.

    With the seven positional arguments alone this computes what the reference
    extension computes, including its use of `firstPropGrad` as the state before
    the first step in the gate gradient (fm_scan.cuh:196,380). `initial_state`
    (B, M, D), when given, is used there instead; `initial_state_grad` (B, M, D), when
    given, receives the gradient with respect to the initial state.
    """
    dev = gates.device
    named = [("gates", gates), ("outGrad", outGrad), ("firstPropGrad", firstPropGrad),
             ("tokenGradOut", tokenGradOut), ("cached_output", cached_output),
             ("input_tokens", input_tokens), ("gateGradOut", gateGradOut)]
    if initial_state is not None:
        named.append(("initial_state", initial_state))
    if initial_state_grad is not None:
        named.append(("initial_state_grad", initial_state_grad))
    for name, t in named:
        _on_gpu(name, t, dev)
        _require(t.is_contiguous(), f"{name} must be contiguous")
        _require(t.dtype == gates.dtype, f"{name} has dtype {t.dtype}, gates has {gates.dtype}")
    _require(cached_output.dim() == 4, "cached_output must be (B, M, D, L)")
    B, M, D, L = cached_output.shape
    full = (B, M, D, L)
    _require(tuple(gates.shape) == (B, M, L), f"gates must be {(B, M, L)}, got {tuple(gates.shape)}")
    _require(tuple(input_tokens.shape) == (B, D, L),
             f"input_tokens must be {(B, D, L)}, got {tuple(input_tokens.shape)}")
    for name, t in (("outGrad", outGrad), ("tokenGradOut", tokenGradOut), ("gateGradOut", gateGradOut)):
        _require(tuple(t.shape) == full, f"{name} must be {full}, got {tuple(t.shape)}")
    _require(firstPropGrad.numel() == B * M * D, f"firstPropGrad must hold {B * M * D} elements")
    for name, t in (("initial_state", initial_state), ("initial_state_grad", initial_state_grad)):
        if t is not None:
            _require(t.numel() == B * M * D, f"{name} must hold {B * M * D} elements")
    code = _dtype_code(gates)
    if cached_output.numel() == 0:
        return None
    flags = _flags(plain, waves_per_row, blocks_per_cu, depth, segments)
    with _on_device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        ws, ws_bytes = _workspace(B, M, D, L, code, flags, dev)
        _lib.check(_raw.fmscan_backward(
            gates.data_ptr(), outGrad.data_ptr(), firstPropGrad.data_ptr(), tokenGradOut.data_ptr(),
            cached_output.data_ptr(), input_tokens.data_ptr(), gateGradOut.data_ptr(),
            None if initial_state is None else initial_state.data_ptr(),
            None if initial_state_grad is None else initial_state_grad.data_ptr(),
            B, M, D, L, code, flags, None if ws is None else ws.data_ptr(), ws_bytes, stream))
    return None


def _reduced_ok(gates, tokens, states, grad_output) -> bool:
    """The fused-sum backward needs both sums to be real (M > 1 and D > 1), 16-byte aligned
    rows and pointers, and one float of LDS per memory row and wave."""
    B, M, D, L = states.shape
    if M < 2 or D < 2 or M > 2048 or (L * states.element_size()) % 16:
        return False
    return all(t.data_ptr() % 16 == 0 for t in (gates, tokens, states, grad_output))


def _packed_reduced_ok(*tensors):
    """fmscan_backward_reduced_packed needs 16-byte aligned pointers (the rows' length is the library's to judge)."""
    return all(t.data_ptr() % 16 == 0 for t in tensors)


def fm_scan_backward_reduced(gates, outGrad, firstPropGrad, cached_output, input_tokens, *,
                             initial_state=None, initial_state_grad=None, plain=False):
    """Backward scan that returns the summed gradients (d_gates (B, M, L), d_tokens (B, D, L))
    without materialising the two (B, M, D, L) per-pair tensors the reference writes and
    sums afterwards (fm_scan.py:70-78). Same mathematics as `fm_scan_backward` followed by
    `.sum(dim=2)` / `.sum(dim=1)`, with the sums accumulated in float32."""
    dev = gates.device
    named = [("gates", gates), ("outGrad", outGrad), ("firstPropGrad", firstPropGrad),
             ("cached_output", cached_output), ("input_tokens", input_tokens)]
    for name, t in (("initial_state", initial_state), ("initial_state_grad", initial_state_grad)):
        if t is not None:
            named.append((name, t))
    for name, t in named:
        _on_gpu(name, t, dev)
        _require(t.is_contiguous(), f"{name} must be contiguous")
        _require(t.dtype == gates.dtype, f"{name} has dtype {t.dtype}, gates has {gates.dtype}")
    _require(cached_output.dim() == 4, "cached_output must be (B, M, D, L)")
    B, M, D, L = cached_output.shape
    _require(tuple(gates.shape) == (B, M, L), f"gates must be {(B, M, L)}, got {tuple(gates.shape)}")
    _require(tuple(input_tokens.shape) == (B, D, L),
             f"input_tokens must be {(B, D, L)}, got {tuple(input_tokens.shape)}")
    _require(tuple(outGrad.shape) == (B, M, D, L), f"outGrad must be {(B, M, D, L)}")
    for name, t in (("firstPropGrad", firstPropGrad), ("initial_state", initial_state),
                    ("initial_state_grad", initial_state_grad)):
        if t is not None:
            _require(t.numel() == B * M * D, f"{name} must hold {B * M * D} elements")
    code = _dtype_code(gates)
    flags = _lib.FLAG_PLAIN if plain else 0
    # short rows: the kernel that puts several rows into a wave, where the library says it applies
    packed_groups = _raw.fmscan_reduced_packed_groups(B, M, D, L, code) if _packed_reduced_ok(
        gates, outGrad, cached_output, input_tokens) else 0
    if packed_groups > 0:
        partial = torch.empty((B, M, packed_groups, L), dtype=torch.float32, device=dev)
        d_tokens = torch.empty((B, D, L), dtype=gates.dtype, device=dev)
        with _on_device(dev):
            _lib.check(_raw.fmscan_backward_reduced_packed(
                gates.data_ptr(), outGrad.data_ptr(), firstPropGrad.data_ptr(), d_tokens.data_ptr(),
                cached_output.data_ptr(), input_tokens.data_ptr(), partial.data_ptr(), _ptr(initial_state),
                _ptr(initial_state_grad), B, M, D, L, code, flags, torch.cuda.current_stream(dev).cuda_stream))
        return _sum_groups(partial, gates.dtype), d_tokens
    # few batch elements: the rows are cut into segments (not in the plain form) and the slots of a batch
    # element dealt to `split` blocks, as the library plans it; those blocks' token gradients are summed after
    split, segments = _reduced_plan(B, M, D, L, code) if cached_output.numel() else (1, 1)
    if plain and segments > 1:
        split, segments = max(1, _raw.fmscan_reduced_split(B, M, D)), 1
    groups = _raw.fmscan_reduced_groups(B * split, D)
    partial = torch.empty((B, M, groups, L), dtype=torch.float32, device=dev)
    common = (cached_output.data_ptr(), input_tokens.data_ptr(), partial.data_ptr(), _ptr(initial_state),
              _ptr(initial_state_grad), B, M, D, L)
    if split > 1 or segments > 1:
        token_partial = torch.empty((B, D, split, L), dtype=torch.float32, device=dev)
        pairs = torch.empty(B * M * D * segments * 8 if segments > 1 else 0, dtype=torch.uint8, device=dev)
        with _on_device(dev):
            _lib.check(_raw.fmscan_backward_reduced_split(
                gates.data_ptr(), outGrad.data_ptr(), firstPropGrad.data_ptr(), token_partial.data_ptr(), *common,
                split, segments, pairs.data_ptr() if segments > 1 else None, pairs.numel(), code, flags,
                torch.cuda.current_stream(dev).cuda_stream))
        return _sum_groups(partial, gates.dtype), _sum_groups(token_partial, gates.dtype)
    d_tokens = torch.empty((B, D, L), dtype=gates.dtype, device=dev)
    if cached_output.numel():
        with _on_device(dev):
            _lib.check(_raw.fmscan_backward_reduced(
                gates.data_ptr(), outGrad.data_ptr(), firstPropGrad.data_ptr(), d_tokens.data_ptr(), *common,
                code, flags, torch.cuda.current_stream(dev).cuda_stream))
    return _sum_groups(partial, gates.dtype), d_tokens


def _sum_groups(partial, dtype):
    """(B, M, L) of `dtype` from the float32 (B, M, G, L) partials of the gates' gradient: their sum over
    G (what the reference does with torch.sum over a (B, M, D, L) tensor, fm_scan.py:76), rounded once.
    The same for the (B, D, split, L) partials of the token gradient."""
    B, M, G, L = partial.shape
    if G == 1 and dtype == torch.float32:
        return partial.squeeze(2)
    out = torch.empty((B, M, L), dtype=dtype, device=partial.device)
    if out.numel():
        with _on_device(partial.device):
            _lib.check(_raw.fmscan_sum_groups(partial.data_ptr(), G, out.data_ptr(), B * M, L, _dtype_code(out),
                                                torch.cuda.current_stream(partial.device).cuda_stream))
    return out


class FM_Scan(torch.autograd.Function):
    """states = FM_Scan.apply(gates, tokens, initial_state=None)

    gates (B, M, L), tokens (B, D, L) -> states (B, M, D, L) in gates.dtype;
    backward returns (d_gates (B, M, L), d_tokens (B, D, L), d_initial_state or None)
    (reference fm_scan.py:37-81, which always returns None in third place).
    """

    @staticmethod
    def forward(ctx, gates, tokens, initial_state=None):
        B_g, M, L_g = gates.shape
        B, D, L = tokens.shape
        assert L_g == L
        assert B_g == B
        assert gates.is_contiguous()
        assert tokens.is_contiguous()

        given_state = initial_state is not None
        if given_state:
            assert initial_state.shape == (B, M, D)
            assert initial_state.is_contiguous()
        else:
            initial_state = torch.zeros((B, M, D), device=gates.device, dtype=gates.dtype)

        states = torch.empty((B, M, D, L), device=gates.device, dtype=gates.dtype)
        fm_scan_forward(gates, tokens, initial_state, states)
        # The state before the first step enters the gate gradient at t = 0. The
        # reference does not keep it (fm_scan.py:55) and its kernel uses zero there;
        # its per-timestep PyTorch path differentiates the true recurrence. Kept
        # here only when the caller supplied one, so both agree in every case.
        ctx.save_for_backward(tokens, gates, states, initial_state if given_state else None)
        return states

    @staticmethod
    def backward(ctx, grad_output):
        tokens, gates, states, initial_state = ctx.saved_tensors
        return _scan_gradients(gates, tokens, states, initial_state, grad_output, ctx.needs_input_grad[2])


def _scan_gradients(gates, tokens, states, initial_state, grad_output, want_initial_state_grad):
    """(d_gates (B, M, L), d_tokens (B, D, L), d_initial_state or None) from the gradient of the
    states (reference fm_scan.py:61-81)."""
    B, M, D, L = states.shape
    assert states.is_contiguous()
    assert gates.is_contiguous()

    first_prop_grad = torch.zeros((B, M, D), device=gates.device, dtype=gates.dtype)
    grad_output = grad_output.contiguous()
    # The reference leaves the initial state's gradient unconnected (fm_scan.py:80-81); it
    # is returned here when autograd asks for it, as its per-timestep PyTorch path would.
    d_initial_state = torch.empty_like(first_prop_grad) if want_initial_state_grad else None

    code = _dtype_code(gates)
    if _reduced_ok(gates, tokens, states, grad_output) and (
            _raw.fmscan_reduced_pays(B, M, D, L, code) or _raw.fmscan_reduced_packed_groups(B, M, D, L, code) > 0):
        # both sums are real: one kernel produces d_gates and d_tokens directly (unless the shape leaves
        # it too few blocks: very few batch elements, slots and channels, rows too short to cut)
        d_gates, d_tokens = fm_scan_backward_reduced(
            gates, grad_output, first_prop_grad, states, tokens,
            initial_state=initial_state, initial_state_grad=d_initial_state)
        return d_gates, d_tokens, d_initial_state

    per_pair_gates = torch.empty_like(states)   # (B, M, D, L)
    per_pair_tokens = torch.empty_like(states)  # (B, M, D, L)
    fm_scan_backward(gates, grad_output, first_prop_grad, per_pair_tokens, states, tokens,
                     per_pair_gates, initial_state=initial_state,
                     initial_state_grad=d_initial_state)

    # (B, M, D, L) -> (B, M, L) and (B, D, L); a sum over an axis of length one
    # is the same tensor, so it is returned as a view without another pass
    d_gates = per_pair_gates.view(B, M, L) if D == 1 else per_pair_gates.sum(dim=2)
    d_tokens = per_pair_tokens.view(B, D, L) if M == 1 else per_pair_tokens.sum(dim=1)
    return d_gates, d_tokens, d_initial_state


def fm_scan(gates, tokens, initial_state=None):
    """First-order recurrence h_t = g_t * h_{t-1} + (1 - g_t) * x_t along the last axis.

    Arguments:
        gates (torch.Tensor): (B, M, L), contiguous, on the GPU.
        tokens (torch.Tensor): (B, D, L), contiguous, same dtype and device.
        initial_state (torch.Tensor, optional): (B, M, D), contiguous; zeros if omitted.
    Any L >= 1 is accepted (the reference needs a power of two in 32..131072).

    Returns:
        torch.Tensor: (B, M, D, L), the state after every step.
    """
    return FM_Scan.apply(gates, tokens, initial_state)


def _ptr(t):
    return None if t is None else t.data_ptr()


def _reduced_plan(B, M, D, L, code):
    """(split, segments) the library would use for the backward kernels with the sums inside at this shape."""
    split, segments = ctypes.c_int64(0), ctypes.c_int64(0)
    _lib.check(_raw.fmscan_reduced_plan(B, M, D, L, code, ctypes.byref(split), ctypes.byref(segments)))
    return max(1, split.value), max(1, segments.value)


def fm_readout_forward(states, read, mem_norm=True, norm_eps=1e-6, *, in_place=False):
    """RMS norm over D and read-out over M of scanned states (reference fm_scan.py:124-131).

    states (B, M, D, L), read (B, M, L) = (alpha * output_scale) with time last; same dtype,
    contiguous, on one GPU. Returns (output (B, D, L), normalised states (B, M, D, L) or None
    without the norm, inv_rms (B, M, L) float32 or None). `in_place` writes the normalised states
    over `states` (for callers that need the scanned states no longer).
    """
    dev = states.device
    for name, t in (("states", states), ("read", read)):
        _on_gpu(name, t, dev)
        _require(t.is_contiguous(), f"{name} must be contiguous")
        _require(t.dtype == states.dtype, f"{name} has dtype {t.dtype}, states has {states.dtype}")
    _require(states.dim() == 4, "states must be (B, M, D, L)")
    B, M, D, L = states.shape
    _require(tuple(read.shape) == (B, M, L), f"read must be {(B, M, L)}, got {tuple(read.shape)}")
    code = _dtype_code(states)
    output = torch.empty((B, D, L), dtype=states.dtype, device=dev)
    normed = (states if in_place else torch.empty_like(states)) if mem_norm else None
    inv_rms = torch.empty((B, M, L), dtype=torch.float32, device=dev) if mem_norm else None
    if states.numel():
        with _on_device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            if mem_norm:
                _lib.check(_raw.fmscan_readout_inv_rms(states.data_ptr(), inv_rms.data_ptr(), B, M, D, L,
                                                         code, float(norm_eps), stream))
            _lib.check(_raw.fmscan_readout_forward(states.data_ptr(), _ptr(inv_rms), read.data_ptr(),
                                                     _ptr(normed), output.data_ptr(), B, M, D, L, code,
                                                     stream))
    return output, normed, inv_rms


def fm_readout_backward(out_grad, ext_grad, read, states_n, inv_rms, *, read_grad_float32=False):
    """Gradients of fm_readout_forward.

    out_grad (B, D, L): gradient of the output; ext_grad (B, M, D, L) or None: gradient that
    arrives at the returned (normalised) states; states_n: the normalised states (the scanned
    states themselves without the norm); inv_rms (B, M, L) float32 or None without the norm.
    Returns (state_grad (B, M, D, L), read_grad (B, M, L)); read_grad stays in the float32 it
    is accumulated in when `read_grad_float32` is set.
    """
    dev = states_n.device
    for name, t in (("out_grad", out_grad), ("ext_grad", ext_grad), ("read", read), ("states_n", states_n),
                    ("inv_rms", inv_rms)):
        if t is None:
            continue
        _on_gpu(name, t, dev)
        _require(t.is_contiguous(), f"{name} must be contiguous")
        if name != "inv_rms":
            _require(t.dtype == states_n.dtype, f"{name} has dtype {t.dtype}, states_n has {states_n.dtype}")
    B, M, D, L = states_n.shape
    _require(tuple(out_grad.shape) == (B, D, L), f"out_grad must be {(B, D, L)}")
    _require(tuple(read.shape) == (B, M, L), f"read must be {(B, M, L)}")
    _require(ext_grad is None or tuple(ext_grad.shape) == (B, M, D, L), f"ext_grad must be {(B, M, D, L)}")
    _require(inv_rms is None or (tuple(inv_rms.shape) == (B, M, L) and inv_rms.dtype == torch.float32),
             f"inv_rms must be float32 {(B, M, L)}")
    code = _dtype_code(states_n)
    q = torch.empty((B, M, L), dtype=torch.float32, device=dev)
    qe = torch.empty_like(q) if (ext_grad is not None and inv_rms is not None) else None
    state_grad = torch.empty_like(states_n)
    if states_n.numel():
        with _on_device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            _lib.check(_raw.fmscan_readout_dot(states_n.data_ptr(), out_grad.data_ptr(),
                                                 None if qe is None else ext_grad.data_ptr(), q.data_ptr(),
                                                 _ptr(qe), None, None, None, None, None, B, M, D, L, code, stream))
            _lib.check(_raw.fmscan_readout_backward(states_n.data_ptr(), _ptr(inv_rms), read.data_ptr(),
                                                      out_grad.data_ptr(), _ptr(ext_grad), q.data_ptr(),
                                                      _ptr(qe), state_grad.data_ptr(), B, M, D, L, code,
                                                      stream))
    return state_grad, (q if read_grad_float32 else q.to(states_n.dtype))


class FM_Readout(torch.autograd.Function):
    """output, states_n = FM_Readout.apply(states, read, mem_norm, norm_eps)

    states (B, M, D, L), read (B, M, L) -> output (B, D, L) and the normalised states
    (None when mem_norm is false: the scanned states are then what the layer returns).
    """

    @staticmethod
    def forward(ctx, states, read, mem_norm=True, norm_eps=1e-6):
        output, normed, inv_rms = fm_readout_forward(states, read, mem_norm, norm_eps)
        ctx.mem_norm = bool(mem_norm)
        # the normalised states and inv_rms carry everything the gradient needs
        ctx.save_for_backward(read, normed if mem_norm else states, inv_rms)
        ctx.set_materialize_grads(False)
        return output, (normed if mem_norm else None)

    @staticmethod
    def backward(ctx, out_grad, ext_grad):
        read, states_n, inv_rms = ctx.saved_tensors
        if out_grad is None and ext_grad is None:
            return None, None, None, None
        if out_grad is None:
            B, M, D, L = states_n.shape
            out_grad = torch.zeros((B, D, L), dtype=states_n.dtype, device=states_n.device)
        state_grad, read_grad = fm_readout_backward(
            out_grad.contiguous(), None if ext_grad is None else ext_grad.contiguous(), read, states_n,
            inv_rms)
        return state_grad, read_grad, None, None


def fm_readout(states, read, mem_norm=True, norm_eps=1e-6):
    """(output (B, D, L), states as the layer returns them (B, M, D, L))."""
    output, normed = FM_Readout.apply(states, read, mem_norm, norm_eps)
    return output, (normed if mem_norm else states)


def _layer_forward(gates, tokens, initial_state, read, mem_norm, norm_eps):
    """Scan, RMS norm and read-out (reference fm_scan.py:121-131), time last. Returns what the
    layer hands back and what its gradient needs."""
    _require(gates.dim() == 3 and tokens.dim() == 3, "gates must be (B, M, L) and tokens (B, D, L)")
    B_g, M, L_g = gates.shape
    B, D, L = tokens.shape
    _require(L_g == L and B_g == B, f"gates {tuple(gates.shape)} and tokens {tuple(tokens.shape)} must agree in B and L")
    # Every tensor whose address goes to the library is checked here, before the route is chosen:
    # the fused routes below hand over raw pointers, and a tensor on the host or on another GPU, or
    # one of another element size, would be a memory fault in the kernel instead of an error here.
    dev = gates.device
    given_state = initial_state is not None
    named = [("gates", gates), ("tokens", tokens), ("read", read)]
    if given_state:
        named.append(("initial_state", initial_state))
    for name, t in named:
        _on_gpu(name, t, dev)
        _require(t.is_contiguous(), f"{name} must be contiguous")
        _require(t.dtype == gates.dtype, f"{name} has dtype {t.dtype}, gates has {gates.dtype}")
    _require(tuple(read.shape) == (B, M, L), f"read must be {(B, M, L)}, got {tuple(read.shape)}")
    if given_state:
        _require(tuple(initial_state.shape) == (B, M, D),
                 f"initial_state must be {(B, M, D)}, got {tuple(initial_state.shape)}")
    code = _dtype_code(gates)
    states = torch.empty((B, M, D, L), device=dev, dtype=gates.dtype)
    kept_state = initial_state if given_state else None
    # (few batch elements with few slots: the kernels below, a block per slot for the whole sequence, would
    # leave most of the GPU idle; the sequence is then cut into segments, or, where it is too short for
    # that or D too large, the separate kernels further down are taken)
    fused = mem_norm and states.numel() and (L * states.element_size()) % 16 == 0 and _aligned(gates, tokens, states, read)
    segments = _raw.fmscan_forward_normed_segments(B, M, D, L, code) if fused else 0  # 0: D beyond one block
    if fused and (segments > 1 or _raw.fmscan_forward_normed_pays(B, M, D)):
        inv_rms = torch.empty((B, M, L), dtype=torch.float32, device=dev)
        with _on_device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            if segments >= 1:
                # scan and norm in one kernel: the scanned states never reach memory
                # (no initial state: NULL, which the library reads as zeros; no fill kernel)
                head = (gates.data_ptr(), tokens.data_ptr(), _ptr(kept_state), states.data_ptr(), inv_rms.data_ptr(),
                        B, M, D, L, code, float(norm_eps))
                if segments > 1:
                    pairs = torch.empty(B * M * D * segments * 8, dtype=torch.uint8, device=dev)
                    _lib.check(_raw.fmscan_forward_normed_cut(*head, segments, pairs.data_ptr(), pairs.numel(), stream))
                else:
                    _lib.check(_raw.fmscan_forward_normed(*head, stream))
                output, _, _ = fm_readout_forward(states, read, mem_norm=False)  # the read-out alone
                return output, None, states, inv_rms, kept_state
            # too many rows per slot for one block: the scan leaves the sums of squares of blocks of rows,
            # so the norm needs no pass over the states of its own; scaling and read-out then in place
            groups = _raw.fmscan_sumsq_groups(D)
            partial = torch.empty((B, M, groups, L), dtype=torch.float32, device=dev)
            output = torch.empty((B, D, L), dtype=states.dtype, device=dev)
            _lib.check(_raw.fmscan_forward_sumsq(gates.data_ptr(), tokens.data_ptr(), _ptr(kept_state),
                                                   states.data_ptr(), partial.data_ptr(), B, M, D, L, code, stream))
            _lib.check(_raw.fmscan_sumsq_finish(partial.data_ptr(), groups, inv_rms.data_ptr(), B, M, D, L,
                                                  float(norm_eps), stream))
            _lib.check(_raw.fmscan_readout_forward(states.data_ptr(), inv_rms.data_ptr(), read.data_ptr(),
                                                     states.data_ptr(), output.data_ptr(), B, M, D, L, code, stream))
        return output, None, states, inv_rms, kept_state
    if not given_state:
        initial_state = torch.zeros((B, M, D), device=dev, dtype=gates.dtype)
    fm_scan_forward(gates, tokens, initial_state, states)
    # with the norm the scanned states are needed no longer (backward takes them back from the
    # normalised ones): normalise in place, one (B, M, D, L) tensor at any time
    output, normed, inv_rms = fm_readout_forward(states, read, mem_norm, norm_eps, in_place=bool(mem_norm))
    return output, (None if mem_norm else states), normed, inv_rms, kept_state


def _layer_gradients(gates, tokens, states, initial_state, read, normed, inv_rms, out_grad, ext_grad,
                     want_initial_state_grad):
    """Gradients of _layer_forward from those of its two results (either may be None, not both):
    (gate_grad_partial (B, M, G, L) float32, to be summed over G; d_tokens (B, D, L);
    d_initial_state or None; read_grad (B, M, L) float32).

    When nothing but the output feeds the loss, no (B, M, D, L) gradient tensor exists between
    the read-out and the scan: the scan's backward kernel makes it from the output's gradient,
    the normalised states and two per-slot coefficient vectors.
    """
    mem_norm = inv_rms is not None
    states_n = normed if mem_norm else states  # with the norm, `states` is None: not kept
    B, M, D, L = states_n.shape
    dev, dtype = states_n.device, states_n.dtype
    if out_grad is not None:
        out_grad = out_grad.contiguous()
    if states_n.numel() == 0:  # no batch element, slot, channel or step: nothing flows back
        zeros32 = torch.zeros((B, M, L), dtype=torch.float32, device=dev)
        return (zeros32.unsqueeze(2), torch.zeros((B, D, L), dtype=dtype, device=dev),
                torch.zeros((B, M, D), dtype=dtype, device=dev) if want_initial_state_grad else None, zeros32)

    if ext_grad is None and _reduced_ok(gates, tokens, states_n, states_n) and _aligned(read, out_grad):
        code = _dtype_code(states_n)
        q = torch.empty((B, M, L), dtype=torch.float32, device=dev)
        coef_out, coef_self = torch.empty_like(q), torch.empty_like(q)  # float32, like q
        rms = torch.empty_like(q) if mem_norm else None  # 1 / inv_rms: takes the scanned states back
        # few batch elements: the rows are cut into segments and the slots of a batch element dealt to
        # `split` blocks, as the library plans it; the token gradients of those blocks are summed after
        split, segments = _reduced_plan(B, M, D, L, code)
        # short rows: the kernel that puts several rows into a wave, where the library says it applies
        packed_groups = _raw.fmscan_reduced_packed_groups(B, M, D, L, code)
        if packed_groups > 0:
            split, segments = 1, 1
        divided = split > 1 or segments > 1
        groups = packed_groups if packed_groups > 0 else _raw.fmscan_reduced_groups(B * split, D)
        partial = torch.empty((B, M, groups, L), dtype=torch.float32, device=dev)
        d_h0 = torch.empty((B, M, D), dtype=dtype, device=dev) if want_initial_state_grad else None
        if divided:
            token_partial = torch.empty((B, D, split, L), dtype=torch.float32, device=dev)
            pairs = torch.empty(B * M * D * segments * 8 if segments > 1 else 0, dtype=torch.uint8, device=dev)
        else:
            d_tokens = torch.empty((B, D, L), dtype=dtype, device=dev)
        with _on_device(dev):
            stream = torch.cuda.current_stream(dev).cuda_stream
            _lib.check(_raw.fmscan_readout_dot(
                states_n.data_ptr(), out_grad.data_ptr(), None, q.data_ptr(), None, _ptr(inv_rms),
                read.data_ptr(), coef_out.data_ptr(), coef_self.data_ptr(), _ptr(rms), B, M, D, L, code, stream))
            head = (gates.data_ptr(), states_n.data_ptr(), coef_out.data_ptr(), coef_self.data_ptr(),
                    out_grad.data_ptr(), None)  # nothing arrives from beyond the last step
            tail = (None if mem_norm else states.data_ptr(),  # with the norm: states = states_n * rms
                    _ptr(rms), tokens.data_ptr(), partial.data_ptr(), _ptr(initial_state), _ptr(d_h0), B, M, D, L)
            if divided:
                _lib.check(_raw.fmscan_backward_layer_split(
                    *head, token_partial.data_ptr(), *tail, split, segments,
                    pairs.data_ptr() if segments > 1 else None, pairs.numel(), code, 0, stream))
            elif packed_groups > 0:
                _lib.check(_raw.fmscan_backward_layer_packed(*head, d_tokens.data_ptr(), *tail, code, 0, stream))
            else:
                _lib.check(_raw.fmscan_backward_layer(*head, d_tokens.data_ptr(), *tail, code, 0, stream))
        if divided:
            d_tokens = _sum_groups(token_partial, dtype)
        return partial, d_tokens, d_h0, q

    if out_grad is None:
        out_grad = torch.zeros((B, D, L), dtype=dtype, device=dev)
    # without the norm the states are returned as they are: ext_grad reaches them unchanged
    state_grad, q = fm_readout_backward(
        out_grad, ext_grad.contiguous() if (ext_grad is not None and mem_norm) else None, read, states_n,
        inv_rms, read_grad_float32=True)
    if ext_grad is not None and not mem_norm:
        state_grad += ext_grad
    if mem_norm:
        # the scanned states were not kept: take them back from the normalised ones, with rms in the
        # float32 it is held in and one rounding, as the fused route's kernel does
        states = (normed.float() * (1.0 / inv_rms).unsqueeze(2)).to(dtype)
    d_gates, d_tokens, d_h0 = _scan_gradients(gates, tokens, states, initial_state, state_grad,
                                              want_initial_state_grad)
    return d_gates.float().unsqueeze(2), d_tokens, d_h0, q


class FM_Layer(torch.autograd.Function):
    """output, memory_states = FM_Layer.apply(gates, tokens, initial_state, read, mem_norm, norm_eps)

    Scan, RMS norm and read-out of the layer as one node of the autograd graph (reference
    fm_scan.py:121-131), time last: gates, read (B, M, L), tokens (B, D, L), initial_state
    (B, M, D) or None -> output (B, D, L), memory states as the layer returns them (B, M, D, L).
    """

    @staticmethod
    def forward(ctx, gates, tokens, initial_state, read, mem_norm=True, norm_eps=1e-6):
        output, states, normed, inv_rms, kept_state = _layer_forward(gates, tokens, initial_state, read,
                                                                     mem_norm, norm_eps)
        # with the norm, the normalised states (returned anyway) and inv_rms stand in for the
        # scanned states: nothing else of size (B, M, D, L) is kept for backward
        ctx.save_for_backward(tokens, gates, None if mem_norm else states, kept_state, read, normed, inv_rms)
        ctx.set_materialize_grads(False)
        return output, (normed if mem_norm else states)

    @staticmethod
    def backward(ctx, out_grad, ext_grad):
        tokens, gates, states, initial_state, read, normed, inv_rms = ctx.saved_tensors
        if out_grad is None and ext_grad is None:
            return None, None, None, None, None, None
        partial, d_tokens, d_h0, q = _layer_gradients(gates, tokens, states, initial_state, read, normed,
                                                      inv_rms, out_grad, ext_grad, ctx.needs_input_grad[2])
        return _sum_groups(partial.contiguous(), gates.dtype), d_tokens, d_h0, q.to(gates.dtype), None, None


class FM_Memory(torch.autograd.Function):
    """output (B, L, D), memory_states (B, M, D, L) = FM_Memory.apply(alpha, update_scale,
    output_scale, inputs, initial_state, mem_norm, norm_eps): the whole layer (reference
    fm_scan.py:102-133) as one node, every step of it a kernel of the library."""

    @staticmethod
    def forward(ctx, alpha, update_scale, output_scale, inputs, initial_state, mem_norm=True, norm_eps=1e-6):
        dev = alpha.device
        for name, t in (("alpha", alpha), ("update_scale", update_scale), ("output_scale", output_scale),
                        ("inputs", inputs)):
            _on_gpu(name, t, dev)
            _require(t.dtype == alpha.dtype, f"{name} has dtype {t.dtype}, alpha has {alpha.dtype}")
        _require(alpha.dim() == 3 and inputs.dim() == 3, "alpha must be (B, L, M) and inputs (B, L, D)")
        B, L, M = alpha.shape
        _require(tuple(update_scale.shape) == (B, L, 1) and tuple(output_scale.shape) == (B, L, 1),
                 f"update_scale and output_scale must be {(B, L, 1)}")
        _require(inputs.shape[:2] == (B, L), f"inputs must be (B, L, D) with B, L = {(B, L)}")
        alpha, update_scale, output_scale = alpha.contiguous(), update_scale.contiguous(), output_scale.contiguous()
        code = _dtype_code(alpha)
        gates = torch.empty((B, M, L), dtype=alpha.dtype, device=dev)
        read = torch.empty_like(gates)
        if gates.numel():
            with _on_device(dev):
                _lib.check(_raw.fmscan_layer_prepare(
                    alpha.data_ptr(), update_scale.data_ptr(), output_scale.data_ptr(), gates.data_ptr(),
                    read.data_ptr(), B, L, M, code, torch.cuda.current_stream(dev).cuda_stream))
        tokens = _swap_last_two(inputs)
        output, states, normed, inv_rms, kept_state = _layer_forward(gates, tokens, initial_state, read,
                                                                     mem_norm, norm_eps)
        ctx.save_for_backward(alpha, update_scale, output_scale, tokens, gates, None if mem_norm else states,
                              kept_state, read, normed, inv_rms)
        ctx.set_materialize_grads(False)
        return _swap_last_two(output), (normed if mem_norm else states)

    @staticmethod
    def backward(ctx, out_grad, ext_grad):
        (alpha, update_scale, output_scale, tokens, gates, states, initial_state, read, normed,
         inv_rms) = ctx.saved_tensors
        if out_grad is None and ext_grad is None:
            return None, None, None, None, None, None, None
        partial, d_tokens, d_h0, q = _layer_gradients(
            gates, tokens, states, initial_state, read, normed, inv_rms,
            None if out_grad is None else _swap_last_two(out_grad), ext_grad, ctx.needs_input_grad[4])
        B, L, M = alpha.shape
        dev = alpha.device
        d_alpha = torch.empty_like(alpha)
        d_update_scale, d_output_scale = torch.empty_like(update_scale), torch.empty_like(output_scale)
        if partial.shape[2] > 64:
            # many groups of d: the finishing kernel walks them one by one, a reduction does better
            partial = _sum_groups(partial.contiguous(), torch.float32).unsqueeze(2)
        partial = partial.contiguous()
        if alpha.numel():
            with _on_device(dev):
                _lib.check(_raw.fmscan_layer_finish(
                    partial.data_ptr(), partial.shape[2], q.data_ptr(), alpha.data_ptr(), update_scale.data_ptr(),
                    output_scale.data_ptr(), d_alpha.data_ptr(), d_update_scale.data_ptr(),
                    d_output_scale.data_ptr(), B, L, M, _dtype_code(alpha),
                    torch.cuda.current_stream(dev).cuda_stream))
        return d_alpha, d_update_scale, d_output_scale, _swap_last_two(d_tokens), d_h0, None, None


def _aligned(*tensors):
    return all(t.data_ptr() % 16 == 0 for t in tensors)


def _swap_last_two(t):
    """Dense (B, C, R) copy of a (B, R, C) tensor: transpose(1, 2).contiguous() as one tiled kernel."""
    _require(t.dim() == 3, "expected a (B, R, C) tensor")
    _on_gpu("tensor", t, t.device)
    _require(t.element_size() in (2, 4), f"Unsupported tensor dtype {t.dtype}")
    t = t.contiguous()
    B, R, C = t.shape
    out = torch.empty((B, C, R), dtype=t.dtype, device=t.device)
    if t.numel():
        with _on_device(t.device):
            _lib.check(_raw.fmscan_swap_last_two(t.data_ptr(), out.data_ptr(), B, R, C, t.element_size(),
                                                   torch.cuda.current_stream(t.device).cuda_stream))
    return out


class _SwapLastTwo(torch.autograd.Function):
    @staticmethod
    def forward(ctx, t):
        return _swap_last_two(t)

    @staticmethod
    def backward(ctx, grad):
        return _swap_last_two(grad)


def fm_layer(gates, tokens, initial_state, read, mem_norm=True, norm_eps=1e-6):
    """(output (B, D, L), memory states (B, M, D, L)) of scan + RMS norm + read-out, time last."""
    return FM_Layer.apply(gates, tokens, initial_state, read, mem_norm, norm_eps)


def fm_memory(alpha, update_scale, output_scale, inputs, initial_state=None, mem_norm=True,
              norm_eps=1e-6):
    """The Factorization-Memory layer around the scan (reference fm_scan.py:102-133).

        alpha:        (B, L, M)  mixing weights over the M memory slots
        update_scale: (B, L, 1)
        output_scale: (B, L, 1)
        inputs:       (B, L, D)
        initial_state (B, M, D), optional
    Returns (output (B, L, D), memory_states (B, M, D, L)).

    The steps of the reference, each a kernel here: decay gates 1 - alpha * update_scale and read
    weights alpha * output_scale with time last (:116-119,130), tokens with time last (:117), the
    scan (:121), the RMS norm over D (:124-127), the read-out over the M slots and its way back to
    (B, L, D) (:130-131).
    """
    return FM_Memory.apply(alpha, update_scale, output_scale, inputs, initial_state, mem_norm, norm_eps)
