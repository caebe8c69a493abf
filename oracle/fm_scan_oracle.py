"""CPU oracle of the Factorization-Memory scan (test infrastructure, not product).

This module restates, in float64 numpy, what the reference computes on the
path `fm_scan -> FM_Scan -> fm_scan_forward / fm_scan_backward`. Only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` may import
it; nothing under `fm_amd/` or `fm/` does, and the product never falls back to
it.

What each function follows in the reference:

* `forward`            fm/scan/fm_pytorch.py:19-42 (the per-timestep loop, the
                       default zero initial state, output order (B, M, D, L)) and
                       fm/scan/fm_scan.cuh:110,116,121-131 (the kernel computes
                       the same recurrence with the input scaled by 1 - gate).
* `backward_per_row`   fm/scan/fm_scan.cuh:86-88,103-108,121 (reverse scan with the
                       gate of the following step, 1.0 at the last step,
                       firstPropGrad as the incoming value), :184-185 (token
                       gradient scaled by 1 - gate) and :188-208 (gate gradient
                       (h[t-1] - x[t]) * delta, h[-1] read from the kernel's
                       `initial_state` argument, which fm_scan_backward fills with
                       firstPropGrad, :380).
* `backward`           fm/scan/fm_scan.py:61-81 (zero firstPropGrad, the sums
                       over D for d_gates and over M for d_tokens).
* `readout_forward`    fm/scan/fm_scan.py:124-131 (inside fm_memory): RMS norm over D
                       of every slot, then einsum 'blm,bmdl->bld'; here with time
                       last: read (B, M, L), output (B, D, L).
* `readout_backward`   the gradients of those lines, which the reference leaves to
                       autograd; written out by hand and pinned against finite
                       differences and against autograd through the same PyTorch
                       operations the reference lines name (tests/test_oracle.py).
* `memory_forward`     fm/scan/fm_scan.py:115-133, the whole layer.
* `memory_backward`    the gradients of the whole layer (left to autograd by the reference):
                       the chain rule through :116-119,130 on top of `readout_backward` and
                       `backward`; pinned against autograd through the operations those lines
                       name and against finite differences (tests/test_oracle.py).

How it is pinned (tests/test_oracle.py): exact rational arithmetic on small
inputs with forward-mode derivatives (tests/golden/), closed forms (constant
gate = geometric series, scipy.signal.lfilter, cumulative sum in plain mode,
reset/hold special cases), central finite differences in float64, the adjoint
identity, and segment chaining. The reference holds no golden vector for this
path (its notebook is stored without outputs), so none is used.

The reference kernel also rounds each (m, d) contribution to the storage dtype
before the D / M sums (fm_scan.cuh:184,207); this oracle keeps float64
throughout, callers round where they compare.
"""
from __future__ import annotations

import numpy as np

__all__ = ["forward", "backward_per_row", "backward", "to_f64", "readout_forward", "readout_backward",
           "memory_forward", "memory_backward"]


def to_f64(a):
    """float64 numpy copy of a numpy array or a torch tensor (any float dtype)."""
    if hasattr(a, "detach"):
        a = a.detach().to("cpu")
        try:
            import torch

            a = a.to(torch.float64).numpy()
        except Exception:  # pragma: no cover
            a = a.double().numpy()
    return np.ascontiguousarray(a, dtype=np.float64)


def _check(gates, tokens):
    assert gates.ndim == 3 and tokens.ndim == 3, "gates (B,M,L), tokens (B,D,L)"
    B, M, L = gates.shape
    B1, D, L1 = tokens.shape
    assert B == B1 and L == L1
    return B, M, D, L


def forward(gates, tokens, initial_state=None, plain=False):
    """h[b,m,d,t] = g[b,m,t] h[b,m,d,t-1] + u[b,m,d,t], u = (1-g) x (plain: u = x).

    gates (B,M,L), tokens (B,D,L), initial_state (B,M,D) or None (zeros).
    Returns float64 (B,M,D,L).
    """
    g = to_f64(gates)
    x = to_f64(tokens)
    B, M, D, L = _check(g, x)
    h = np.zeros((B, M, D), np.float64) if initial_state is None else to_f64(initial_state).copy()
    assert h.shape == (B, M, D)
    out = np.empty((B, M, D, L), np.float64)
    for t in range(L):
        gt = g[:, :, t][:, :, None]
        xt = x[:, :, t][:, None, :]
        u = xt if plain else (1.0 - gt) * xt
        h = gt * h + u
        out[:, :, :, t] = h
    return out


def backward_per_row(gates, out_grad, states, tokens, first_prop_grad=None, initial_state=None,
                     plain=False):
    """The two (B,M,D,L) tensors the reference kernel writes in backward mode.

    delta[t] = G[t] + g[t+1] delta[t+1], delta[L] = first_prop_grad (zeros if None)
    token_grad[b,m,d,t] = (1 - g[t]) delta[t]               (plain: delta[t])
    gate_grad [b,m,d,t] = (h[t-1] - x[t]) delta[t]          (plain: h[t-1] delta[t])
    `states` is the h the forward pass stored (what the kernel reads back).
    h[-1] is `initial_state`; None reproduces the reference kernel, which uses
    first_prop_grad there.
    Returns (token_grad, gate_grad, delta), float64.
    """
    g = to_f64(gates)
    G = to_f64(out_grad)
    h = to_f64(states)
    x = to_f64(tokens)
    B, M, D, L = _check(g, x)
    assert G.shape == (B, M, D, L) and h.shape == (B, M, D, L)
    fpg = np.zeros((B, M, D)) if first_prop_grad is None else to_f64(first_prop_grad)
    hm1 = fpg if initial_state is None else to_f64(initial_state)
    delta = np.empty_like(G)
    nxt = fpg.copy()  # g[t+1] * delta[t+1]; at t = L-1 the gate is 1
    for t in range(L - 1, -1, -1):
        d = G[:, :, :, t] + nxt
        delta[:, :, :, t] = d
        nxt = g[:, :, t][:, :, None] * d
    hprev = np.concatenate([hm1[:, :, :, None], h[:, :, :, :-1]], axis=3)
    gb = g[:, :, None, :]
    xb = x[:, None, :, :]
    if plain:
        token_grad = delta.copy()
        gate_grad = hprev * delta
    else:
        token_grad = (1.0 - gb) * delta
        gate_grad = (hprev - xb) * delta
    return token_grad, gate_grad, delta


def backward(gates, tokens, out_grad, initial_state=None, plain=False, states=None,
             first_prop_grad=None, exact_h0=True):
    """Gradients of sum(out_grad * forward(gates, tokens, initial_state)).

    Returns (d_gates (B,M,L), d_tokens (B,D,L), d_initial_state (B,M,D)).
    exact_h0=True uses the true initial state for the gate gradient at t = 0 (the
    derivative of the recurrence); False reproduces the reference's CUDA path,
    which uses first_prop_grad (zeros) there. The reference returns None for the
    third gradient (fm_scan.py:80-81); the value g[0] * delta[0] is returned here
    because the reference's per-timestep PyTorch path yields it through autograd.
    """
    g = to_f64(gates)
    if states is None:
        states = forward(gates, tokens, initial_state, plain)
    h0 = None
    if exact_h0:
        B, M, L = g.shape
        D = to_f64(tokens).shape[1]
        h0 = np.zeros((B, M, D)) if initial_state is None else to_f64(initial_state)
    tg, gg, delta = backward_per_row(gates, out_grad, states, tokens, first_prop_grad, h0, plain)
    d_gates = gg.sum(axis=2)
    d_tokens = tg.sum(axis=1)
    d_h0 = g[:, :, 0][:, :, None] * delta[:, :, :, 0]
    return d_gates, d_tokens, d_h0


def readout_forward(states, read, mem_norm=True, eps=1e-6):
    """states (B, M, D, L), read (B, M, L) -> (output (B, D, L), states as returned, inv_rms).

    fm_scan.py:125-127: inv_rms = rsqrt(mean(states**2, dim=2) + eps), states * inv_rms;
    fm_scan.py:130-131: output[b,l,d] = sum_m read[b,l,m] * states[b,m,d,l].
    """
    states = to_f64(states)
    read = to_f64(read)
    inv_rms = None
    if mem_norm:
        inv_rms = 1.0 / np.sqrt(np.mean(states * states, axis=2) + eps)  # (B, M, L)
        states = states * inv_rms[:, :, None, :]
    output = np.einsum("bml,bmdl->bdl", read, states)
    return output, states, inv_rms


def readout_backward(out_grad, ext_grad, read, states, mem_norm=True, eps=1e-6):
    """Gradients of readout_forward with respect to `states` (before the norm) and `read`.

    out_grad (B, D, L) is the gradient of the output, ext_grad (B, M, D, L) or None the
    one arriving at the returned states. With n = states * r, r = inv_rms:
        dn = read * out_grad + ext_grad,  d read = sum_d out_grad * n,
        d states = r * (dn - n * mean_d(dn * n)).
    """
    states = to_f64(states)
    read = to_f64(read)
    out_grad = to_f64(out_grad)
    _, normed, inv_rms = readout_forward(states, read, mem_norm, eps)
    dn = read[:, :, None, :] * out_grad[:, None, :, :]
    if ext_grad is not None:
        dn = dn + to_f64(ext_grad)
    read_grad = np.einsum("bdl,bmdl->bml", out_grad, normed)
    if not mem_norm:
        return dn, read_grad
    inner = np.mean(dn * normed, axis=2, keepdims=True)
    return inv_rms[:, :, None, :] * (dn - normed * inner), read_grad


def _layer_operands(alpha, update_scale, output_scale, inputs, storage):
    """gates (B, M, L), tokens (B, D, L), read (B, M, L) as the layer hands them to the scan and
    the read-out. `storage`, when given, rounds an array to the layer's storage dtype, and it is
    applied wherever the reference holds a tensor of that dtype: fm_scan.py:116 makes
    `update_weight = alpha * update_scale` (one tensor, rounded), :119 makes
    `decay_weight = 1.0 - update_weight` from the rounded product (a second tensor, rounded
    again), :130 makes `alpha * output_scale` (rounded once). Two roundings for the gates, not
    one: 1 - round(a * u) and round(1 - a * u) differ by a unit in the last place for about one
    gate in a hundred, and a gate near one moves by up to 2^-9 per rounding in bfloat16, which
    changes the decay it stands for. Pinned bit for bit against those PyTorch operations on
    bfloat16, float16 and float32 tensors in tests/test_oracle.py."""
    storage = storage or (lambda a: a)
    write = storage(np.ascontiguousarray(np.transpose(alpha * update_scale, (0, 2, 1))))  # :116,118
    tokens = np.ascontiguousarray(np.transpose(inputs, (0, 2, 1)))                    # :117
    gates = storage(1.0 - write)                                                       # :119
    read = storage(np.ascontiguousarray(np.transpose(alpha * output_scale, (0, 2, 1))))  # :130
    return gates, tokens, read


def memory_forward(alpha, update_scale, output_scale, inputs, initial_state=None, mem_norm=True, eps=1e-6,
                   storage=None):
    """fm_memory (fm_scan.py:102-133): alpha (B, L, M), scales (B, L, 1), inputs (B, L, D)
    -> (output (B, L, D), memory states (B, M, D, L)). `storage`: see _layer_operands."""
    alpha, update_scale, output_scale, inputs = (to_f64(a) for a in (alpha, update_scale, output_scale, inputs))
    gates, tokens, read = _layer_operands(alpha, update_scale, output_scale, inputs, storage)
    states = forward(gates, tokens, initial_state)                                     # :121
    output, states, _ = readout_forward(states, read, mem_norm, eps)
    return np.ascontiguousarray(np.transpose(output, (0, 2, 1))), states


def memory_backward(alpha, update_scale, output_scale, inputs, out_grad, mem_grad=None, initial_state=None,
                    mem_norm=True, eps=1e-6, storage=None):
    """Gradients of sum(out_grad * output) + sum(mem_grad * memory_states) for memory_forward.

    out_grad (B, L, D) or None, mem_grad (B, M, D, L) or None. Returns a dict with d_alpha (B, L, M),
    d_update_scale (B, L, 1), d_output_scale (B, L, 1), d_inputs (B, L, D), d_initial_state (B, M, D).
    `storage` (see _layer_operands) rounds the gates and read weights the gradients are taken at; the
    rounding itself passes gradients through unchanged, as autograd does for a cast.
    """
    alpha, update_scale, output_scale, inputs = (to_f64(a) for a in (alpha, update_scale, output_scale, inputs))
    B, L, M = alpha.shape
    D = inputs.shape[2]
    gates, tokens, read = _layer_operands(alpha, update_scale, output_scale, inputs, storage)
    states = forward(gates, tokens, initial_state)
    og = np.zeros((B, D, L)) if out_grad is None else np.ascontiguousarray(np.transpose(to_f64(out_grad), (0, 2, 1)))
    ext = None if mem_grad is None else to_f64(mem_grad)
    if mem_norm:
        d_states, d_read = readout_backward(og, ext, read, states, True, eps)
    else:  # the states are returned as they are: mem_grad reaches them unchanged
        d_states, d_read = readout_backward(og, None, read, states, False, eps)
        if ext is not None:
            d_states = d_states + ext
    d_gates, d_tokens, d_h0 = backward(gates, tokens, d_states, initial_state, states=states)
    dg = np.transpose(d_gates, (0, 2, 1))   # (B, L, M): gates = 1 - alpha * update_scale
    dr = np.transpose(d_read, (0, 2, 1))    # (B, L, M): read = alpha * output_scale
    return {"d_alpha": dr * output_scale - dg * update_scale,
            "d_update_scale": -(dg * alpha).sum(axis=2, keepdims=True),
            "d_output_scale": (dr * alpha).sum(axis=2, keepdims=True),
            "d_inputs": np.ascontiguousarray(np.transpose(d_tokens, (0, 2, 1))),
            "d_initial_state": d_h0}
