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

__all__ = ["forward", "backward_per_row", "backward", "to_f64"]


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
