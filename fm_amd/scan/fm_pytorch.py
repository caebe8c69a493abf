"""Per-timestep PyTorch form of the scan, on whatever device its inputs live.

Stands where the reference's `fm/scan/fm_pytorch.py` stands: a slow, readable
statement of the recurrence that autograd can differentiate. `fm_scan` never
calls it; it is exported because the reference exports it (its notebook
compares the kernel against it, fm_test.ipynb:64,89).
"""
import torch

__all__ = ["fm_scan_pytorch"]


def fm_scan_pytorch(gates, tokens, initial_state=None):
    """h_t = g_t * h_{t-1} + (1 - g_t) * x_t, one step of t at a time.

    gates (B, M, L), tokens (B, D, L), initial_state (B, M, D) or None (zeros)
    -> (B, M, D, L), in the dtype of the inputs (reference fm_pytorch.py:19-42).
    """
    B, M, L = gates.shape
    B_t, D, L_t = tokens.shape
    assert L_t == L
    assert B_t == B
    if initial_state is None:
        state = gates.new_zeros((B, M, D))
    else:
        assert initial_state.shape == (B, M, D)
        assert initial_state.is_contiguous()
        state = initial_state

    keep = gates.unsqueeze(2)          # (B, M, 1, L)
    write = (1 - gates).unsqueeze(2)   # (B, M, 1, L)
    value = tokens.unsqueeze(1)        # (B, 1, D, L)
    steps = []
    for t in range(L):
        state = keep[..., t] * state + write[..., t] * value[..., t]
        steps.append(state)
    return torch.stack(steps, dim=3)
