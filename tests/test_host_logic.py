"""Host-side behaviour that needs no GPU: import paths, argument checks of the
extension functions and of FM_Scan, and the layer arithmetic of fm_memory around
the scan (with the scan itself replaced by the per-timestep PyTorch form)."""
import numpy as np
import pytest
import torch

import fm_scan_oracle as O


def test_reference_import_paths():
    from fm.scan.fm_pytorch import fm_scan_pytorch  # noqa: F401
    from fm.scan.fm_scan import (FM_Scan, fm_memory, fm_scan, fm_scan_backward,  # noqa: F401
                                 fm_scan_forward, module)
    import fm_amd.scan.fm_scan as impl

    assert fm_scan is impl.fm_scan and FM_Scan is impl.FM_Scan


def test_product_does_not_import_the_oracle():
    import sys
    import subprocess

    code = ("import sys; import fm.scan.fm_scan, fm.scan.fm_pytorch; "
            "bad=[m for m in sys.modules if 'oracle' in m or m=='fmscan_cpu']; print(bad); sys.exit(bool(bad))")
    from pathlib import Path
    root = Path(__file__).resolve().parent.parent
    res = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr


def test_cpu_tensors_are_rejected_loudly():
    from fm.scan.fm_scan import fm_scan, fm_scan_backward, fm_scan_forward

    g, x = torch.rand(1, 1, 32), torch.rand(1, 1, 32)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        fm_scan(g, x)
    out = torch.empty(1, 1, 1, 32)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        fm_scan_forward(g, x, torch.zeros(1, 1, 1), out)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        fm_scan_backward(g, out, torch.zeros(1, 1, 1), out.clone(), out, x, out.clone())
    from fm.scan.fm_scan import fm_memory, fm_readout

    with pytest.raises(RuntimeError, match="GPU tensor"):
        fm_readout(out, g)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        fm_memory(torch.rand(1, 32, 2), torch.rand(1, 32, 1), torch.rand(1, 32, 1), torch.rand(1, 32, 3))


def test_fm_scan_shape_asserts_match_reference_behaviour():
    from fm.scan.fm_scan import fm_scan

    with pytest.raises(AssertionError):  # sequence lengths differ
        fm_scan(torch.rand(2, 1, 32), torch.rand(2, 1, 64))
    with pytest.raises(AssertionError):  # batch sizes differ
        fm_scan(torch.rand(2, 1, 32), torch.rand(3, 1, 32))
    with pytest.raises(AssertionError):  # gates not contiguous
        fm_scan(torch.rand(2, 32, 2).transpose(1, 2), torch.rand(2, 1, 32))
    with pytest.raises(AssertionError):  # initial state of the wrong shape
        fm_scan(torch.rand(2, 3, 32), torch.rand(2, 4, 32), torch.zeros(2, 4, 3))


def test_fm_memory_layer_wiring(monkeypatch):
    """What fm_memory does around the two kernels' worth of work: gates 1 - alpha*update_scale
    with time last, tokens with time last, read weights alpha*output_scale with time last, and
    the output back to (B, L, D) (reference fm_scan.py:115-133). The scan is served by the
    per-timestep PyTorch form, the read-out by the oracle and the axis swaps by PyTorch here
    (no GPU); the result is
    compared with a direct numpy statement of the layer."""
    # (scan + norm + read-out are one call in the product, `fm_layer`: that is what is served here)
    import fm_amd.scan.fm_scan as impl
    from fm_amd.scan.fm_pytorch import fm_scan_pytorch

    def layer_on_cpu(gates, tokens, initial_state, read, mem_norm, eps):
        states = fm_scan_pytorch(gates, tokens, initial_state)
        out, normed, _ = O.readout_forward(states.numpy(), read.numpy(), mem_norm, eps)
        return torch.from_numpy(out), torch.from_numpy(normed)

    monkeypatch.setattr(impl, "fm_layer", layer_on_cpu)
    monkeypatch.setattr(impl, "_swap_last_two", lambda t: t.transpose(1, 2).contiguous())
    gen = torch.Generator().manual_seed(0)
    B, L, M, D = 2, 16, 3, 5
    alpha = torch.softmax(torch.randn(B, L, M, generator=gen, dtype=torch.float64), dim=-1)
    us = torch.rand(B, L, 1, generator=gen, dtype=torch.float64)
    os_ = torch.rand(B, L, 1, generator=gen, dtype=torch.float64)
    inp = torch.randn(B, L, D, generator=gen, dtype=torch.float64)
    h0 = torch.randn(B, M, D, generator=gen, dtype=torch.float64)
    for norm in (True, False):
        out, states = impl.fm_memory(alpha, us, os_, inp, h0, mem_norm=norm, norm_eps=1e-6)
        assert out.shape == (B, L, D) and states.shape == (B, M, D, L) and out.is_contiguous()
        g = 1.0 - (alpha * us).numpy().transpose(0, 2, 1)
        h = O.forward(g, inp.numpy().transpose(0, 2, 1), h0.numpy())
        if norm:
            h = h / np.sqrt((h ** 2).mean(axis=2, keepdims=True) + 1e-6)
        ref = np.einsum("blm,bmdl->bld", (alpha * os_).numpy(), h)
        np.testing.assert_allclose(states.numpy(), h, rtol=1e-12, atol=1e-12)
        np.testing.assert_allclose(out.numpy(), ref, rtol=1e-12, atol=1e-12)
