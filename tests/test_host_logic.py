"""Host-side behaviour that needs no GPU: import paths, the `module` object, argument
checks of the extension functions and of FM_Scan, loud failure on CPU tensors."""
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


def test_module_stands_in_for_the_reference_extension():
    """`module` is what load_inline returns in the reference (fm_scan.py:18-35): it carries the
    two extension functions; here it also gives access to the library's C entry points."""
    import fm.scan.fm_scan as m

    assert m.module.fm_scan_forward is m.fm_scan_forward
    assert m.module.fm_scan_backward is m.fm_scan_backward
    assert m.module.fmscan_abi_version() >= 3
    with pytest.raises(AttributeError):
        m.module.no_such_entry_point


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


def test_layer_checks_every_tensor_before_anything_is_launched(monkeypatch):
    """fm_memory / fm_layer hand raw pointers to the library; every tensor that goes there is checked for
    device, dtype, contiguity and shape first, whichever route the shape then takes. Run on the CPU with
    the device test relaxed to "same device as the gates" and a library that fails the test when called."""
    import fm_amd.scan.fm_scan as m

    class NoLaunch:
        def __getattr__(self, name):
            raise AssertionError(f"{name} was called before the arguments were checked")

    def same_device(name, t, dev):
        m._require(t.device == dev, f"{name} is on {t.device}, expected {dev}")

    monkeypatch.setattr(m, "_raw", NoLaunch())
    monkeypatch.setattr(m, "_on_gpu", same_device)
    B, M, D, L = 2, 3, 4, 64
    g, x, r = torch.rand(B, M, L), torch.rand(B, D, L), torch.rand(B, M, L)
    h0 = torch.rand(B, M, D)
    bad = [
        (dict(initial_state=h0.to("meta")), "initial_state is on meta"),
        (dict(initial_state=h0.double()), "initial_state has dtype"),
        (dict(initial_state=h0.to(torch.bfloat16)), "initial_state has dtype"),
        (dict(initial_state=torch.rand(B, D, M).transpose(1, 2)), "initial_state must be contiguous"),
        (dict(initial_state=torch.rand(B, M, D + 1)), "initial_state must be"),
        (dict(read=r.to("meta")), "read is on meta"),
        (dict(read=r.half()), "read has dtype"),
        (dict(read=torch.rand(B, M + 1, L)), "read must be"),
        (dict(tokens=x.to("meta")), "tokens is on meta"),
        (dict(tokens=x.to(torch.float16)), "tokens has dtype"),
        (dict(tokens=torch.rand(B, D, L + 8)), "must agree in B and L"),
    ]
    for mem_norm in (True, False):
        for change, message in bad:
            args = dict(gates=g, tokens=x, initial_state=h0, read=r)
            args.update(change)
            with pytest.raises(RuntimeError, match=message):
                m._layer_forward(args["gates"], args["tokens"], args["initial_state"], args["read"], mem_norm, 1e-6)


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



def test_bench_refuses_more_than_one_gpu_and_no_gpu():
    """bench.py runs on one GPU: asked for more it says so and exits; without a GPU it says
    that the scan has no CPU path to benchmark (it never falls back to the CPU checker)."""
    import subprocess
    import sys
    from pathlib import Path

    bench = Path(__file__).resolve().parents[1] / "bench.py"
    two = subprocess.run([sys.executable, str(bench), "--gpus", "2"], capture_output=True, text=True)
    assert two.returncode == 2 and "one GPU" in two.stderr and not two.stdout.strip()
    if not torch.cuda.is_available():
        one = subprocess.run([sys.executable, str(bench)], capture_output=True, text=True)
        assert one.returncode == 1 and "no GPU" in one.stderr and not one.stdout.strip()
