"""fmscan_forward_static — the forward entry point that allocates nothing: the pairs that carry
the state between the segments of a cut row live in a static device array of the library
instead of a caller's workspace — against fmscan_forward with a workspace, through the C ABI.
Same kernels, same plan: the results must be bit-identical. Two calls in a row, the second on a
smaller problem (the array keeps the first call's pairs)."""
import pytest
import torch

import fmscan_cpu as C

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


@pytest.fixture(scope="module")
def lib():
    import fm.scan.fm_scan as m

    assert torch.cuda.is_available(), "these tests need the GPU"
    return m.module


def problem(B, M, D, L, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 3).to(dtype).to(DEV)
    x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
    h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
    return g, x, h0


def both_ways(lib, shape, dtype, seed, flags=0):
    B, M, D, L = shape
    g, x, h0 = problem(B, M, D, L, dtype, seed)
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.fmscan_workspace_bytes(B, M, D, L, CODE[dtype], flags)
    assert need > 0, "the case is meant to cut its rows into segments"
    ws = torch.empty(need, dtype=torch.uint8, device=DEV)
    want = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
    rc = lib.fmscan_forward(g.data_ptr(), x.data_ptr(), h0.data_ptr(), want.data_ptr(), B, M, D, L, CODE[dtype],
                            flags, ws.data_ptr(), need, stream)
    assert rc == 0, lib.fmscan_last_error()
    got = torch.full_like(want, float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.fmscan_forward_static(g.data_ptr(), x.data_ptr(), h0.data_ptr(), got.data_ptr(), B, M, D, L,
                                   CODE[dtype], flags, stream)
    assert rc == 0, lib.fmscan_last_error()
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(got, want), f"{shape} {dtype}: differs from fmscan_forward"
    # and both are the scan: float64 oracle on the same quantised inputs
    ref = C.forward_f64(g, x, h0)
    err = (got.double().cpu() - torch.from_numpy(ref)).abs().max().item() / abs(ref).max()
    assert err <= (1e-5 if dtype == torch.float32 else 1e-2), err


def test_static_workspace_matches_the_callers_workspace(lib):
    # two calls in a row, the second smaller: what the first left in the array must not matter
    both_ways(lib, (3, 1, 1, 131072), torch.bfloat16, seed=1)
    both_ways(lib, (2, 1, 1, 40000), torch.bfloat16, seed=2)
    # a requested cut, another dtype, ragged length; then a problem whose rows are not cut at all
    both_ways(lib, (5, 1, 3, 8200), torch.float32, seed=3, flags=7 << 20)
    B, M, D, L = 64, 1, 1, 4096
    g, x, h0 = problem(B, M, D, L, torch.float32, 4)
    a, b = (torch.empty(B, M, D, L, device=DEV) for _ in range(2))
    st = torch.cuda.current_stream().cuda_stream
    assert lib.fmscan_forward(g.data_ptr(), x.data_ptr(), h0.data_ptr(), a.data_ptr(), B, M, D, L, 0, 0, None, 0, st) == 0
    assert lib.fmscan_forward_static(g.data_ptr(), x.data_ptr(), h0.data_ptr(), b.data_ptr(), B, M, D, L, 0, 0, st) == 0
    torch.cuda.synchronize()
    assert torch.equal(a, b)


def test_static_workspace_rejects_cuts_beyond_its_size(lib):
    B, M, D, L = 300, 1, 1, 131072  # 300 rows x 255 segments = 76500 pairs, the array holds 8192
    g, x, h0 = problem(B, M, D, L, torch.bfloat16, 5)
    out = torch.empty(B, M, D, L, dtype=torch.bfloat16, device=DEV)
    rc = lib.fmscan_forward_static(g.data_ptr(), x.data_ptr(), h0.data_ptr(), out.data_ptr(), B, M, D, L, 2,
                                   255 << 20, torch.cuda.current_stream().cuda_stream)
    assert rc == -6 and b"workspace" in lib.fmscan_last_error()
