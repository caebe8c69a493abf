"""Parity of the Factorization-Memory layer around the scan (fm_memory, fm_layer: scan, RMS norm
over D, read-out over M, and every gradient) with the float64 CPU oracle of the same layer
(reference fm/scan/fm_scan.py:102-133, gradients by the chain rule), on an MI355X.

Both sides start from the same, already quantised inputs, and the oracle forms the gates and the
read weights where the reference's lines hold tensors of the storage dtype (fm_scan.py:116-119,130):
alpha * update_scale rounded, one minus that rounded again, alpha * output_scale rounded once. The
layer's prepare kernel gives the same bits (tests/test_gpu_parity.py::
test_layer_prepare_and_finish_kernels; the oracle's side is pinned against the PyTorch operations in
tests/test_oracle.py), so both sides scan with the reference's gates: stored in bfloat16 a gate near
one moves by up to 2^-9 per rounding, which is a different decay and not an error of the scan.
Errors are normwise,
    max|y - ref| / max|ref|   and   ||y - ref||_2 / ||ref||_2,
per returned quantity. Tolerances, with what they pay for:

  float32            1e-5 for every quantity (the benchmark's bar); measured below 1e-6.
  bfloat16/float16   1e-2 for every quantity (the benchmark's bar). The results of the forward
                     pass are one to three roundings of the storage type away from float32
                     arithmetic (states -> normalised states -> output); the gradients are made
                     from the stored normalised states, pass through the cancellation
                     dn - n * mean(dn * n) of the norm's gradient and through
                     (h[t-1] - x[t]) * delta of the scan's, and are rounded once on store.
                     Measured: up to 7e-3 in bfloat16, 1e-3 in float16. Values are printed.

The shapes take every branch of the layer's backward: both sums inside one kernel (M > 1, D > 1,
16-byte rows), M = 1, D = 1, D not a multiple of the 8 rows a block sums over, rows that are not
16-byte multiples (element access), rows shorter than a tile, a loss on the output alone and on
both results, with and without an initial state, and the routes that depend on how many blocks a
shape gives (scan and norm in one kernel or apart; the slots of a batch element in one block or several). D = 1 with the norm is run with eps of the order
of the squared states: for eps << h^2 that gradient is pure cancellation and no implementation
that stores the normalised states can deliver it (tests/test_oracle.py::
test_norm_gradient_with_one_channel_is_all_cancellation).
"""
import numpy as np
import pytest
import torch

import fm_scan_oracle as O

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
FWD_TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}
GRAD_TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}


@pytest.fixture(scope="module")
def scan():
    import fm.scan.fm_scan as m

    assert torch.cuda.is_available(), "these tests need the GPU"
    return m


def storage(dtype):
    """Rounds a float64 array to `dtype` and back."""
    return lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(torch.float64).numpy()


def errs(y, ref):
    y = y.detach().double().cpu().numpy().reshape(ref.shape)
    d = y - ref
    return (float(np.abs(d).max() / max(np.abs(ref).max(), 1e-300)),
            float(np.linalg.norm(d.ravel()) / max(np.linalg.norm(ref.ravel()), 1e-300)))


def check_all(tag, got, want, tols):
    worst = []
    for name in want:
        e_max, e_l2 = errs(got[name], want[name])
        print(f"{tag} {name}: max-norm {e_max:.2e} l2 {e_l2:.2e} (tolerance {tols[name]:g})", flush=True)
        if not (e_max <= tols[name] and e_l2 <= tols[name]):
            worst.append(f"{name}: max-norm {e_max:.3e}, l2 {e_l2:.3e} > {tols[name]:g}")
    assert not worst, f"{tag}: " + "; ".join(worst)


# (B, L, M, D), norm eps, what the shape is there for
LAYER_SHAPES = [
    ((2, 512, 4, 24), 1e-4, "both sums inside one kernel"),
    ((2, 304, 1, 16), 1e-4, "M = 1"),
    ((1, 7, 5, 1), 1.0, "D = 1, row shorter than 16 bytes"),
    ((2, 264, 3, 5), 1e-4, "D below the 8 rows of a block"),
    ((1, 1001, 3, 12), 1e-4, "rows that are not 16-byte multiples"),
    ((3, 40, 2, 9), 1e-4, "row shorter than a tile, ragged D"),
    ((1, 2048, 2, 130), 1e-4, "D beyond one block of the read-out"),
    ((64, 40, 3, 60), 1e-4, "enough blocks for groups of 8 rows in backward, the last group ragged"),
    ((16, 520, 5, 256), 1e-4, "groups of 8 rows, a ragged last tile, waves with one slot or none"),
    ((16, 264, 4, 24), 1e-4, "64 slots: scan and norm in one kernel, 8 waves of 4 rows"),
    ((1, 1032, 16, 20), 1e-4, "one batch element: separate kernels forward, slots dealt to four blocks backward"),
    ((1, 4104, 8, 24), 1e-4, "few slots, long rows: the sequence cut in 2 (4 in float32), in scan + norm and in backward"),
    ((2060, 24, 2, 20), 1e-4, "rows of at most 256 bytes, many batch elements: several rows to a wave in backward "
                              "(4 lanes a row in bfloat16, 8 in float32; D not a multiple of the rows of a wave)"),
    ((1400, 32, 3, 70), 1e-4, "the same with 4 / 8 lanes a row and three slots"),
    ((420, 200, 2, 20), 1e-4, "rows of 400 bytes in bfloat16: the read-out's kernels alone put two rows into a wave"),
]


def layer_inputs(shape, dtype, with_h0, seed):
    B, L, M, D = shape
    gen = torch.Generator().manual_seed(seed)
    q = lambda t: t.to(dtype).to(torch.float64)  # both sides start from the same quantised values
    alpha = q(torch.softmax(torch.randn(B, L, M, generator=gen, dtype=torch.float64), dim=-1))
    us = q(torch.rand(B, L, 1, generator=gen, dtype=torch.float64))
    osc = q(torch.rand(B, L, 1, generator=gen, dtype=torch.float64) + 0.5)
    inp = q(torch.randn(B, L, D, generator=gen, dtype=torch.float64))
    h0 = q(torch.randn(B, M, D, generator=gen, dtype=torch.float64)) if with_h0 else None
    w_out = q(torch.randn(B, L, D, generator=gen, dtype=torch.float64))
    w_mem = q(torch.randn(B, M, D, L, generator=gen, dtype=torch.float64) * 0.1)
    return alpha, us, osc, inp, h0, w_out, w_mem


@pytest.mark.parametrize("mem_in_loss", [False, True])
@pytest.mark.parametrize("mem_norm", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fm_memory_against_the_oracle(scan, dtype, mem_norm, mem_in_loss):
    for i, (shape, eps, why) in enumerate(LAYER_SHAPES):
        B, L, M, D = shape
        with_h0 = i % 2 == 0
        alpha, us, osc, inp, h0, w_out, w_mem = layer_inputs(shape, dtype, with_h0, seed=100 + i)
        leaves = [t.to(dtype).to(DEV).requires_grad_() for t in (alpha, us, osc, inp)]
        h0_gpu = None if h0 is None else h0.to(dtype).to(DEV).requires_grad_()
        y, mem = scan.fm_memory(*leaves, h0_gpu, mem_norm=mem_norm, norm_eps=eps)
        assert y.shape == (B, L, D) and mem.shape == (B, M, D, L) and y.is_contiguous()
        # a linear loss: its gradients with respect to the two results are w_out and w_mem exactly
        loss = (y.float() * w_out.to(DEV).float()).sum()
        if mem_in_loss:
            loss = loss + (mem.float() * w_mem.to(DEV).float()).sum()
        loss.backward()
        o_y, o_mem = O.memory_forward(alpha, us, osc, inp, h0, mem_norm, eps, storage(dtype))
        want = O.memory_backward(alpha, us, osc, inp, w_out, w_mem if mem_in_loss else None, h0, mem_norm, eps,
                                 storage(dtype))
        got = {"output": y, "memory_states": mem, "d_alpha": leaves[0].grad, "d_update_scale": leaves[1].grad,
               "d_output_scale": leaves[2].grad, "d_inputs": leaves[3].grad}
        want = dict(output=o_y, memory_states=o_mem, **want)
        if h0 is None:
            del want["d_initial_state"]
        else:
            got["d_initial_state"] = h0_gpu.grad
        tols = {k: (FWD_TOL if k in ("output", "memory_states") else GRAD_TOL)[dtype] for k in want}
        check_all(f"fm_memory {shape} ({why}) {dtype} norm={mem_norm} mem_in_loss={mem_in_loss} h0={with_h0}",
                  got, want, tols)


@pytest.mark.parametrize("mem_in_loss", [False, True])
@pytest.mark.parametrize("mem_norm", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_fm_layer_against_the_oracle(scan, dtype, mem_norm, mem_in_loss):
    """fm_layer: the same layer with time last (gates, read (B, M, L), tokens (B, D, L))."""
    for i, (shape, eps, why) in enumerate(LAYER_SHAPES):
        B, L, M, D = shape
        gen = torch.Generator().manual_seed(200 + i)
        q = lambda t: t.to(dtype).to(torch.float64)
        g = q(torch.sigmoid(torch.randn(B, M, L, generator=gen, dtype=torch.float64) + 2))
        x = q(torch.randn(B, D, L, generator=gen, dtype=torch.float64))
        read = q(torch.randn(B, M, L, generator=gen, dtype=torch.float64))
        h0 = q(torch.randn(B, M, D, generator=gen, dtype=torch.float64)) if i % 2 else None
        w_out = q(torch.randn(B, D, L, generator=gen, dtype=torch.float64))
        w_mem = q(torch.randn(B, M, D, L, generator=gen, dtype=torch.float64) * 0.1)
        leaves = [t.to(dtype).to(DEV).requires_grad_() for t in (g, x, read)]
        h0_gpu = None if h0 is None else h0.to(dtype).to(DEV).requires_grad_()
        y, mem = scan.fm_layer(leaves[0], leaves[1], h0_gpu, leaves[2], mem_norm, eps)
        loss = (y.float() * w_out.to(DEV).float()).sum()
        if mem_in_loss:
            loss = loss + (mem.float() * w_mem.to(DEV).float()).sum()
        loss.backward()
        states = O.forward(g, x, h0)
        o_y, o_mem, _ = O.readout_forward(states, read, mem_norm, eps)
        ext = w_mem.numpy() if mem_in_loss else None
        if mem_norm:
            d_states, d_read = O.readout_backward(w_out, ext, read, states, True, eps)
        else:
            d_states, d_read = O.readout_backward(w_out, None, read, states, False, eps)
            if ext is not None:
                d_states = d_states + ext
        d_g, d_x, d_h0 = O.backward(g, x, d_states, h0, states=states)
        got = {"output": y, "memory_states": mem, "d_gates": leaves[0].grad, "d_tokens": leaves[1].grad,
               "d_read": leaves[2].grad}
        want = {"output": o_y, "memory_states": o_mem, "d_gates": d_g, "d_tokens": d_x, "d_read": d_read}
        if h0 is not None:
            got["d_initial_state"], want["d_initial_state"] = h0_gpu.grad, d_h0
        tols = {k: (FWD_TOL if k in ("output", "memory_states") else GRAD_TOL)[dtype] for k in want}
        check_all(f"fm_layer {shape} ({why}) {dtype} norm={mem_norm} mem_in_loss={mem_in_loss}", got, want, tols)


def test_layer_at_the_benchmark_shape(scan):
    """fm_memory at the shape bench.py --workload layer times, (B, L, M, D) = (32, 2048, 32, 128)
    bfloat16 with the norm and a loss on the output: forward results and all four input gradients
    against the float64 oracle on batch elements 0 and B - 1 (the batch elements are independent)."""
    B, L, M, D, dt = 32, 2048, 32, 128, torch.bfloat16
    gen = torch.Generator(device=DEV).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=DEV, generator=gen)
    alpha = torch.softmax(rn(B, L, M), -1).to(dt).requires_grad_()
    us = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt).requires_grad_()
    osc = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt).requires_grad_()
    inp = rn(B, L, D).to(dt).requires_grad_()
    w_out = rn(B, L, D).to(dt)
    y, mem = scan.fm_memory(alpha, us, osc, inp)
    (y.float() * w_out.float()).sum().backward()
    torch.cuda.synchronize()
    for b in (0, B - 1):
        sel = lambda t: t.detach()[b:b + 1].double().cpu()
        a, u, o, x, w = (sel(t) for t in (alpha, us, osc, inp, w_out))
        o_y, o_mem = O.memory_forward(a, u, o, x, None, True, 1e-6, storage(dt))
        want = O.memory_backward(a, u, o, x, w, None, None, True, 1e-6, storage(dt))
        del want["d_initial_state"]
        want = dict(output=o_y, memory_states=o_mem, **want)
        got = {"output": y[b:b + 1], "memory_states": mem[b:b + 1], "d_alpha": alpha.grad[b:b + 1],
               "d_update_scale": us.grad[b:b + 1], "d_output_scale": osc.grad[b:b + 1], "d_inputs": inp.grad[b:b + 1]}
        tols = {k: (FWD_TOL if k in ("output", "memory_states") else GRAD_TOL)[dt] for k in want}
        check_all(f"fm_memory bench shape, batch element {b}", got, want, tols)


@pytest.mark.parametrize("shape", [(0, 64, 4, 8), (2, 64, 4, 0)])
def test_empty_problems_pass_through(scan, shape):
    """No batch element, or no channel: nothing to launch (the C ABI rejects empty problems, the
    Python side never calls it with one), the results are empty tensors of the right shapes and the
    gradients of what is not empty are zero."""
    B, L, M, D = shape
    dt = torch.bfloat16
    g = torch.rand(B, M, L, device=DEV).to(dt).requires_grad_()
    x = torch.randn(B, D, L, device=DEV).to(dt).requires_grad_()
    states = scan.fm_scan(g, x)
    assert tuple(states.shape) == (B, M, D, L)
    states.float().sum().backward()
    assert tuple(g.grad.shape) == (B, M, L) and tuple(x.grad.shape) == (B, D, L)
    assert not g.grad.float().abs().sum().item() and not x.grad.float().abs().sum().item()
    alpha = torch.softmax(torch.randn(B, L, M, device=DEV), -1).to(dt).requires_grad_()
    us = torch.rand(B, L, 1, device=DEV).to(dt).requires_grad_()
    osc = torch.rand(B, L, 1, device=DEV).to(dt).requires_grad_()
    inp = torch.randn(B, L, D, device=DEV).to(dt).requires_grad_()
    y, mem = scan.fm_memory(alpha, us, osc, inp)
    assert tuple(y.shape) == (B, L, D) and tuple(mem.shape) == (B, M, D, L)
    y.float().sum().backward()
    for t in (alpha, us, osc, inp):
        assert t.grad is not None and t.grad.shape == t.shape and not t.grad.float().abs().sum().item()


def test_layer_rejects_a_misplaced_initial_state(scan):
    """An initial state on the host, or of another dtype than the rest, is an error raised in Python
    (the fused forward route passes raw pointers: it must never reach a kernel), for shapes of both routes;
    a valid call still works afterwards."""
    for (B, L, M, D) in ((2, 512, 4, 24), (1, 1001, 3, 12)):
        dt = torch.bfloat16
        alpha = torch.softmax(torch.randn(B, L, M, device=DEV), -1).to(dt)
        us, osc = torch.rand(B, L, 1, device=DEV).to(dt), torch.rand(B, L, 1, device=DEV).to(dt)
        inp = torch.randn(B, L, D, device=DEV).to(dt)
        h0 = torch.randn(B, M, D, device=DEV)
        with pytest.raises(RuntimeError, match="initial_state has dtype"):
            scan.fm_memory(alpha, us, osc, inp, h0)  # float32 state, bfloat16 layer
        with pytest.raises(RuntimeError, match="GPU tensor"):
            scan.fm_memory(alpha, us, osc, inp, h0.to(dt).cpu())
        with pytest.raises(RuntimeError, match="initial_state must be"):
            scan.fm_memory(alpha, us, osc, inp, torch.zeros(B, M, D + 1, dtype=dt, device=DEV))
        y, mem = scan.fm_memory(alpha, us, osc, inp, h0.to(dt))
        assert torch.isfinite(y.float()).all() and torch.isfinite(mem.float()).all()


def test_layer_with_more_than_2_31_state_elements(scan):
    """(B, L, M, D) = (9, 65536, 32, 128): 2^31 + 2^28 elements of the states, which the reference's
    32-bit indices could not address (fm_scan.cuh:76-82). Batch elements are independent, so the last
    batch element, all of it beyond element 2^31, must come out as a layer call on that batch element
    alone does: to rounding, not bit for bit, since a single batch element takes other routes (scan and
    norm in separate kernels, its slots dealt to several blocks in backward) whose float32 sums run in
    another order. A wrong index would be an error of order one."""
    B, L, M, D, dt = 9, 65536, 32, 128, torch.bfloat16
    gen = torch.Generator(device=DEV).manual_seed(5)
    rn = lambda *s: torch.randn(*s, device=DEV, generator=gen)
    alpha = torch.softmax(rn(B, L, M), -1).to(dt)
    us = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt)
    osc = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt)
    inp = rn(B, L, D).to(dt)
    w_out = rn(B, L, D).to(dt)

    def run(sl):
        leaves = [t[sl].clone().requires_grad_() for t in (alpha, us, osc, inp)]
        y, mem = scan.fm_memory(*leaves)
        (y.float() * w_out[sl].float()).sum().backward()
        return [y.detach(), mem.detach()] + [t.grad for t in leaves]

    whole = run(slice(0, B))
    assert whole[1].numel() > 1 << 31
    last = [t[B - 1:].clone() for t in whole]
    del whole
    torch.cuda.empty_cache()
    alone = run(slice(B - 1, B))
    for name, a, b in zip(("output", "memory_states", "d_alpha", "d_update_scale", "d_output_scale", "d_inputs"),
                          last, alone):
        a, b = a.float(), b.float()
        differing = float((a != b).float().mean())
        err = float((a - b).norm() / b.norm())
        print(f"{name}: {differing:.2%} of the entries differ, {err:.1e} normwise")
        assert err < 1e-3, (name, err)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_forward_scan_and_norm_in_one_kernel(scan, dtype):
    """fmscan_forward_normed (through the C interface) against the float64 oracle and against the three
    separate calls it stands for; D up to the limit, ragged D and L, with and without initial state."""
    lib, st = scan.module, torch.cuda.current_stream().cuda_stream
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    limit = lib.fmscan_forward_normed_max_d()
    assert limit >= 128
    for (B, M, D, L), with_h0 in [((2, 3, 5, 512), True), ((1, 2, 33, 1000), False), ((2, 4, 64, 4096), True),
                                  ((1, 3, 128, 2056), True), ((3, 2, 100, 8), False), ((1, 1, 1, 2048), True)]:
        gen = torch.Generator().manual_seed(D * 10 + L)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV) if with_h0 else None
        eps = 1e-5
        normed = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        inv = torch.empty(B, M, L, device=DEV)
        rc = lib.fmscan_forward_normed(g.data_ptr(), x.data_ptr(), None if h0 is None else h0.data_ptr(),
                                       normed.data_ptr(), inv.data_ptr(), B, M, D, L, code, eps, st)
        assert rc == 0, lib.fmscan_last_error()
        states = O.forward(g, x, h0)
        _, o_normed, o_inv = O.readout_forward(states, np.ones((B, M, L)), True, eps)
        tag = f"{(B, M, D, L)} {dtype}"
        tol = FWD_TOL[dtype]
        check_all(tag, {"normalised states": normed, "inv_rms": inv}, {"normalised states": o_normed, "inv_rms": o_inv},
                  {"normalised states": tol, "inv_rms": tol})
        # the separate calls: scan, sum of squares, scaling
        z = torch.zeros(B, M, D, dtype=dtype, device=DEV)
        out = torch.empty_like(normed)
        scan.fm_scan_forward(g, x, z if h0 is None else h0, out)
        _, n3, r3 = scan.fm_readout_forward(out, torch.ones(B, M, L, dtype=dtype, device=DEV), True, eps)
        check_all(tag + " vs three calls", {"normalised states": normed, "inv_rms": inv},
                  {"normalised states": n3.double().cpu().numpy(), "inv_rms": r3.double().cpu().numpy()},
                  {"normalised states": tol, "inv_rms": 1e-5})
        # the sequence cut into segments (two passes): every number of segments the tiles allow up to 5,
        # against the oracle and against the uncut call (the state that enters a segment is composed from
        # step pairs instead of carried along: equal to float32 rounding before the states are stored)
        tile = 256 if dtype == torch.float32 else 512
        for segments in range(2, min(5, (L + tile - 1) // tile) + 1):
            ws = torch.empty(B * M * D * segments * 8, dtype=torch.uint8, device=DEV)
            cut_n, cut_inv = torch.full_like(normed, float("nan")), torch.full_like(inv, float("nan"))
            rc = lib.fmscan_forward_normed_cut(g.data_ptr(), x.data_ptr(), None if h0 is None else h0.data_ptr(),
                                               cut_n.data_ptr(), cut_inv.data_ptr(), B, M, D, L, code, eps, segments,
                                               ws.data_ptr(), ws.numel(), st)
            assert rc == 0, lib.fmscan_last_error()
            check_all(f"{tag} cut into {segments}", {"normalised states": cut_n, "inv_rms": cut_inv},
                      {"normalised states": o_normed, "inv_rms": o_inv}, {"normalised states": tol, "inv_rms": tol})
            check_all(f"{tag} cut into {segments} vs uncut", {"normalised states": cut_n, "inv_rms": cut_inv},
                      {"normalised states": normed.double().cpu().numpy(), "inv_rms": inv.double().cpu().numpy()},
                      {"normalised states": tol, "inv_rms": 1e-5})
    # beyond the limit and unaligned: rejected, nothing launched
    D = limit + 1
    g = torch.rand(1, 1, 64, device=DEV); x = torch.rand(1, D, 64, device=DEV)
    n = torch.empty(1, 1, D, 64, device=DEV); r = torch.empty(1, 1, 64, device=DEV)
    assert lib.fmscan_forward_normed(g.data_ptr(), x.data_ptr(), None, n.data_ptr(), r.data_ptr(), 1, 1, D, 64, 0,
                                     1e-6, st) == -2
    assert lib.fmscan_forward_normed(g.data_ptr(), x.data_ptr(), None, n.data_ptr(), r.data_ptr(), 1, 1, 4, 63, 0,
                                     1e-6, st) == -7


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_scan_and_norm_several_rows_to_a_wave(scan, dtype):
    """fmscan_forward_normed on rows of at most 256 bytes with 4096 slots or more: the kernel that puts several
    rows into a wave and gives a slot a wave. Groups of 1 to 16 lanes, D that is not a multiple of the rows of
    a wave, 2 to 32 tiles a slot (the three register budgets), with and without initial state; against the
    three separate calls on everything, and against the float64 oracle on the first and last batch elements."""
    lib, st = scan.module, torch.cuda.current_stream().cuda_stream
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    E = 4 if dtype == torch.float32 else 8
    for chunks, M, D, with_h0 in ((1, 2, 70, True), (3, 3, 40, False), (5, 2, 128, True), (8, 4, 33, False),
                                  (16, 2, 100, True), (12, 3, 128, False)):
        L = chunks * E
        B = -(-4096 // M) + 1
        gen = torch.Generator().manual_seed(500 + chunks)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV) if with_h0 else None
        eps = 1e-5
        normed = torch.full((B, M, D, L), float("nan"), dtype=dtype, device=DEV)
        inv = torch.full((B, M, L), float("nan"), device=DEV)
        rc = lib.fmscan_forward_normed(g.data_ptr(), x.data_ptr(), None if h0 is None else h0.data_ptr(),
                                       normed.data_ptr(), inv.data_ptr(), B, M, D, L, code, eps, st)
        assert rc == 0, lib.fmscan_last_error()
        tag = f"{(B, M, D, L)} {dtype}"
        tol = FWD_TOL[dtype]
        z = torch.zeros(B, M, D, dtype=dtype, device=DEV)
        out = torch.empty_like(normed)
        scan.fm_scan_forward(g, x, z if h0 is None else h0, out)
        _, n3, r3 = scan.fm_readout_forward(out, torch.ones(B, M, L, dtype=dtype, device=DEV), True, eps)
        check_all(tag + " vs three calls", {"normalised states": normed, "inv_rms": inv},
                  {"normalised states": n3.double().cpu().numpy(), "inv_rms": r3.double().cpu().numpy()},
                  {"normalised states": tol, "inv_rms": 1e-5})
        sel = torch.tensor([0, 1, 2, B - 2, B - 1], device=DEV)
        states = O.forward(g[sel], x[sel], None if h0 is None else h0[sel])
        _, o_normed, o_inv = O.readout_forward(states, np.ones((len(sel), M, L)), True, eps)
        check_all(tag, {"normalised states": normed[sel], "inv_rms": inv[sel]},
                  {"normalised states": o_normed, "inv_rms": o_inv}, {"normalised states": tol, "inv_rms": tol})


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_forward_scan_with_the_sums_of_squares(scan, dtype):
    """fmscan_forward_sumsq + fmscan_sumsq_finish (any D: the scan leaves the sums of squares over blocks
    of 128 rows) against the float64 oracle, and against fmscan_forward + fmscan_readout_inv_rms."""
    lib, st = scan.module, torch.cuda.current_stream().cuda_stream
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    for (B, M, D, L), with_h0 in [((1, 2, 300, 1024), True), ((2, 3, 129, 520), False), ((1, 3, 1024, 4096), True),
                                  ((2, 2, 5, 64), False)]:
        gen = torch.Generator().manual_seed(D + L)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV) if with_h0 else None
        groups = lib.fmscan_sumsq_groups(D)
        assert groups == (D + 127) // 128
        states = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        partial = torch.full((B, M, groups, L), float("nan"), device=DEV)
        inv = torch.empty(B, M, L, device=DEV)
        assert lib.fmscan_forward_sumsq(g.data_ptr(), x.data_ptr(), None if h0 is None else h0.data_ptr(),
                                        states.data_ptr(), partial.data_ptr(), B, M, D, L, code, st) == 0, \
            lib.fmscan_last_error()
        assert lib.fmscan_sumsq_finish(partial.data_ptr(), groups, inv.data_ptr(), B, M, D, L, 1e-5, st) == 0
        tag = f"{(B, M, D, L)} {dtype}"
        o_states = O.forward(g, x, h0)
        _, _, o_inv = O.readout_forward(o_states, np.ones((B, M, L)), True, 1e-5)
        check_all(tag, {"states": states, "inv_rms": inv}, {"states": o_states, "inv_rms": o_inv},
                  {"states": FWD_TOL[dtype], "inv_rms": FWD_TOL[dtype]})
        z = torch.zeros(B, M, D, dtype=dtype, device=DEV)
        ref = torch.empty_like(states)
        scan.fm_scan_forward(g, x, z if h0 is None else h0, ref)
        assert torch.equal(ref, states), tag + ": the states differ from fmscan_forward's"
        _, _, r3 = scan.fm_readout_forward(ref, torch.ones(B, M, L, dtype=dtype, device=DEV), True, 1e-5)
        check_all(tag + " vs the separate sum", {"inv_rms": inv}, {"inv_rms": r3.double().cpu().numpy()}, {"inv_rms": 1e-5})
