"""Pins the CPU oracle (oracle/fm_scan_oracle.py, oracle/fmscan_cpu.c) without the
reference: exact rational vectors, closed forms, library routines, finite
differences and structural identities. Each check is chosen so that a plausible
slip (dropped (1-g) factor, gate shifted the wrong way, h[t] in place of h[t-1],
wrong reduction axis, transposed row mapping) fails it.
"""
import numpy as np
import pytest
import torch
from scipy.signal import lfilter

import fm_scan_oracle as O
import fmscan_cpu as C


def rng(seed=0):
    return np.random.default_rng(seed)


def rand_problem(B, M, D, L, seed=0, state=True):
    r = rng(seed)
    g = r.random((B, M, L))
    x = r.standard_normal((B, D, L))
    G = r.standard_normal((B, M, D, L))
    h0 = r.standard_normal((B, M, D)) if state else None
    fpg = r.standard_normal((B, M, D)) if state else None
    return g, x, G, h0, fpg


# ------------------------------------------------------------------ exact vectors

CASES = ["fm_zero_state", "fm_with_state", "fm_single_row", "fm_length_one", "plain_with_state",
         "fm_gates_outside_unit_interval", "fm_vector_rows", "plain_vector_rows"]


@pytest.mark.parametrize("name", CASES)
@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_exact_rational_vectors(exact_cases, name, impl):
    c = exact_cases[name]
    a = lambda k: np.array(c[k], dtype=np.float64)
    g, x, G, h0, fpg = a("gates"), a("tokens"), a("out_grad"), a("initial_state"), a("first_prop_grad")
    plain = c["plain"]
    if impl == "numpy":
        h = O.forward(g, x, h0, plain)
        tg, gg, delta = O.backward_per_row(g, G, h, x, fpg, h0, plain)
    else:
        h = C.forward_f64(g, x, h0, plain)
        tg, gg = C.backward_f64(g, G, h, x, fpg, h0, plain)
    np.testing.assert_allclose(h, a("states"), rtol=1e-14, atol=1e-14)
    np.testing.assert_allclose(tg, a("token_grad"), rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(gg, a("gate_grad"), rtol=1e-13, atol=1e-13)
    if impl == "numpy":
        d_g, d_x, d_h0 = O.backward(g, x, G, h0, plain, first_prop_grad=fpg)
        np.testing.assert_allclose(d_g, a("gate_grad").sum(axis=2), rtol=1e-13, atol=1e-13)
        np.testing.assert_allclose(d_x, a("token_grad").sum(axis=1), rtol=1e-13, atol=1e-13)
        np.testing.assert_allclose(d_h0, a("d_initial_state"), rtol=1e-13, atol=1e-13)


# ------------------------------------------------------------------ closed forms, forward

def test_constant_gate_unit_input_is_geometric_series():
    L, a = 40, 0.8
    h = O.forward(np.full((1, 1, L), a), np.ones((1, 1, L)))
    np.testing.assert_allclose(h[0, 0, 0], 1.0 - a ** np.arange(1, L + 1), rtol=1e-13)


@pytest.mark.parametrize("plain", [False, True])
def test_constant_gate_matches_iir_filter(plain):
    L, a = 200, 0.93
    x = rng(1).standard_normal(L)
    h0 = 0.7
    h = O.forward(np.full((1, 1, L), a), x[None, None], np.full((1, 1, 1), h0), plain)[0, 0, 0]
    b = [1.0] if plain else [1.0 - a]
    ref, _ = lfilter(b, [1.0, -a], x, zi=[a * h0])
    np.testing.assert_allclose(h, ref, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(C.forward_f64(np.full((1, 1, L), a), x[None, None], np.full((1, 1, 1), h0), plain)
                               [0, 0, 0], ref, rtol=1e-12, atol=1e-12)


def test_plain_unit_gate_is_cumulative_sum():
    x = rng(2).standard_normal((2, 3, 50))
    h = O.forward(np.ones((2, 1, 50)), x, None, plain=True)
    np.testing.assert_allclose(h[:, 0], np.cumsum(x, axis=2), rtol=1e-13, atol=1e-13)


def test_reset_hold_and_fixed_point():
    r = rng(3)
    x = r.standard_normal((2, 3, 17))
    h0 = r.standard_normal((2, 2, 3))
    # gate 0: the state is the token, for every memory row
    h = O.forward(np.zeros((2, 2, 17)), x, h0)
    assert np.array_equal(h, np.broadcast_to(x[:, None], h.shape))
    # gate 1: the state never moves
    h = O.forward(np.ones((2, 2, 17)), x, h0)
    assert np.array_equal(h, np.broadcast_to(h0[..., None], h.shape))
    # tokens == state == c: convex combination keeps c whatever the gates are
    g = r.random((2, 2, 17))
    h = O.forward(g, np.full((2, 3, 17), 0.25), np.full((2, 2, 3), 0.25))
    np.testing.assert_allclose(h, 0.25, rtol=1e-14)


def test_convexity_bounds():
    g, x, _, _, _ = rand_problem(2, 2, 3, 64, seed=4, state=False)
    h = O.forward(g, x)
    hi = np.maximum.accumulate(np.maximum(x, 0.0), axis=2)[:, None]
    lo = np.minimum.accumulate(np.minimum(x, 0.0), axis=2)[:, None]
    assert np.all(h <= hi + 1e-12) and np.all(h >= lo - 1e-12)


def test_row_mapping_against_scalar_loops():
    """(B, M, D) broadcasting: every output row equals the one-row scan of its own
    gate row b*M+m and token row b*D+d, written as a scalar Python loop."""
    g, x, _, h0, _ = rand_problem(2, 3, 4, 11, seed=5)
    h = O.forward(g, x, h0)
    hc = C.forward_f64(g, x, h0)
    for b in range(2):
        for m in range(3):
            for d in range(4):
                s = h0[b, m, d]
                for t in range(11):
                    s = g[b, m, t] * s + (1.0 - g[b, m, t]) * x[b, d, t]
                    assert abs(h[b, m, d, t] - s) < 1e-14
                    assert abs(hc[b, m, d, t] - s) < 1e-14


def test_segment_chaining_and_linearity():
    g, x, _, h0, _ = rand_problem(2, 2, 2, 64, seed=6)
    h = O.forward(g, x, h0)
    first = O.forward(g[..., :24], x[..., :24], h0)
    second = O.forward(g[..., 24:], x[..., 24:], first[..., -1])
    np.testing.assert_allclose(np.concatenate([first, second], axis=3), h, rtol=1e-14, atol=1e-14)
    x2 = rng(7).standard_normal(x.shape)
    h2 = O.forward(g, x2, 0 * h0)
    np.testing.assert_allclose(O.forward(g, 2 * x - 3 * x2, 2 * h0), 2 * h - 3 * h2, rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ backward

def fd_grad(f, a, eps=1e-6):
    out = np.zeros_like(a)
    it = np.nditer(a, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        old = a[i]
        a[i] = old + eps
        fp = f()
        a[i] = old - eps
        fm = f()
        a[i] = old
        out[i] = (fp - fm) / (2 * eps)
    return out


@pytest.mark.parametrize("plain", [False, True])
def test_backward_matches_finite_differences(plain):
    g, x, G, h0, _ = rand_problem(2, 2, 3, 7, seed=8)
    loss = lambda: float((G * O.forward(g, x, h0, plain)).sum())
    d_g, d_x, d_h0 = O.backward(g, x, G, h0, plain)
    np.testing.assert_allclose(d_g, fd_grad(loss, g), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(d_x, fd_grad(loss, x), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(d_h0, fd_grad(loss, h0), rtol=1e-6, atol=1e-7)


def test_backward_constant_gate_closed_form():
    # G == 1, constant gate a: delta[t] = (1 - a^(L-t)) / (1 - a)
    L, a = 30, 0.9
    g = np.full((1, 1, L), a)
    x = rng(9).standard_normal((1, 1, L))
    h = O.forward(g, x)
    tg, gg, delta = O.backward_per_row(g, np.ones((1, 1, 1, L)), h, x)
    expect = (1.0 - a ** (L - np.arange(L))) / (1.0 - a)
    np.testing.assert_allclose(delta[0, 0, 0], expect, rtol=1e-12)
    np.testing.assert_allclose(tg[0, 0, 0], (1.0 - a) * expect, rtol=1e-12)
    hprev = np.concatenate([[0.0], h[0, 0, 0, :-1]])
    np.testing.assert_allclose(gg[0, 0, 0], (hprev - x[0, 0]) * expect, rtol=1e-12)


def test_adjoint_identity():
    """Forward is linear in the tokens: <G, J v> == <J^T G, v>."""
    g, x, G, _, _ = rand_problem(2, 3, 2, 33, seed=10, state=False)
    v = rng(11).standard_normal(x.shape)
    _, d_x, _ = O.backward(g, x, G)
    lhs = float((G * O.forward(g, v)).sum())
    np.testing.assert_allclose(lhs, float((d_x * v).sum()), rtol=1e-12)


def test_first_prop_grad_chains_segments():
    """Backward over [0, L) equals backward over the second half, then the first half
    fed with the gradient that crosses the cut (g[k] * delta[k])."""
    g, x, G, h0, _ = rand_problem(1, 2, 2, 32, seed=12)
    h = O.forward(g, x, h0)
    tg, gg, delta = O.backward_per_row(g, G, h, x, None, h0)
    k = 20
    tg2, gg2, d2 = O.backward_per_row(g[..., k:], G[..., k:], h[..., k:], x[..., k:], None, h[..., k - 1])
    cross = g[:, :, k][:, :, None] * d2[..., 0]
    tg1, gg1, _ = O.backward_per_row(g[..., :k], G[..., :k], h[..., :k], x[..., :k], cross, h0)
    np.testing.assert_allclose(np.concatenate([tg1, tg2], 3), tg, rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(np.concatenate([gg1, gg2], 3), gg, rtol=1e-13, atol=1e-13)


def test_kernel_literal_mode_differs_only_at_first_step():
    """Without an initial state handed to backward the reference kernel takes
    first_prop_grad as h[-1]: only gate_grad[..., 0] changes, by (h0 - fpg) * delta[0]."""
    g, x, G, h0, fpg = rand_problem(2, 2, 2, 9, seed=13)
    h = O.forward(g, x, h0)
    tg_e, gg_e, delta = O.backward_per_row(g, G, h, x, fpg, h0)
    tg_k, gg_k, _ = O.backward_per_row(g, G, h, x, fpg, None)
    assert np.array_equal(tg_e, tg_k)
    assert np.array_equal(gg_e[..., 1:], gg_k[..., 1:])
    np.testing.assert_allclose(gg_e[..., 0] - gg_k[..., 0], (h0 - fpg) * delta[..., 0], rtol=1e-13)
    tc, gc = C.backward_f64(g, G, h, x, fpg, None)
    np.testing.assert_allclose(gc, gg_k, rtol=1e-14, atol=1e-14)


def test_torch_loop_autograd_agrees_with_oracle():
    """The per-timestep PyTorch form (product module fm_amd.scan.fm_pytorch, the
    counterpart of the reference's CPU path) differentiated by autograd gives the
    oracle's analytic gradients, the one for the initial state included."""
    from fm_amd.scan.fm_pytorch import fm_scan_pytorch

    g, x, G, h0, _ = rand_problem(2, 3, 4, 19, seed=14)
    tg = torch.tensor(g, requires_grad=True)
    tx = torch.tensor(x, requires_grad=True)
    th = torch.tensor(h0, requires_grad=True)
    states = fm_scan_pytorch(tg, tx, th)
    np.testing.assert_allclose(states.detach().numpy(), O.forward(g, x, h0), rtol=1e-13, atol=1e-13)
    (states * torch.tensor(G)).sum().backward()
    d_g, d_x, d_h0 = O.backward(g, x, G, h0)
    np.testing.assert_allclose(tg.grad.numpy(), d_g, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(tx.grad.numpy(), d_x, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(th.grad.numpy(), d_h0, rtol=1e-12, atol=1e-12)


# ------------------------------------------------------------------ read-out of the layer

def rand_readout(B, M, D, L, seed):
    rng = np.random.default_rng(seed)
    return (rng.standard_normal((B, M, D, L)), rng.standard_normal((B, M, L)),
            rng.standard_normal((B, D, L)), rng.standard_normal((B, M, D, L)))


def test_readout_forward_brute_force_and_invariants():
    states, read, _, _ = rand_readout(2, 3, 4, 5, seed=21)
    eps = 1e-3
    out, normed, inv_rms = O.readout_forward(states, read, True, eps)
    B, M, D, L = states.shape
    for b in range(B):          # scalar loops straight from the formulas
        for t in range(L):
            for d in range(D):
                acc = 0.0
                for m in range(M):
                    ms = sum(states[b, m, k, t] ** 2 for k in range(D)) / D
                    acc += read[b, m, t] * states[b, m, d, t] / (ms + eps) ** 0.5
                assert abs(acc - out[b, d, t]) < 1e-12
    # eps = 0: unit mean square per slot and step, and invariance to the scale of the states
    out0, normed0, _ = O.readout_forward(states, read, True, 0.0)
    np.testing.assert_allclose((normed0 ** 2).mean(axis=2), 1.0, rtol=1e-13)
    out1, _, _ = O.readout_forward(3.7 * states, read, True, 0.0)
    np.testing.assert_allclose(out1, out0, rtol=1e-12, atol=1e-13)
    # D = 1, eps = 0: the norm leaves the sign
    s1, r1, _, _ = rand_readout(2, 3, 1, 6, seed=22)
    o1, n1, _ = O.readout_forward(s1, r1, True, 0.0)
    np.testing.assert_allclose(n1, np.sign(s1), rtol=1e-13)
    np.testing.assert_allclose(o1[:, 0, :], (r1 * np.sign(s1[:, :, 0, :])).sum(axis=1), rtol=1e-12, atol=1e-13)
    # no norm, read == 1: the plain sum over the slots
    o2, n2, r2 = O.readout_forward(states, np.ones_like(read), False)
    assert r2 is None and n2 is not None
    np.testing.assert_allclose(o2, states.sum(axis=1), rtol=1e-13, atol=1e-13)


@pytest.mark.parametrize("mem_norm", [True, False])
@pytest.mark.parametrize("with_ext", [False, True])
def test_readout_backward_matches_finite_differences(mem_norm, with_ext):
    states, read, out_grad, ext = rand_readout(2, 3, 4, 5, seed=23)
    ext = ext if with_ext else None
    eps = 1e-2

    def loss():
        out, normed, _ = O.readout_forward(states, read, mem_norm, eps)
        return float((out * out_grad).sum() + ((normed * ext).sum() if with_ext else 0.0))

    d_states, d_read = O.readout_backward(out_grad, ext, read, states, mem_norm, eps)
    np.testing.assert_allclose(d_states, fd_grad(loss, states), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(d_read, fd_grad(loss, read), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("mem_norm", [True, False])
def test_memory_layer_agrees_with_the_operations_the_reference_names(mem_norm):
    """fm_memory written with the PyTorch operations of fm_scan.py:115-133 (the scan through
    the per-timestep form) and differentiated by autograd: same outputs and gradients as the
    oracle's layer, read-out gradients included."""
    from fm_amd.scan.fm_pytorch import fm_scan_pytorch

    rng = np.random.default_rng(24)
    B, L, M, D = 2, 9, 3, 4
    alpha = rng.random((B, L, M))
    us, osc = rng.random((B, L, 1)), rng.standard_normal((B, L, 1))
    x = rng.standard_normal((B, L, D))
    h0 = rng.standard_normal((B, M, D))
    w_out, w_mem = rng.standard_normal((B, L, D)), rng.standard_normal((B, M, D, L))
    t = {k: torch.tensor(v, requires_grad=True) for k, v in dict(alpha=alpha, us=us, osc=osc, x=x, h0=h0).items()}
    write = (t["alpha"] * t["us"]).transpose(1, 2).contiguous()
    states = fm_scan_pytorch(1.0 - write, t["x"].transpose(1, 2).contiguous(), t["h0"])
    raw = states
    if mem_norm:
        states = states * torch.rsqrt(torch.mean(states ** 2, dim=2, keepdim=True) + 1e-3)
    out = torch.einsum("blm,bmdl->bld", t["alpha"] * t["osc"], states)
    o_out, o_states = O.memory_forward(alpha, us, osc, x, h0, mem_norm, 1e-3)
    np.testing.assert_allclose(out.detach().numpy(), o_out, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(states.detach().numpy(), o_states, rtol=1e-12, atol=1e-12)

    raw.retain_grad()
    ((out * torch.tensor(w_out)).sum() + (states * torch.tensor(w_mem)).sum()).backward()
    read = np.ascontiguousarray(np.transpose(alpha * osc, (0, 2, 1)))
    d_states, d_read = O.readout_backward(np.transpose(w_out, (0, 2, 1)), w_mem, read, raw.detach().numpy(),
                                          mem_norm, 1e-3)
    np.testing.assert_allclose(raw.grad.numpy(), d_states, rtol=1e-11, atol=1e-12)
    # d read reaches alpha and output_scale: d osc[b,l] = sum_m alpha * d_read, checked through osc
    d_osc = (np.transpose(d_read, (0, 2, 1)) * alpha).sum(axis=2, keepdims=True)
    np.testing.assert_allclose(t["osc"].grad.numpy(), d_osc, rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("mem_norm", [True, False])
@pytest.mark.parametrize("loss_on", ["output", "memory", "both"])
def test_memory_backward_against_autograd_and_finite_differences(mem_norm, loss_on):
    """The oracle's gradients of the whole layer against (i) autograd through the PyTorch operations
    fm_scan.py:115-133 names, in float64, and (ii) central finite differences of the oracle's own
    forward: every input, with a non-zero initial state, for a loss on either result or both."""
    from fm_amd.scan.fm_pytorch import fm_scan_pytorch

    rng = np.random.default_rng(31)
    B, L, M, D = 2, 7, 3, 4
    alpha = rng.random((B, L, M))
    us, osc = rng.random((B, L, 1)), rng.standard_normal((B, L, 1))
    x, h0 = rng.standard_normal((B, L, D)), rng.standard_normal((B, M, D))
    w_out = rng.standard_normal((B, L, D)) if loss_on != "memory" else None
    w_mem = rng.standard_normal((B, M, D, L)) if loss_on != "output" else None
    eps = 1e-2
    got = O.memory_backward(alpha, us, osc, x, w_out, w_mem, h0, mem_norm, eps)

    t = [torch.tensor(v, requires_grad=True) for v in (alpha, us, osc, x, h0)]
    write = (t[0] * t[1]).transpose(1, 2).contiguous()
    states = fm_scan_pytorch(1.0 - write, t[3].transpose(1, 2).contiguous(), t[4])
    if mem_norm:
        states = states * torch.rsqrt(torch.mean(states ** 2, dim=2, keepdim=True) + eps)
    out = torch.einsum("blm,bmdl->bld", t[0] * t[2], states)
    loss = 0.0
    if w_out is not None:
        loss = loss + (out * torch.tensor(w_out)).sum()
    if w_mem is not None:
        loss = loss + (states * torch.tensor(w_mem)).sum()
    loss.backward()
    names = ("d_alpha", "d_update_scale", "d_output_scale", "d_inputs", "d_initial_state")
    for name, leaf in zip(names, t):
        want = np.zeros(leaf.shape) if leaf.grad is None else leaf.grad.numpy()  # output_scale without the output
        np.testing.assert_allclose(got[name], want, rtol=1e-10, atol=1e-11, err_msg=name)

    def f():
        o, m = O.memory_forward(alpha, us, osc, x, h0, mem_norm, eps)
        return float((0.0 if w_out is None else (o * w_out).sum()) + (0.0 if w_mem is None else (m * w_mem).sum()))

    for name, arr in zip(names, (alpha, us, osc, x, h0)):
        np.testing.assert_allclose(got[name], fd_grad(f, arr), rtol=2e-6, atol=1e-7, err_msg=name)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_layer_operands_round_where_the_reference_holds_a_tensor(dtype):
    """The `storage=` branch of the oracle's layer: gates and read weights bit for bit what the PyTorch
    operations of fm_scan.py:116-119,130 give on tensors of the storage type,
        update_weight = alpha * update_scale; update_weight.transpose(1, 2).contiguous();
        decay_weight = 1.0 - update_weight;  output_weight = alpha * output_scale
    (evaluated here by PyTorch on CPU tensors, not retyped): the product is a tensor of its own, so the
    gate is rounded twice. The single-rounded gate round(1 - alpha * update_scale) must differ from it
    somewhere in the 16-bit types, or this test could not tell the two orders apart."""
    gen = torch.Generator().manual_seed(7)
    B, L, M = 3, 257, 32
    alpha = torch.softmax(torch.randn(B, L, M, generator=gen), -1).to(dtype)
    us = torch.rand(B, L, 1, generator=gen).to(dtype)
    osc = torch.rand(B, L, 1, generator=gen).to(dtype)
    want_gates = 1.0 - (alpha * us).transpose(1, 2).contiguous()
    want_read = (alpha * osc).transpose(1, 2).contiguous()
    assert want_gates.dtype == dtype and want_read.dtype == dtype

    storage = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(torch.float64).numpy()
    x = np.zeros((B, L, 1))
    gates, _, read = O._layer_operands(O.to_f64(alpha), O.to_f64(us), O.to_f64(osc), x, storage)
    assert np.array_equal(gates, want_gates.double().numpy())
    assert np.array_equal(read, want_read.double().numpy())

    once = storage(1.0 - np.transpose(O.to_f64(alpha) * O.to_f64(us), (0, 2, 1)))
    differ = np.mean(once != gates)
    if dtype != torch.float32:
        assert 1e-3 < differ < 0.1, differ  # about one gate in a hundred, each by one unit in the last place
    # without `storage` nothing is rounded: the float64 layer the other tests pin
    g64, _, r64 = O._layer_operands(O.to_f64(alpha), O.to_f64(us), O.to_f64(osc), x, None)
    assert np.array_equal(g64, 1.0 - np.transpose(O.to_f64(alpha) * O.to_f64(us), (0, 2, 1)))
    assert np.array_equal(r64, np.transpose(O.to_f64(alpha) * O.to_f64(osc), (0, 2, 1)))


def test_norm_gradient_with_one_channel_is_all_cancellation():
    """D = 1: the norm maps a state to n = h / sqrt(h^2 + eps), close to its sign, and the
    gradient that comes back through it is r * dn * (1 - n^2) = r * dn * eps / (h^2 + eps): what
    is left of dn after a cancellation to one part in (h^2 + eps) / eps. Made from normalised
    states that were stored in bfloat16 (spacing 2^-8 below one) or float32 (2^-24), the factor
    1 - n^2 is rounding noise unless eps is of the order of h^2: an implementation that keeps the
    normalised states (this one does; the reference's autograd keeps the bfloat16 factors of the
    same product) cannot do better there. With D >= 2 the part of dn across n survives and the
    same rounding is harmless."""
    rng = np.random.default_rng(5)
    B, M, L = 1, 5, 64
    read, out_grad = rng.standard_normal((B, M, L)), None

    def grad_from_stored(states, eps, quantum):
        D = states.shape[2]
        og = rng.standard_normal((B, D, L))
        exact, _ = O.readout_backward(og, None, read, states, True, eps)
        _, n, r = O.readout_forward(states, read, True, eps)
        n_stored = np.round(n / quantum) * quantum            # the stored, rounded normalised states
        dn = read[:, :, None, :] * og[:, None, :, :]
        approx = r[:, :, None, :] * (dn - n_stored * np.mean(dn * n_stored, axis=2, keepdims=True))
        return np.abs(approx - exact).max() / np.abs(exact).max()

    h1 = rng.standard_normal((B, M, 1, L)) + 3.0 * np.sign(rng.standard_normal((B, M, 1, L)))
    assert grad_from_stored(h1, 1e-6, 2.0 ** -8) > 0.5       # bfloat16, eps << h^2: n rounds to +-1, nothing is left
    assert grad_from_stored(h1, 1e-6, 2.0 ** -24) > 1e-3     # float32 too, against a 1e-5 bar
    assert grad_from_stored(h1, 16.0, 2.0 ** -8) < 1e-2      # eps of the order of h^2: fine
    h4 = rng.standard_normal((B, M, 4, L))
    assert grad_from_stored(h4, 1e-6, 2.0 ** -8) < 1e-2      # D = 4: fine with the same rounding


def test_single_step_gate_gradient_vanishes_under_the_norm():
    """L = 1 without an initial state: the one state is (1 - g) x, the norm makes the output blind to
    its length, so the gradient that reaches the gate (and with it update_scale) is what eps lets
    through: zero up to eps / mean(h^2), a difference of terms of order one. Against a reference that
    small, a normwise error says nothing; random-shape runs on the GPU meet their tolerance everywhere
    but here and at a few entries of very short sequences that cancel the same way."""
    rng = np.random.default_rng(11)
    B, L, M, D = 2, 1, 5, 16
    alpha = rng.random((B, L, M)) * 0.8 + 0.1
    us, osc = rng.random((B, L, 1)) * 0.8 + 0.1, rng.random((B, L, 1)) + 0.5
    inp, w_out = rng.standard_normal((B, L, D)), rng.standard_normal((B, L, D))
    for eps in (1e-4, 1e-8):
        g = O.memory_backward(alpha, us, osc, inp, w_out, None, None, True, eps)
        assert np.abs(g["d_update_scale"]).max() < 200 * eps * np.abs(g["d_output_scale"]).max()  # eps / mean(h^2), h = (1 - g) x
    # with a second step the first one's gate also sees what arrives from the future: not small any more
    L = 2
    alpha = rng.random((B, L, M)) * 0.8 + 0.1
    us, osc = rng.random((B, L, 1)) * 0.8 + 0.1, rng.random((B, L, 1)) + 0.5
    inp, w_out = rng.standard_normal((B, L, D)), rng.standard_normal((B, L, D))
    g = O.memory_backward(alpha, us, osc, inp, w_out, None, None, True, 1e-8)
    assert np.abs(g["d_update_scale"]).max() > 1e-3 * np.abs(g["d_output_scale"]).max()


# ------------------------------------------------------------------ compiled oracle and port

@pytest.mark.parametrize("plain", [False, True])
def test_c_oracle_equals_numpy_oracle(plain):
    g, x, G, h0, fpg = rand_problem(3, 2, 5, 257, seed=15)
    h = O.forward(g, x, h0, plain)
    np.testing.assert_allclose(C.forward_f64(g, x, h0, plain), h, rtol=1e-14, atol=1e-14)
    for state in (h0, None):
        tg, gg, _ = O.backward_per_row(g, G, h, x, fpg, state, plain)
        tc, gc = C.backward_f64(g, G, h, x, fpg, state, plain)
        np.testing.assert_allclose(tc, tg, rtol=1e-14, atol=1e-14)
        np.testing.assert_allclose(gc, gg, rtol=1e-14, atol=1e-14)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2), (torch.float16, 1e-2)])
def test_cpu_port_within_tolerance_of_f64(dtype, tol):
    gen = torch.Generator().manual_seed(16)
    B, M, D, L = 2, 2, 3, 1000
    g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype)
    x = torch.randn(B, D, L, generator=gen).to(dtype)
    G = torch.randn(B, M, D, L, generator=gen).to(dtype)
    h0 = torch.randn(B, M, D, generator=gen).to(dtype)
    out = torch.empty(B, M, D, L, dtype=dtype)
    C.port_forward(g, x, h0, out)
    ref = C.forward_f64(g, x, h0)
    nerr = lambda a, r: np.abs(a.double().numpy() - r).max() / np.abs(r).max()
    assert nerr(out, ref) <= tol
    dx, dg = torch.empty_like(out), torch.empty_like(out)
    C.port_backward(g, G, None, dx, out, x, dg, initial_state=h0)
    tr, gr = C.backward_f64(g, G, out, x, None, h0)
    assert nerr(dx, tr) <= tol and nerr(dg, gr) <= tol


def test_cpu_port_float16_conversions_equal_numpy():
    """The port's own binary16 conversions (the host compiler has no half type) against numpy's:
    the scan with gate 0 stores exactly the token (a load, a multiply by one, a store), so every
    binary16 value must come back unchanged; and the store's float32 -> binary16 rounding must be
    numpy's (nearest even, subnormals, overflow to infinity)."""
    bits = np.arange(65536, dtype=np.uint16)
    vals = bits.view(np.float16)
    # (an infinite state times a zero gate is NaN for the step after; 0 * h + (-0) is +0)
    keep = np.isfinite(vals) & (bits != 0x8000)
    x = torch.from_numpy(vals[keep].copy()).view(1, 1, -1)
    g = torch.zeros_like(x)
    out = torch.empty(1, 1, 1, x.shape[-1], dtype=torch.float16)
    C.port_forward(g, x, None, out)
    assert np.array_equal(out.view(-1).numpy().view(np.uint16), vals[keep].view(np.uint16))
    # rounding on store
    rng = np.random.default_rng(3)
    cases = np.concatenate([rng.standard_normal(4096).astype(np.float32) * np.float32(s)
                            for s in (1e-8, 1e-6, 1e-4, 1.0, 300.0, 70000.0)])
    ties = (np.arange(1, 2049, dtype=np.float32) * 2 + 1) * np.float32(2.0 ** -11)  # halfway between neighbours
    cases = np.concatenate([cases, ties, ties * np.float32(2.0 ** -14), [65504.0, 65519.9, 65520.0, 1e9]]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = cases.astype(np.float16)
    lib = C.load()
    got = np.empty(cases.shape, np.uint16)
    import ctypes
    lib.fmscan_cpu_round_f16.restype = None
    lib.fmscan_cpu_round_f16.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
    lib.fmscan_cpu_round_f16(cases.ctypes.data, got.ctypes.data, cases.size)
    assert np.array_equal(got, want.view(np.uint16))
