"""Parity of the HIP scan (through the C ABI, as fm_scan_forward / fm_scan_backward /
FM_Scan call it) with the float64 CPU oracle, on an MI355X.

Tolerance (stated by the benchmark definition): normwise error against the float64
sequential oracle evaluated on the same, already quantised inputs,
    max|y - ref| / max|ref| <= tol   and   ||y - ref||_2 / ||ref||_2 <= tol,
tol = 1e-5 for float32, 1e-2 for bfloat16 / float16. Backward is checked against
the oracle fed with the states the GPU stored: the plain form reads them all, the
default form reads one of them per wave and tile and makes the others again from the
gates and tokens in float32 (closer to the exact states than the stored ones by up to
one rounding of the storage type, which the tolerance covers).
Where the arithmetic allows it the checks are bit-exact (resets, scaling by two,
row permutation, run-to-run determinism).
"""
import numpy as np
import pytest
import torch

import fm_scan_oracle as O
import fmscan_cpu as C

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-5, torch.bfloat16: 1e-2, torch.float16: 1e-2}
DEV = "cuda:0"


@pytest.fixture(scope="module")
def scan():
    import fm.scan.fm_scan as m

    assert torch.cuda.is_available(), "these tests need the GPU"
    return m


def errs(y, ref):
    y = y.detach().double().cpu().numpy().reshape(ref.shape)
    d = y - ref
    return (float(np.abs(d).max() / max(np.abs(ref).max(), 1e-300)),
            float(np.linalg.norm(d.ravel()) / max(np.linalg.norm(ref.ravel()), 1e-300)))


def check(name, y, ref, tol):
    e_max, e_l2 = errs(y, ref)
    assert e_max <= tol and e_l2 <= tol, f"{name}: max-norm {e_max:.3e}, l2 {e_l2:.3e} > {tol:g}"


# ----------------------------------------------------------------------------- inputs

def gpu_gen(seed=0):
    return torch.Generator(device=DEV).manual_seed(seed)


def baseline_inputs(cfg, dtype=None):
    """(gates, tokens, out_grad) of benchmark configuration `cfg` (1-5) as (rows, 1, L) / (rows, 1, 1, L)
    tensors: a (B, C, T) problem is the zero-copy fold B' = B*C, M = D = 1."""
    gen = gpu_gen(0)
    rn = lambda *s: torch.randn(*s, device=DEV, generator=gen)
    ru = lambda *s: torch.rand(*s, device=DEV, generator=gen)
    if cfg == 1:
        B, Cn, T, dt = 2, 64, 1024, torch.float32
        x, g, G = rn(B * Cn, 1, T), torch.sigmoid(rn(B * Cn, 1, T) + 2.0), rn(B * Cn, 1, 1, T)
    elif cfg == 2:
        B, Cn, T, dt = 8, 1024, 4096, torch.float32
        x, g, G = rn(B * Cn, 1, T), 0.9 + 0.1 * ru(B * Cn, 1, T), rn(B * Cn, 1, 1, T)
    elif cfg == 3:
        B, Cn, T, dt = 16, 2048, 16384, torch.bfloat16
        g = 1.0 - torch.exp(-torch.nn.functional.softplus(rn(B * Cn, 1, T)))
        x, G = rn(B * Cn, 1, T), rn(B * Cn, 1, 1, T)
    elif cfg == 4:
        B, Cn, T, dt = 4, 1024, 65536, torch.bfloat16
        g = 0.99 + 0.01 * ru(B * Cn, 1, T)
        g[ru(B * Cn, 1, T) < 0.01] = 0.0
        x, G = 0.1 * rn(B * Cn, 1, T), rn(B * Cn, 1, 1, T)
    elif cfg == 5:
        B, Cn, T, dt = 32, 4096, 2048, torch.bfloat16
        decay = torch.exp(-torch.exp(-6.0 * ru(1, Cn, 1)))
        g = decay.expand(B, Cn, T).reshape(B * Cn, 1, T)
        x = (rn(B * Cn, 1, T) * rn(B * Cn, 1, T)) / 128.0
        G = rn(B * Cn, 1, 1, T)
    else:
        raise ValueError(cfg)
    dt = dtype or dt
    return g.to(dt).contiguous(), x.to(dt).contiguous(), G.to(dt).contiguous()


def run_fwd_bwd(scan, g, x, G, h0=None, fpg=None, **kw):
    rows, M, L = g.shape
    D = x.shape[1]
    z = torch.zeros(rows, M, D, dtype=g.dtype, device=g.device)
    out = torch.empty(rows, M, D, L, dtype=g.dtype, device=g.device)
    scan.fm_scan_forward(g, x, z if h0 is None else h0, out, **kw)
    dx, dg = torch.empty_like(out), torch.empty_like(out)
    scan.fm_scan_backward(g, G, z if fpg is None else fpg, dx, out, x, dg,
                          initial_state=z if h0 is None else h0, **kw)
    return out, dx, dg


def oracle_rows(g, x, G, out, idx, h0=None, fpg=None, plain=False):
    """float64 oracle on the rows `idx` of a fold-mapped (rows, 1, L) problem."""
    sel = lambda t: None if t is None else t[idx]
    h_ref = C.forward_f64(sel(g), sel(x), sel(h0), plain)
    tg, gg = C.backward_f64(sel(g), sel(G), sel(out), sel(x), sel(fpg),
                            sel(h0) if h0 is not None else np.zeros((len(idx), 1, 1)), plain)
    return h_ref, tg, gg


# ----------------------------------------------------------------------------- the five benchmark configurations

@pytest.mark.parametrize("cfg", [1, 2, 3, 4, 5])
def test_baseline_config(scan, cfg):
    g, x, G = baseline_inputs(cfg)
    out, dx, dg = run_fwd_bwd(scan, g, x, G)
    torch.cuda.synchronize()
    rows = g.shape[0]
    if cfg in (1, 2):
        idx = torch.arange(rows, device=DEV)
    else:
        pick = torch.randperm(rows, device=DEV, generator=gpu_gen(1))[:254]
        idx = torch.cat([torch.tensor([0, rows - 1], device=DEV), pick])
    h_ref, tg, gg = oracle_rows(g, x, G, out, idx)
    tol = TOL[g.dtype]
    check(f"cfg{cfg} states", out[idx], h_ref, tol)
    check(f"cfg{cfg} token grad", dx[idx], tg, tol)
    check(f"cfg{cfg} gate grad", dg[idx], gg, tol)

    # full-size properties, bit-exact
    out2, dx2, dg2 = run_fwd_bwd(scan, g, x, G)
    assert torch.equal(out, out2) and torch.equal(dx, dx2) and torch.equal(dg, dg2), "not deterministic"
    del out2, dx2, dg2
    # doubling tokens and upstream gradient: states and token gradient double, the gate
    # gradient (h_prev - x) * delta quadruples; scaling by two is exact in every dtype
    o3, dx3, dg3 = run_fwd_bwd(scan, g, x * 2, G * 2)
    assert torch.equal(o3, out * 2), "states not linear in tokens"
    del o3
    assert torch.equal(dx3, dx * 2)
    assert torch.equal(dg3, dg * 4)
    del dx3, dg3
    if cfg == 4:  # exact resets: g == 0 -> h == x
        zero = (g.view(rows, -1) == 0)
        assert zero.any()
        assert torch.equal(out.view(rows, -1)[zero], x.view(rows, -1)[zero])
        assert torch.isfinite(out).all() and torch.isfinite(dx).all() and torch.isfinite(dg).all()


@pytest.mark.parametrize("dtype", [torch.float16])
def test_baseline_config5_float16(scan, dtype):
    g, x, G = baseline_inputs(5, dtype)
    out, dx, dg = run_fwd_bwd(scan, g, x, G)
    rows = g.shape[0]
    idx = torch.randperm(rows, device=DEV, generator=gpu_gen(2))[:256]
    h_ref, tg, gg = oracle_rows(g, x, G, out, idx)
    check("states", out[idx], h_ref, TOL[dtype])
    check("token grad", dx[idx], tg, TOL[dtype])
    check("gate grad", dg[idx], gg, TOL[dtype])


def test_config5_native_shape_through_autograd(scan):
    """Config 5 read as the layer shapes it: M = 32 memory rows, D = 128 state
    channels; gates (B, 32, T), tokens (B, 128, T), states (B, 32, 128, T)."""
    B, M, D, L, dt = 32, 32, 128, 2048, torch.bfloat16
    gen = gpu_gen(3)
    decay = torch.exp(-torch.exp(-6.0 * torch.rand(1, M, 1, device=DEV, generator=gen)))
    g = decay.expand(B, M, L).contiguous().to(dt).requires_grad_()
    x = (torch.randn(B, D, L, device=DEV, generator=gen) *
         torch.randn(B, D, L, device=DEV, generator=gen) / 128.0).to(dt).requires_grad_()
    G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    states = scan.fm_scan(g, x)
    states.backward(G)
    for b in (0, B - 1):
        gb, xb, Gb = g[b:b + 1].detach(), x[b:b + 1].detach(), G[b:b + 1]
        h_ref = C.forward_f64(gb, xb)
        check("states", states[b:b + 1], h_ref, TOL[dt])
        tg, gg = C.backward_f64(gb, Gb, states[b:b + 1], xb, None, np.zeros((1, M, D)))
        check("d_gates", g.grad[b:b + 1], gg.sum(axis=2), TOL[dt])
        check("d_tokens", x.grad[b:b + 1], tg.sum(axis=1), TOL[dt])
    # every batch element, at full size: the kernel with the sums inside against the reference's route
    # (both (B, M, D, L) tensors written in full, then torch.sum); two rounded results, hence 2 * TOL
    zeros = torch.zeros(B, M, D, dtype=dt, device=DEV)
    dx, dg = torch.empty_like(states), torch.empty_like(states)
    scan.fm_scan_backward(g.detach(), G, zeros, dx, states.detach(), x.detach(), dg, initial_state=zeros)
    check("d_gates, all batch elements", g.grad, dg.sum(dim=2).double().cpu().numpy(), 2 * TOL[dt])
    check("d_tokens, all batch elements", x.grad, dx.sum(dim=1).double().cpu().numpy(), 2 * TOL[dt])
    for b in range(B):  # and no batch element stands out
        e = (g.grad[b].float() - dg[b].sum(dim=1).float()).abs().max().item() / dg[b].sum(dim=1).float().abs().max().item()
        assert e <= 2 * TOL[dt], (b, e)


# ----------------------------------------------------------------------------- shapes, dtypes, variants

SHAPES = [(1, 1, 1, 1), (1, 1, 1, 7), (2, 1, 1, 32), (1, 2, 3, 33), (2, 3, 5, 512), (3, 1, 2, 1000),
          (1, 1, 2, 4096), (2, 2, 1, 5000), (1, 1, 1, 131072), (5, 1, 1, 2048)]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("waves", [0, 1, 2, 4, 8])
@pytest.mark.parametrize("plain", [False, True])
def test_shapes_and_variants(scan, dtype, waves, plain):
    for (B, M, D, L) in SHAPES:
        gen = torch.Generator().manual_seed(B * 1000 + L)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        G = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        fpg = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        out, dx, dg = run_fwd_bwd(scan, g, x, G, h0, fpg, plain=plain, waves_per_row=waves)
        h_ref = C.forward_f64(g, x, h0, plain)
        tg, gg = C.backward_f64(g, G, out, x, fpg, h0, plain)
        tag = f"{(B, M, D, L)} {dtype} waves={waves} plain={plain}"
        check(tag + " states", out, h_ref, TOL[dtype])
        check(tag + " token grad", dx, tg, TOL[dtype])
        check(tag + " gate grad", dg, gg, TOL[dtype])


def test_every_compiled_variant_runs_once(scan):
    """A fixed-seed walk over the kernel variants the library holds, each asked for explicitly through the
    flags: element type x waves per row (1, 2, 4, 8) x prefetch depth (2, 4) x plain / FM form x access
    (fold rows with 16-byte vectors, shared rows with 16-byte vectors, rows off 16-byte alignment), with
    the cap on resident blocks cycling through its range; then the same for rows cut into segments, and
    the 16-wave backward that only the library chooses, with shared rows. Random small shapes, forward
    and backward against the compiled float64 oracle at the usual tolerance."""
    rnd = np.random.default_rng(20240607)
    caps = [1, 2, 3, 4, 6, 8, 12, 15]
    n = 0
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        vec = 16 // torch.empty(0, dtype=dtype).element_size()  # elements per 16 bytes
        for waves in (1, 2, 4, 8):
            for depth in (2, 4):
                for plain in (False, True):
                    for access in ("fold", "shared", "unaligned"):
                        tile = vec * 64 * waves
                        # a few tiles, so that the loops with unchecked whole tiles (2 * depth and more) and
                        # the checked ends both run; every third case is shorter than that
                        tiles = int(rnd.integers(1, 4)) if n % 3 == 0 else int(rnd.integers(2 * depth, 3 * depth + 2))
                        L = tiles * tile - int(rnd.integers(0, tile // vec)) * vec
                        if access == "unaligned":
                            L += int(rnd.integers(1, vec))
                        B = int(rnd.integers(1, 4))
                        M, D = (1, 1) if access == "fold" else (int(rnd.integers(1, 4)), int(rnd.integers(2, 5)))
                        if access == "fold":
                            B = int(rnd.integers(3, 9))
                        gen = torch.Generator().manual_seed(1000 + n)
                        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
                        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
                        G = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
                        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
                        fpg = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
                        kw = dict(plain=plain, waves_per_row=waves, depth=depth, blocks_per_cu=caps[n % len(caps)])
                        tag = f"case {n}: {(B, M, D, L)} {dtype} {access} {kw}"
                        print(tag, flush=True)
                        out, dx, dg = run_fwd_bwd(scan, g, x, G, h0, fpg, **kw)
                        h_ref = C.forward_f64(g, x, h0, plain)
                        tg, gg = C.backward_f64(g, G, out, x, fpg, h0, plain)
                        check(tag + " states", out, h_ref, TOL[dtype])
                        check(tag + " token grad", dx, tg, TOL[dtype])
                        check(tag + " gate grad", dg, gg, TOL[dtype])
                        n += 1
        # rows cut into segments (single waves, both depths), and 16 waves per row in backward with shared rows
        for depth, segments, (B, M, D, L) in ((2, 3, (2, 1, 1, 40 * vec * 64)), (4, 5, (1, 2, 2, 50 * vec * 64 + vec)),
                                              (2, 0, (2, 4, 5, 70 * vec * 64)), (4, 0, (3, 2, 7, 64 * vec * 64 + 3))):
            for plain in (False, True):
                gen = torch.Generator().manual_seed(2000 + n)
                g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
                x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
                G = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
                h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
                fpg = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
                kw = dict(plain=plain, depth=depth, segments=segments)
                tag = f"case {n}: {(B, M, D, L)} {dtype} {kw}"
                print(tag, flush=True)
                out, dx, dg = run_fwd_bwd(scan, g, x, G, h0, fpg, **kw)
                h_ref = C.forward_f64(g, x, h0, plain)
                tg, gg = C.backward_f64(g, G, out, x, fpg, h0, plain)
                check(tag + " states", out, h_ref, TOL[dtype])
                check(tag + " token grad", dx, tg, TOL[dtype])
                check(tag + " gate grad", dg, gg, TOL[dtype])
                n += 1
    assert n == 3 * (4 * 2 * 2 * 3 + 8)


def test_exact_rational_vectors_on_the_gpu(scan, exact_cases):
    """The committed exact vectors (tests/golden/fm_scan_exact.json: small problems solved in rational
    arithmetic, derivatives by dual numbers) through fmscan_forward, fmscan_backward and, where the shape
    fits it, fmscan_backward_reduced. Every input is a small dyadic rational that float32, float16 and
    bfloat16 hold exactly, so the only error is the kernels' own arithmetic: 1e-6 in float32 (the states
    need up to 27 bits, more than a float32 holds: not bit-exact), the storage type's 1e-2 otherwise."""
    lib, st = scan.module, torch.cuda.current_stream().cuda_stream
    for name, c in exact_cases.items():
        B, M, D, L, plain = c["B"], c["M"], c["D"], c["L"], c["plain"]
        a = lambda k: np.array(c[k], dtype=np.float64)
        for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2), (torch.float16, 1e-2)):
            t = lambda k: torch.from_numpy(a(k)).to(dtype).to(DEV)
            g, x, G, h0, fpg = t("gates"), t("tokens"), t("out_grad"), t("initial_state"), t("first_prop_grad")
            for k, v in (("gates", g), ("tokens", x), ("out_grad", G), ("initial_state", h0), ("first_prop_grad", fpg)):
                assert np.array_equal(v.double().cpu().numpy(), a(k)), (name, k, dtype)  # held exactly
            out = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
            dx, dg, dh0 = torch.empty_like(out), torch.empty_like(out), torch.empty_like(h0)
            scan.fm_scan_forward(g, x, h0, out, plain=plain)
            tag = f"{name} {dtype}"
            check(tag + " states", out, a("states"), tol)
            if dtype == torch.float32 and L == 1:
                assert np.array_equal(out.double().cpu().numpy(), a("states")), tag  # one step: representable, exact
            # backward from the exact states (what a float64 forward would have stored, rounded to the dtype)
            saved = t("states")
            scan.fm_scan_backward(g, G, fpg, dx, saved, x, dg, initial_state=h0, initial_state_grad=dh0, plain=plain)
            check(tag + " token grad", dx, a("token_grad"), tol)
            check(tag + " gate grad", dg, a("gate_grad"), tol)
            check(tag + " initial state grad", dh0, a("d_initial_state"), tol)
            aligned = (L * out.element_size()) % 16 == 0
            if M > 1 and D > 1 and aligned:
                dh0r = torch.empty_like(h0)
                d_g, d_x = scan.fm_scan_backward_reduced(g, G, fpg, saved, x, initial_state=h0,
                                                         initial_state_grad=dh0r, plain=plain)
                check(tag + " d_gates (sums inside)", d_g, a("gate_grad").sum(axis=2), tol)
                check(tag + " d_tokens (sums inside)", d_x, a("token_grad").sum(axis=1), tol)
                check(tag + " initial state grad (sums inside)", dh0r, a("d_initial_state"), tol)
            elif M > 1 and D > 1:
                groups = lib.fmscan_reduced_groups(B, D)
                part = torch.empty(B, M, groups, L, device=DEV)
                dxr = torch.empty(B, D, L, dtype=dtype, device=DEV)
                code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
                rc = lib.fmscan_backward_reduced(g.data_ptr(), G.data_ptr(), fpg.data_ptr(), dxr.data_ptr(),
                                                 saved.data_ptr(), x.data_ptr(), part.data_ptr(), None, None,
                                                 B, M, D, L, code, 1 if plain else 0, st)
                assert rc == -7, (tag, rc)  # rows that are not 16-byte multiples: refused, nothing launched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_long_rows_with_rows_enough_not_to_be_cut(scan, dtype):
    """Rows of 64 tiles or more, 32 rows or more: the library's own choice there is 8 waves per row
    forward and 16 backward (a choice only it makes). Whole tiles and a ragged end, aligned rows and
    rows one element off (element access)."""
    for rows, L in ((40, 40000), (33, 40001), (64, 65536)):
        if dtype == torch.float32:
            L = L // 2 + (L & 1)  # still 64 tiles or more of 256 elements
        gen = torch.Generator().manual_seed(L)
        g = torch.sigmoid(torch.randn(rows, 1, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(rows, 1, L, generator=gen).to(dtype).to(DEV)
        G = torch.randn(rows, 1, 1, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(rows, 1, 1, generator=gen).to(dtype).to(DEV)
        fpg = torch.randn(rows, 1, 1, generator=gen).to(dtype).to(DEV)
        for plain in (False, True):
            out, dx, dg = run_fwd_bwd(scan, g, x, G, h0, fpg, plain=plain)
            h_ref = C.forward_f64(g, x, h0, plain)
            tg, gg = C.backward_f64(g, G, out, x, fpg, h0, plain)
            tag = f"{(rows, L)} {dtype} plain={plain}"
            check(tag + " states", out, h_ref, TOL[dtype])
            check(tag + " token grad", dx, tg, TOL[dtype])
            check(tag + " gate grad", dg, gg, TOL[dtype])
            # the same rows with 8 waves per row, as asked for by the caller: the same mathematics
            _, dx8, dg8 = run_fwd_bwd(scan, g, x, G, h0, fpg, plain=plain, waves_per_row=8)
            check(tag + " token grad vs 8 waves", dx, dx8.double().cpu().numpy(), 2 * TOL[dtype])
            check(tag + " gate grad vs 8 waves", dg, dg8.double().cpu().numpy(), 2 * TOL[dtype])


def test_more_than_2_31_elements(scan):
    """The reference indexes with 32-bit ints (fm_scan.cuh:76-82: N < 2^31); here offsets are 64-bit.
    Rows that lie beyond element 2^31 of a problem must come out exactly as the same rows of a small
    problem of their own do (same kernel, same arithmetic per row: bit-exact), fold mapping and
    Factorization-Memory shape (the kernel with the sums inside) alike."""
    dt = torch.bfloat16
    gen = gpu_gen(3)
    # fold mapping: 2^17 + 8 rows of 16384 = 2^31 + 131072 elements per (rows, 1, 1, L) tensor
    rows, L, tail = (1 << 17) + 8, 16384, 8
    g = torch.rand(rows, 1, L, device=DEV, generator=gen).to(dt)
    x = torch.randn(rows, 1, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(rows, 1, 1, L, device=DEV, generator=gen).to(dt)
    assert G.numel() > 1 << 31
    out, dx, dg = run_fwd_bwd(scan, g, x, G)
    o2, dx2, dg2 = run_fwd_bwd(scan, g[-tail:].contiguous(), x[-tail:].contiguous(), G[-tail:].contiguous())
    assert torch.equal(out[-tail:], o2) and torch.equal(dx[-tail:], dx2) and torch.equal(dg[-tail:], dg2)
    h_ref, tg, gg = oracle_rows(g, x, G, out, [rows - 1])
    check("states of the last row", out[rows - 1:], h_ref, TOL[dt])
    check("token gradient of the last row", dx[rows - 1:], tg, TOL[dt])
    check("gate gradient of the last row", dg[rows - 1:], gg, TOL[dt])
    del g, x, G, out, dx, dg, o2, dx2, dg2
    torch.cuda.empty_cache()

    # (B, M, D, L) = (9, 32, 128, 65536): 2^31 + 2^28 elements; the last batch element lies beyond 2^31
    B, M, D, L = 9, 32, 128, 65536
    g = torch.rand(B, M, L, device=DEV, generator=gen).to(dt)
    x = torch.randn(B, D, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    assert G.numel() > 1 << 31
    z = torch.zeros(B, M, D, dtype=dt, device=DEV)
    states = torch.empty(B, M, D, L, dtype=dt, device=DEV)
    scan.fm_scan_forward(g, x, z, states)
    d_gates, d_tokens = scan.fm_scan_backward_reduced(g, G, z, states, x)
    s1 = torch.empty(1, M, D, L, dtype=dt, device=DEV)
    scan.fm_scan_forward(g[-1:].contiguous(), x[-1:].contiguous(), z[-1:], s1)
    assert torch.equal(states[-1:], s1)
    dg1, dt1 = scan.fm_scan_backward_reduced(g[-1:].contiguous(), G[-1:].contiguous(), z[-1:], s1, x[-1:].contiguous())
    # a single batch element has its slots dealt to more blocks than nine have, and its rows summed in
    # groups of 4 instead of 8, so both gradients' float32 sums run in another order: equal to one
    # bfloat16 rounding of the largest entry, 2^-8 (a wrong index would be an error of order one)
    check("gate gradient of the last batch element", d_gates[-1:], dg1.double().cpu().numpy(), 4e-3)
    check("token gradient of the last batch element", d_tokens[-1:], dt1.double().cpu().numpy(), 4e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unaligned_pointers_take_the_element_path(scan, dtype):
    """Tensors that start one element past a 16-byte boundary (still contiguous)."""
    B, M, D, L = 2, 2, 3, 520
    gen = torch.Generator().manual_seed(5)

    def shifted(*shape):
        n = int(np.prod(shape))
        buf = torch.randn(n + 1, generator=gen).to(dtype).to(DEV)
        t = buf[1:].view(*shape)
        assert t.data_ptr() % 16 != 0 and t.is_contiguous()
        return t

    g = shifted(B, M, L).sigmoid_()
    x, G, h0 = shifted(B, D, L), shifted(B, M, D, L), shifted(B, M, D)
    out, dx, dg = shifted(B, M, D, L), shifted(B, M, D, L), shifted(B, M, D, L)
    scan.fm_scan_forward(g, x, h0, out)
    scan.fm_scan_backward(g, G, torch.zeros_like(h0), dx, out, x, dg, initial_state=h0)
    check("states", out, C.forward_f64(g, x, h0), TOL[dtype])
    tg, gg = C.backward_f64(g, G, out, x, None, h0)
    check("token grad", dx, tg, TOL[dtype])
    check("gate grad", dg, gg, TOL[dtype])


def test_reset_and_hold_gates_are_exact(scan):
    """g = 0 restarts the row at the token, bit-exactly in every dtype; g = 1 passes no
    gradient to its token, exactly; long runs of exact ones and zeros give no NaN / Inf
    and stay within tolerance of the oracle."""
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        rows, L = 64, 8192
        gen = gpu_gen(6)
        r = torch.rand(rows, 1, L, device=DEV, generator=gen)
        g = torch.where(r < 0.3, torch.zeros_like(r), torch.where(r < 0.8, torch.ones_like(r), r)).to(dtype)
        x = torch.randn(rows, 1, L, device=DEV, generator=gen).to(dtype)
        G = torch.randn(rows, 1, 1, L, device=DEV, generator=gen).to(dtype)
        out, dx, dg = run_fwd_bwd(scan, g, x, G)
        g2, x2, o2 = g.view(rows, L), x.view(rows, L), out.view(rows, L)
        assert torch.equal(o2[g2 == 0], x2[g2 == 0])
        assert (dx.view(rows, L)[g2 == 1] == 0).all()
        for t in (out, dx, dg):
            assert torch.isfinite(t).all()
        idx = torch.arange(rows, device=DEV)
        h_ref, tg, gg = oracle_rows(g, x, G, out, idx)
        check("states", out, h_ref, TOL[dtype])
        check("token grad", dx, tg, TOL[dtype])
        check("gate grad", dg, gg, TOL[dtype])


def test_row_permutation_is_bit_exact(scan):
    rows, L, dt = 1000, 4096, torch.bfloat16
    gen = gpu_gen(7)
    g = torch.rand(rows, 1, L, device=DEV, generator=gen).to(dt)
    x = torch.randn(rows, 1, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(rows, 1, 1, L, device=DEV, generator=gen).to(dt)
    perm = torch.randperm(rows, device=DEV, generator=gen)
    a = run_fwd_bwd(scan, g, x, G)
    b = run_fwd_bwd(scan, g[perm].contiguous(), x[perm].contiguous(), G[perm].contiguous())
    for ta, tb in zip(a, b):
        assert torch.equal(ta[perm], tb)


def test_broadcast_rows_equal_explicit_rows(scan):
    """(B, M, D) broadcasting equals the fold-mapped problem with gates and tokens
    expanded by hand, bit for bit."""
    B, M, D, L, dt = 2, 3, 4, 2048, torch.bfloat16
    gen = gpu_gen(8)
    g = torch.rand(B, M, L, device=DEV, generator=gen).to(dt)
    x = torch.randn(B, D, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    out, dx, dg = run_fwd_bwd(scan, g, x, G, waves_per_row=1)
    ge = g[:, :, None, :].expand(B, M, D, L).reshape(B * M * D, 1, L).contiguous()
    xe = x[:, None, :, :].expand(B, M, D, L).reshape(B * M * D, 1, L).contiguous()
    oe, dxe, dge = run_fwd_bwd(scan, ge, xe, G.view(B * M * D, 1, 1, L), waves_per_row=1)
    assert torch.equal(out.view(-1), oe.view(-1))
    assert torch.equal(dx.view(-1), dxe.view(-1)) and torch.equal(dg.view(-1), dge.view(-1))


@pytest.mark.parametrize("shape", [(1, 16, 1024, 4096), (1, 3, 1024, 4096), (2, 2, 600, 8192)])
def test_rows_visited_out_of_memory_order_equal_explicit_rows(scan, shape):
    """When the tokens of a batch element are too many for one L2 (D * L * element size > 4 MiB) the
    kernels visit the rows slot after slot in groups of d instead of in memory order. Same rows, same
    arithmetic: bit for bit what the fold-mapped problem with gates and tokens expanded by hand gives
    (one wave per row in the first shape, several in the others)."""
    B, M, D, L = shape
    dt = torch.bfloat16
    gen = gpu_gen(31)
    g = torch.rand(B, M, L, device=DEV, generator=gen).to(dt)
    x = torch.randn(B, D, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    assert D * L * 2 > (4 << 20)
    out, dx, dg = run_fwd_bwd(scan, g, x, G)
    ge = g[:, :, None, :].expand(B, M, D, L).reshape(B * M * D, 1, L).contiguous()
    xe = x[:, None, :, :].expand(B, M, D, L).reshape(B * M * D, 1, L).contiguous()
    kw = {"waves_per_row": 1} if B * M * D >= 16384 else {}
    oe, dxe, dge = run_fwd_bwd(scan, ge, xe, G.view(B * M * D, 1, 1, L), **kw)
    if kw:
        assert torch.equal(out.view(-1), oe.view(-1))
        assert torch.equal(dx.view(-1), dxe.view(-1)) and torch.equal(dg.view(-1), dge.view(-1))
    else:  # the two problems may be given different numbers of waves per row: equal to rounding
        for a, b, name in ((out, oe, "states"), (dx, dxe, "token grad"), (dg, dge, "gate grad")):
            check(name, a, b.double().cpu().numpy().reshape(a.shape), TOL[dt])
    idx = torch.randperm(B * M * D, device=DEV, generator=gen)[:64]
    h_ref = C.forward_f64(ge[idx], xe[idx])
    check("states", out.view(B * M * D, 1, 1, L)[idx], h_ref, TOL[dt])


def test_segment_chaining(scan):
    """scan(L) == scan(first part) followed by scan(rest, initial_state = last state),
    and backward chains through first_prop_grad the same way."""
    rows, L, k, dt = 256, 8192, 3000 // 8 * 8, torch.float32
    gen = gpu_gen(9)
    g = (0.9 + 0.09 * torch.rand(rows, 1, L, device=DEV, generator=gen)).to(dt)
    x = torch.randn(rows, 1, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(rows, 1, 1, L, device=DEV, generator=gen).to(dt)
    out, dx, dg = run_fwd_bwd(scan, g, x, G)
    cut = lambda t, a, b: t[..., a:b].contiguous()
    o1, _, _ = run_fwd_bwd(scan, cut(g, 0, k), cut(x, 0, k), cut(G, 0, k))
    h_mid = o1[..., -1].contiguous()
    o2, dx2, dg2 = run_fwd_bwd(scan, cut(g, k, L), cut(x, k, L), cut(G, k, L), h0=h_mid)
    ref = out.double().cpu().numpy()
    check("chained states", torch.cat([o1, o2], dim=3), ref, 1e-5)
    # gradient crossing the cut: g[k] * delta[k]; delta[k] = dx2[k] / (1 - g[k])
    delta_k = dx2[..., 0] / (1 - g[:, :, k].view(rows, 1, 1))
    cross = (g[:, :, k].view(rows, 1, 1) * delta_k).contiguous()
    _, dx1, dg1 = run_fwd_bwd(scan, cut(g, 0, k), cut(x, 0, k), cut(G, 0, k), fpg=cross)
    # 1e-4: the gradient that crosses the cut was rebuilt above by a division by 1 - g >= 0.01, which
    # magnifies the float32 rounding of dx2 a hundredfold before it enters the first part
    check("chained token grad", torch.cat([dx1, dx2], dim=3), dx.double().cpu().numpy(), 1e-4)
    check("chained gate grad", torch.cat([dg1, dg2], dim=3), dg.double().cpu().numpy(), 1e-4)


# ----------------------------------------------------------------------------- few rows: cut rows

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("plain", [False, True])
def test_few_long_rows_are_cut_into_segments(scan, dtype, plain):
    """Fewer rows than compute units: rows are cut into segments (two passes, carries
    through a workspace). Automatic and requested cuts, aligned and ragged lengths,
    non-zero initial state and first_prop_grad, initial-state gradient."""
    cases = [((3, 1, 1, 131072), 0), ((1, 2, 2, 65536), 0), ((2, 1, 1, 40000), 0), ((2, 1, 1, 40001), 0),
             ((5, 1, 1, 8192), 7), ((300, 1, 1, 4096), 2), ((1, 1, 1, 131072), 255), ((2, 1, 3, 2051), 3)]
    for (B, M, D, L), segments in cases:
        gen = torch.Generator().manual_seed(L + segments)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 3).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        G = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        fpg = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
        need = scan.module.fmscan_workspace_bytes(B, M, D, L, code, segments << 20)
        assert need > 0, "this case is meant to take the segmented path"
        out = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        dx, dg, dh0 = torch.empty_like(out), torch.empty_like(out), torch.empty_like(h0)
        scan.fm_scan_forward(g, x, h0, out, plain=plain, segments=segments)
        scan.fm_scan_backward(g, G, fpg, dx, out, x, dg, initial_state=h0, initial_state_grad=dh0,
                              plain=plain, segments=segments)
        tag = f"{(B, M, D, L)} {dtype} segments={segments} plain={plain}"
        check(tag + " states", out, C.forward_f64(g, x, h0, plain), TOL[dtype])
        tg, gg, delta = O.backward_per_row(g, G, out, x, fpg, h0, plain)
        check(tag + " token grad", dx, tg, TOL[dtype])
        check(tag + " gate grad", dg, gg, TOL[dtype])
        check(tag + " initial state grad", dh0, O.to_f64(g)[:, :, 0][:, :, None] * delta[..., 0], TOL[dtype])
        # the same problem scanned in one piece agrees to rounding
        out1 = torch.empty_like(out)
        scan.fm_scan_forward(g, x, h0, out1, plain=plain, segments=1)
        check(tag + " cut vs uncut", out, out1.double().cpu().numpy(), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_short_rows_several_per_wave(scan, dtype):
    """Rows of at most 64 chunks of 16 bytes take the kernels that put several rows into a wave: every
    number of chunks from 1 to 64, lengths that are not whole chunks, row counts that leave the last wave part empty, fold mapping and shared
    gates / tokens, both forms, non-zero initial state and first_prop_grad, the initial-state gradient;
    against the oracle, and against the one-row-per-wave kernels (asked for by flag) to rounding."""
    E = 4 if dtype == torch.float32 else 8
    shapes = [(37, 1, 1), (2, 3, 5), (1, 4, 33), (130, 1, 1)]
    n = 0
    # whole chunks, then lengths that leave the last chunk ragged and the rows at odd addresses
    lengths = [(chunks, chunks * E) for chunks in range(1, 65)]
    lengths += [(k, L) for k, L in enumerate((1, 2, 3, 5, 7, 9, 13, 31, 33, 50, 100, 101, 127, 250, 255, 500, 511))
                if L * (16 // E) <= 1024]
    for chunks, L in lengths:
        B, M, D = shapes[chunks % len(shapes)]
        for plain in ((False, True) if chunks % 5 == 0 else (chunks % 2 == 1,)):
            gen = torch.Generator().manual_seed(1000 + chunks)
            g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
            x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
            G = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
            h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
            fpg = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
            out = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
            dx, dg, dh0 = torch.empty_like(out), torch.empty_like(out), torch.empty_like(h0)
            scan.fm_scan_forward(g, x, h0, out, plain=plain)
            scan.fm_scan_backward(g, G, fpg, dx, out, x, dg, initial_state=h0, initial_state_grad=dh0, plain=plain)
            tag = f"{(B, M, D, L)} {dtype} plain={plain}"
            check(tag + " states", out, C.forward_f64(g, x, h0, plain), TOL[dtype])
            tg, gg, delta = O.backward_per_row(g, G, out, x, fpg, h0, plain)
            check(tag + " token grad", dx, tg, TOL[dtype])
            check(tag + " gate grad", dg, gg, TOL[dtype])
            check(tag + " initial state grad", dh0, O.to_f64(g)[:, :, 0][:, :, None] * delta[..., 0], TOL[dtype])
            # the general kernels on the same problem
            out1 = torch.empty_like(out)
            dx1, dg1, dh1 = torch.empty_like(out), torch.empty_like(out), torch.empty_like(h0)
            scan.fm_scan_forward(g, x, h0, out1, plain=plain, waves_per_row=1)
            scan.fm_scan_backward(g, G, fpg, dx1, out, x, dg1, initial_state=h0, initial_state_grad=dh1,
                                  plain=plain, waves_per_row=1)
            for name, a, b in (("states", out, out1), ("token grad", dx, dx1), ("gate grad", dg, dg1),
                               ("initial state grad", dh0, dh1)):
                check(tag + f" {name} vs a row per wave", a, b.double().cpu().numpy(), 2 * TOL[dtype])
            # no initial state given: the reference's first_prop_grad stands in for it in the gate gradient
            dx2, dg2 = torch.empty_like(out), torch.empty_like(out)
            scan.fm_scan_backward(g, G, fpg, dx2, out, x, dg2, plain=plain)
            tg2, gg2 = C.backward_f64(g, G, out, x, fpg, None, plain)
            check(tag + " token grad (reference call)", dx2, tg2, TOL[dtype])
            check(tag + " gate grad (reference call)", dg2, gg2, TOL[dtype])
            n += 1
    assert n == (64 + 12) + (15 + 3 if dtype == torch.float32 else 17 + 4)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_short_rows_backward_with_the_sums_inside(scan, dtype):
    """fmscan_backward_reduced_packed (rows of up to 256 bytes, through fm_scan_backward_reduced, which asks the
    library whether it applies): groups of 1 to 16 lanes, numbers of chunks that are not powers of two, D that is
    not a multiple of the rows of a wave and D below them, both forms, initial state, first_prop_grad and the
    initial-state gradient; against the oracle's sums, and against fmscan_backward followed by torch.sum."""
    E = 4 if dtype == torch.float32 else 8
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    lib = scan.module
    n = 0
    for chunks, M, D, plain in ((1, 2, 5, False), (2, 3, 70, False), (3, 2, 9, True), (4, 2, 16, False), (5, 3, 20, False),
                                (8, 2, 24, True), (13, 2, 6, False), (16, 3, 10, False)):
        L = chunks * E
        lanes = 1
        while lanes < chunks:
            lanes *= 2
        G = -(-D // (64 // lanes))
        B = -(-4096 // G) + 3
        assert lib.fmscan_reduced_packed_groups(B, M, D, L, code) == G, (B, M, D, L)
        gen = torch.Generator().manual_seed(77 + chunks)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        G_out = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        fpg = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        out = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        scan.fm_scan_forward(g, x, h0, out, plain=plain)
        dh0 = torch.empty_like(h0)
        d_g, d_x = scan.fm_scan_backward_reduced(g, G_out, fpg, out, x, initial_state=h0, initial_state_grad=dh0,
                                                 plain=plain)
        assert d_g.shape == (B, M, L) and d_x.shape == (B, D, L) and d_g.dtype == dtype
        tag = f"{(B, M, D, L)} {dtype} plain={plain}"
        tg, gg, delta = O.backward_per_row(g, G_out, out, x, fpg, h0, plain)
        check(tag + " d_gates", d_g, gg.sum(axis=2), TOL[dtype])
        check(tag + " d_tokens", d_x, tg.sum(axis=1), TOL[dtype])
        check(tag + " d_initial_state", dh0, O.to_f64(g)[:, :, 0][:, :, None] * delta[..., 0], TOL[dtype])
        dx, dg, dh1 = torch.empty_like(out), torch.empty_like(out), torch.empty_like(h0)
        scan.fm_scan_backward(g, G_out, fpg, dx, out, x, dg, initial_state=h0, initial_state_grad=dh1, plain=plain)
        check(tag + " vs two-tensor route (gates)", d_g, dg.float().sum(dim=2).double().cpu().numpy(), 2 * TOL[dtype])
        check(tag + " vs two-tensor route (tokens)", d_x, dx.float().sum(dim=1).double().cpu().numpy(), 2 * TOL[dtype])
        assert torch.equal(dh0, dh1), tag + ": the initial-state gradient is the same arithmetic in both"
        # the reference's call: no initial state (first_prop_grad stands in for it in the gate gradient)
        d_g2, d_x2 = scan.fm_scan_backward_reduced(g, G_out, fpg, out, x, plain=plain)
        tg2, gg2 = C.backward_f64(g, G_out, out, x, fpg, None, plain)
        check(tag + " d_gates (reference call)", d_g2, gg2.sum(axis=2), TOL[dtype])
        check(tag + " d_tokens (reference call)", d_x2, tg2.sum(axis=1), TOL[dtype])
        again = scan.fm_scan_backward_reduced(g, G_out, fpg, out, x, plain=plain)
        assert torch.equal(again[0], d_g2) and torch.equal(again[1], d_x2), tag + ": not deterministic"
        n += 1
    assert n == 8


def test_short_rows_do_not_see_their_neighbours(scan):
    """Several rows share a wave, and the wave scan runs across all of its lanes: a row's results must be
    the same bits wherever it sits and whatever its neighbours hold, NaN and infinity included."""
    dt = torch.bfloat16
    for L in (8, 24, 64, 136, 256, 392, 512):
        rows = 203
        gen = gpu_gen(L)
        g = torch.rand(rows, 1, L, device=DEV, generator=gen).to(dt)
        x = torch.randn(rows, 1, L, device=DEV, generator=gen).to(dt)
        G = torch.randn(rows, 1, 1, L, device=DEV, generator=gen).to(dt)
        a = run_fwd_bwd(scan, g, x, G)
        perm = torch.randperm(rows, device=DEV, generator=gen)
        b = run_fwd_bwd(scan, g[perm].contiguous(), x[perm].contiguous(), G[perm].contiguous())
        for ta, tb in zip(a, b):
            assert torch.equal(ta[perm], tb), L
        # every third row poisoned
        bad = torch.arange(rows, device=DEV) % 3 == 1
        g2, x2, G2 = g.clone(), x.clone(), G.clone()
        x2[bad] = float("nan")
        g2[bad] = float("inf")
        G2[bad] = float("-inf")
        c = run_fwd_bwd(scan, g2, x2, G2)
        for ta, tc in zip(a, c):
            assert torch.equal(ta[~bad], tc[~bad]), L
            assert not torch.isfinite(tc[bad].float()).all()


def test_segment_requests_without_room_fail_loudly(scan):
    g = torch.rand(2, 1, 65536, device=DEV)
    x = torch.rand(2, 1, 65536, device=DEV)
    z = torch.zeros(2, 1, 1, device=DEV)
    out = torch.empty(2, 1, 1, 65536, device=DEV)
    lib = scan.module
    rc = lib.fmscan_forward(g.data_ptr(), x.data_ptr(), z.data_ptr(), out.data_ptr(), 2, 1, 1, 65536, 0,
                            8 << 20, None, 0, None)
    assert rc == -6 and b"workspace" in lib.fmscan_last_error()
    # an automatic cut silently falls back to whole rows when no workspace is offered
    rc = lib.fmscan_forward(g.data_ptr(), x.data_ptr(), z.data_ptr(), out.data_ptr(), 2, 1, 1, 65536, 0,
                            0, None, 0, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    check("states", out, C.forward_f64(g, x), 1e-5)


# ----------------------------------------------------------------------------- sums inside the kernel

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("plain", [False, True])
def test_backward_with_sums_inside(scan, dtype, plain):
    """fm_scan_backward_reduced (d_gates, d_tokens straight from one kernel) against the
    float64 oracle's summed gradients, and against the two-tensor path plus torch.sum."""
    # (the last three: enough blocks for groups of 8 rows, with a ragged last group, a ragged last
    # tile, an odd count of slots per wave and waves without a slot)
    for (B, M, D, L) in [(2, 3, 5, 512), (1, 2, 2, 8), (2, 4, 8, 4096), (1, 33, 17, 1000 // 8 * 8),
                         (3, 2, 9, 2048), (1, 70, 3, 640), (2, 3, 4, 2568),
                         (64, 3, 60, 40), (16, 5, 256, 520), (128, 2, 28, 1032)]:
        gen = torch.Generator().manual_seed(M * 100 + D)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        G = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        fpg = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        out = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        scan.fm_scan_forward(g, x, h0, out, plain=plain)
        dh0 = torch.empty_like(h0)
        d_g, d_x = scan.fm_scan_backward_reduced(g, G, fpg, out, x, initial_state=h0,
                                                 initial_state_grad=dh0, plain=plain)
        assert d_g.shape == (B, M, L) and d_x.shape == (B, D, L) and d_g.dtype == dtype
        tg, gg, delta = O.backward_per_row(g, G, out, x, fpg, h0, plain)
        tag = f"{(B, M, D, L)} {dtype} plain={plain}"
        check(tag + " d_gates", d_g, gg.sum(axis=2), TOL[dtype])
        check(tag + " d_tokens", d_x, tg.sum(axis=1), TOL[dtype])
        check(tag + " d_initial_state", dh0, O.to_f64(g)[:, :, 0][:, :, None] * delta[..., 0], TOL[dtype])
        # the reference's route: two full tensors, then torch.sum (2 * TOL: two rounded results
        # against each other, each within TOL of the exact one)
        dx, dg = torch.empty_like(out), torch.empty_like(out)
        scan.fm_scan_backward(g, G, fpg, dx, out, x, dg, initial_state=h0, plain=plain)
        check(tag + " vs two-tensor route (gates)", d_g, dg.sum(dim=2).double().cpu().numpy(), 2 * TOL[dtype])
        check(tag + " vs two-tensor route (tokens)", d_x, dx.sum(dim=1).double().cpu().numpy(), 2 * TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_sum_of_the_gate_gradient_partials(scan, dtype):
    """fmscan_sum_groups through the C ABI: the (rows, G, L) float32 partials added over G in float32 and
    rounded once, for rows of whole 16-byte vectors and not, one group and many; twice the same bits."""
    lib = scan.module
    stream = torch.cuda.current_stream().cuda_stream
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    for rows, G, L in ((6, 32, 2048), (3, 5, 1001), (2, 1, 64), (1, 130, 7)):
        partial = torch.randn(rows, G, L, device=DEV, generator=gpu_gen(rows + G + L))
        out = torch.empty(rows, L, dtype=dtype, device=DEV)
        assert lib.fmscan_sum_groups(partial.data_ptr(), G, out.data_ptr(), rows, L, code, stream) == 0
        want = partial.double().sum(dim=1)
        assert torch.equal(out, want.to(dtype)) or float((out.double() - want).abs().max()) <= (
            2e-6 if dtype == torch.float32 else 2.0 ** -8) * float(want.abs().max())
        again = torch.empty_like(out)
        assert lib.fmscan_sum_groups(partial.data_ptr(), G, again.data_ptr(), rows, L, code, stream) == 0
        assert torch.equal(out, again)


def test_backward_with_sums_inside_is_deterministic(scan):
    B, M, D, L, dt = 2, 8, 24, 2048, torch.bfloat16
    gen = gpu_gen(21)
    g = torch.rand(B, M, L, device=DEV, generator=gen).to(dt)
    x = torch.randn(B, D, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    z = torch.zeros(B, M, D, dtype=dt, device=DEV)
    out = torch.empty(B, M, D, L, dtype=dt, device=DEV)
    scan.fm_scan_forward(g, x, z, out)
    a = scan.fm_scan_backward_reduced(g, G, z, out, x)
    b = scan.fm_scan_backward_reduced(g, G, z, out, x)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])


# ----------------------------------------------------------------------------- autograd level

def test_notebook_design(scan):
    """The reference's only check (fm_test.ipynb:63-101): batch 1, D 5, L 32, M 1,
    gates 0.5 + 0.5 rand, tokens rand, loss = states.sum(); kernel in bfloat16 and in
    float32 against the per-timestep PyTorch form. Here with a seed and thresholds."""
    from fm.scan.fm_pytorch import fm_scan_pytorch

    torch.manual_seed(0)
    gates0 = 0.5 + 0.5 * torch.rand(1, 1, 32, device=DEV)
    tokens0 = torch.rand(1, 5, 32, device=DEV)
    res = {}
    for name, dt, fn in (("bf16", torch.bfloat16, scan.fm_scan), ("fp32", torch.float32, scan.fm_scan),
                         ("loop", torch.float32, fm_scan_pytorch)):
        g = gates0.to(dt).clone().requires_grad_()
        x = tokens0.to(dt).clone().requires_grad_()
        states = fn(g, x)
        states.sum().backward()
        res[name] = (states.detach().float().clone(), x.grad.float().clone(), g.grad.float().clone())
    # 2e-2 where bfloat16 is involved: as in the notebook the inputs themselves differ there (the same
    # rand() values rounded to bfloat16 on one side, kept in float32 on the other)
    for a, b, tol in (("fp32", "loop", 1e-5), ("bf16", "loop", 2e-2), ("bf16", "fp32", 2e-2)):
        for ta, tb, what in zip(res[a], res[b], ("states", "token grad", "gate grad")):
            scale = tb.abs().max().item()
            assert (ta - tb).abs().max().item() <= tol * scale, (a, b, what)
    # and the float32 run against the float64 oracle's summed gradients
    d_g, d_x, _ = O.backward(gates0, tokens0, np.ones((1, 1, 5, 32)))
    check("d_gates", res["fp32"][2], d_g, 1e-5)
    check("d_tokens", res["fp32"][1], d_x, 1e-5)


def test_notebook_usage_cell_shape(scan):
    """The reference's usage cell (fm_test.ipynb:29-45): batch 1, dim 2048, seqlen 8192, mem 32, bfloat16;
    fm_scan on gates 0.9 + 0.1 rand and tokens rand, then fm_memory on alpha = softmax(rand), scales
    rand + 0.001, inputs rand, mem_norm, eps 1e-6. The notebook only prints shapes; here the results are
    checked. fm_scan: states and both gradients (upstream gradient randn) against the compiled float64
    oracle on sampled slots and channels, every step of their rows. fm_memory: see below."""
    B, D, L, M, dt = 1, 2048, 8192, 32, torch.bfloat16
    gen = gpu_gen(29)
    gates = (0.9 + 0.1 * torch.rand(B, M, L, device=DEV, generator=gen)).to(dt).requires_grad_()
    tokens = torch.rand(B, D, L, device=DEV, generator=gen).to(dt).requires_grad_()
    states = scan.fm_scan(gates, tokens, initial_state=None)
    assert tuple(states.shape) == (B, M, D, L) and states.dtype == dt
    G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    states.backward(G)
    torch.cuda.synchronize()
    g, x, h = gates.detach(), tokens.detach(), states.detach()
    ms, ds = [0, 13, 31], [0, 1, 777, 2047]
    for m in ms:  # a slot with all its channels: the states of sampled channels, and d_gates (a sum over all d)
        gm, Gm, hm = g[:, m:m + 1], G[:, m:m + 1], h[:, m:m + 1]
        h_ref = C.forward_f64(gm, x[:, ds])
        check(f"states of slot {m}", hm[:, :, ds], h_ref, TOL[dt])
        _, gg = C.backward_f64(gm, Gm, hm, x, None, np.zeros((B, 1, D)))
        check(f"d_gates of slot {m}", gates.grad[:, m:m + 1], gg.sum(axis=2), TOL[dt])
    tg, _ = C.backward_f64(g, G[:, :, ds].contiguous(), h[:, :, ds].contiguous(), x[:, ds].contiguous(), None,
                           np.zeros((B, M, len(ds))))
    check("d_tokens of sampled channels", tokens.grad[:, ds], tg.sum(axis=1), TOL[dt])
    del G, states, h, tg
    gates.grad = tokens.grad = None
    torch.cuda.empty_cache()

    # fm_memory at the same shape. The float64 oracle of the whole layer on 2^29 states would take minutes
    # and tens of GiB, so the check leans on causality: outputs and memory states up to step T0 depend on
    # the inputs up to T0 only, and with a loss that weighs the output up to T0 only, every gradient is
    # that of the layer cut at T0 (and exactly zero afterwards). The oracle runs on that cut, 640 steps: a
    # whole tile of 512 and a part of the next. The kernels run over all 8192 steps of the D = 2048 route
    # (scan with the sums of squares per block of rows, groups of 8 channels in backward).
    T0 = 640
    alpha = torch.softmax(torch.rand(B, L, M, device=DEV, generator=gen).to(dt).float(), -1).to(dt).requires_grad_()
    us = (torch.rand(B, L, 1, device=DEV, generator=gen) + 0.001).to(dt).requires_grad_()
    osc = (torch.rand(B, L, 1, device=DEV, generator=gen) + 0.001).to(dt).requires_grad_()
    inp = torch.rand(B, L, D, device=DEV, generator=gen).to(dt).requires_grad_()
    out, mem = scan.fm_memory(alpha, us, osc, inp, initial_state=None, mem_norm=True, norm_eps=1e-6)
    assert tuple(out.shape) == (B, L, D) and tuple(mem.shape) == (B, M, D, L) and out.dtype == dt
    w = torch.randn(B, L, D, device=DEV, generator=gen).to(dt)
    w[:, T0:] = 0
    (out.float() * w.float()).sum().backward()
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all() and torch.isfinite(mem.float()).all()
    rounded = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dt).to(torch.float64).numpy()
    cut = lambda t: t.detach()[:, :T0].double().cpu()
    a, u, o, xi, wc = cut(alpha), cut(us), cut(osc), cut(inp), cut(w)
    o_out, o_mem = O.memory_forward(a, u, o, xi, None, True, 1e-6, rounded)
    want = O.memory_backward(a, u, o, xi, wc, None, None, True, 1e-6, rounded)
    check("fm_memory output up to T0", out[:, :T0], o_out, TOL[dt])
    check("fm_memory memory states up to T0", mem[..., :T0], o_mem, TOL[dt])
    for name, leaf in (("d_alpha", alpha), ("d_update_scale", us), ("d_output_scale", osc), ("d_inputs", inp)):
        check(f"fm_memory {name} up to T0", leaf.grad[:, :T0], want[name], TOL[dt])
        assert not leaf.grad[:, T0:].float().abs().max().item(), name + " beyond the last weighted step"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_autograd_with_initial_state(scan, dtype):
    """FM_Scan with a non-zero initial state: gradients equal the derivative of the
    recurrence (what autograd gives through the per-timestep form), the one for the
    initial state included (the reference's CUDA path leaves that one unconnected)."""
    B, M, D, L = 2, 3, 4, 256
    gen = torch.Generator().manual_seed(11)
    g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 1).to(dtype).to(DEV).requires_grad_()
    x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV).requires_grad_()
    h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV).requires_grad_()
    G = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
    states = scan.fm_scan(g, x, h0)
    assert states.shape == (B, M, D, L) and states.dtype == dtype
    states.backward(G)
    tg, gg = C.backward_f64(g, G, states, x, None, h0)
    check("states", states, C.forward_f64(g, x, h0), TOL[dtype])
    check("d_gates", g.grad, gg.sum(axis=2), TOL[dtype])
    check("d_tokens", x.grad, tg.sum(axis=1), TOL[dtype])
    _, _, d_h0 = O.backward(g, x, G, h0, states=states)
    check("d_initial_state", h0.grad, d_h0, TOL[dtype])
    # without a gradient request for the initial state the third gradient stays None
    g2, x2 = g.detach().clone().requires_grad_(), x.detach().clone().requires_grad_()
    scan.fm_scan(g2, x2, h0.detach()).backward(G)
    assert torch.equal(g2.grad, g.grad) and torch.equal(x2.grad, x.grad)


def test_seven_argument_backward_reproduces_reference_kernel(scan):
    """fm_scan_backward with the reference's seven arguments uses firstPropGrad as the
    state before the first step (reference fm_scan.cuh:196,380)."""
    B, M, D, L, dt = 2, 2, 2, 64, torch.float32
    gen = torch.Generator().manual_seed(12)
    g = torch.rand(B, M, L, generator=gen).to(DEV)
    x = torch.randn(B, D, L, generator=gen).to(DEV)
    G = torch.randn(B, M, D, L, generator=gen).to(DEV)
    h0 = torch.randn(B, M, D, generator=gen).to(DEV)
    fpg = torch.randn(B, M, D, generator=gen).to(DEV)
    out = torch.empty(B, M, D, L, device=DEV)
    assert scan.fm_scan_forward(g, x, h0, out) is out
    dx, dg = torch.empty_like(out), torch.empty_like(out)
    assert scan.fm_scan_backward(g, G, fpg, dx, out, x, dg) is None
    tg, gg, _ = O.backward_per_row(g, G, out, x, fpg, None)
    check("token grad", dx, tg, 1e-5)
    check("gate grad", dg, gg, 1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mem_norm", [True, False])
def test_readout_kernels(scan, dtype, mem_norm):
    """RMS norm + read-out and their gradients (four kernels) against the float64 oracle on
    the same quantised inputs; shapes cover ragged tiles, D beyond and below a block's 16
    rows, and lengths that force the element path."""
    for (B, M, D, L), with_ext in [((2, 3, 5, 512), True), ((1, 2, 16, 8), False), ((2, 4, 40, 4096), True),
                                   ((1, 33, 17, 1000), False), ((3, 2, 9, 2055), True),
                                   ((1, 5, 130, 640), False)]:
        gen = torch.Generator().manual_seed(B * 1000 + D)
        states = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV)
        read = torch.randn(B, M, L, generator=gen).to(dtype).to(DEV)
        out_grad = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        ext = torch.randn(B, M, D, L, generator=gen).to(dtype).to(DEV) if (with_ext and mem_norm) else None
        eps = 1e-6
        out, normed, inv_rms = scan.fm_readout_forward(states, read, mem_norm, eps)
        o_out, o_normed, o_inv = O.readout_forward(states, read, mem_norm, eps)
        tag = f"{(B, M, D, L)} {dtype} norm={mem_norm}"
        check(tag + " output", out, o_out, TOL[dtype])
        if mem_norm:
            check(tag + " normalised states", normed, o_normed, TOL[dtype])
            check(tag + " inv_rms", inv_rms, o_inv, 1e-5)
        else:
            assert normed is None and inv_rms is None
        # gradients: the kernels work from the stored (rounded) normalised states, the oracle
        # from exact ones; the difference is inside the storage type's tolerance
        states_n = normed if mem_norm else states
        d_states, d_read = scan.fm_readout_backward(out_grad, ext, read, states_n, inv_rms)
        o_ds, o_dr = O.readout_backward(out_grad, ext, read, states, mem_norm, eps)
        check(tag + " d_states", d_states, o_ds, TOL[dtype])
        check(tag + " d_read", d_read, o_dr, TOL[dtype])


def test_readout_in_place_and_determinism(scan):
    B, M, D, L, dt = 2, 8, 64, 2048, torch.bfloat16
    gen = gpu_gen(5)
    states = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    read = torch.randn(B, M, L, device=DEV, generator=gen).to(dt)
    out1, n1, r1 = scan.fm_readout_forward(states, read)
    out2, n2, r2 = scan.fm_readout_forward(states, read)
    assert torch.equal(out1, out2) and torch.equal(n1, n2) and torch.equal(r1, r2)
    # in place through the C interface: states_out == states
    lib = scan.module
    buf = states.clone()
    out3 = torch.empty_like(out1)
    rc = lib.fmscan_readout_forward(buf.data_ptr(), r1.data_ptr(), read.data_ptr(), buf.data_ptr(),
                                    out3.data_ptr(), B, M, D, L, 2, torch.cuda.current_stream().cuda_stream)
    assert rc == 0
    torch.cuda.synchronize()
    assert torch.equal(buf, n1) and torch.equal(out3, out1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mem_norm", [True, False])
def test_layer_backward_kernel_equals_the_two_step_route(scan, dtype, mem_norm):
    """fmscan_backward_layer (states' gradient made inside the scan's backward kernel) against
    fmscan_readout_backward followed by fmscan_backward_reduced, and against the oracle."""
    for (B, M, D, L) in [(2, 3, 5, 512), (1, 2, 16, 8), (2, 4, 24, 4096), (1, 5, 9, 1000), (2, 3, 4, 2568)]:
        gen = torch.Generator().manual_seed(7 * M + D)
        g = torch.sigmoid(torch.randn(B, M, L, generator=gen) + 2).to(dtype).to(DEV)
        x = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        h0 = torch.randn(B, M, D, generator=gen).to(dtype).to(DEV)
        read = torch.randn(B, M, L, generator=gen).to(dtype).to(DEV)
        og = torch.randn(B, D, L, generator=gen).to(dtype).to(DEV)
        zeros = torch.zeros(B, M, D, dtype=dtype, device=DEV)
        states = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        scan.fm_scan_forward(g, x, h0, states)
        out, normed, inv_rms = scan.fm_readout_forward(states, read, mem_norm, 1e-5)
        states_n = normed if mem_norm else states
        # two steps: a (B, M, D, L) gradient in between
        sg, d_read = scan.fm_readout_backward(og, None, read, states_n, inv_rms)
        dh0_a = torch.empty_like(zeros)
        dg_a, dx_a = scan.fm_scan_backward_reduced(g, sg, zeros, states, x, initial_state=h0, initial_state_grad=dh0_a)
        # one step, through the autograd node
        leaves = [t.clone().requires_grad_() for t in (g, x, h0, read)]
        out_b, _ = scan.fm_layer(*leaves[:3], leaves[3], mem_norm, 1e-5)
        # (the one node runs scan and norm as one kernel where it can: its sum of squares is
        # taken in another order, so the outputs agree to rounding, not to the bit)
        check("output vs separate calls", out_b, out.double().cpu().numpy(), TOL[dtype])
        out_b.backward(og)
        tag = f"{(B, M, D, L)} {dtype} norm={mem_norm}"
        tol = 2 * TOL[dtype]  # two rounded results against each other, each within TOL of the exact one
        check(tag + " d_gates vs two steps", leaves[0].grad, dg_a.double().cpu().numpy(), tol)
        check(tag + " d_tokens vs two steps", leaves[1].grad, dx_a.double().cpu().numpy(), tol)
        check(tag + " d_initial_state vs two steps", leaves[2].grad, dh0_a.double().cpu().numpy(), tol)
        check(tag + " d_read vs two steps", leaves[3].grad, d_read.double().cpu().numpy(), tol)
        tol = TOL[dtype]
        # oracle: read-out gradient, then the scan's
        o_sg, o_dr = O.readout_backward(og, None, read, states, mem_norm, 1e-5)
        tg, gg, delta = O.backward_per_row(g, o_sg, states, x, None, h0, False)
        check(tag + " d_gates", leaves[0].grad, gg.sum(axis=2), tol)
        check(tag + " d_tokens", leaves[1].grad, tg.sum(axis=1), tol)
        check(tag + " d_read", leaves[3].grad, o_dr, tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("plain", [False, True])
def test_layer_form_of_the_backward_kernel_through_the_c_abi(scan, dtype, plain):
    """fmscan_backward_layer with arbitrary coefficient vectors, with the saved states or with rms in
    their place, plain form included, against fmscan_backward_reduced fed the states' gradient
    G = coef_out * out_grad - coef_self * states_n as a tensor. Blocks of 4 rows and of 8."""
    lib = scan.module
    st = torch.cuda.current_stream().cuda_stream
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    flags = 1 if plain else 0
    P = lambda t: t.data_ptr()
    for (B, M, D, L) in [(2, 5, 12, 520), (64, 3, 60, 40), (16, 6, 256, 1032)]:
        gen = gpu_gen(B + M + D)
        g = torch.sigmoid(torch.randn(B, M, L, device=DEV, generator=gen) + 2).to(dtype)
        x = torch.randn(B, D, L, device=DEV, generator=gen).to(dtype)
        og = torch.randn(B, D, L, device=DEV, generator=gen).to(dtype)
        co = torch.randn(B, M, L, device=DEV, generator=gen)
        cs = torch.randn(B, M, L, device=DEV, generator=gen) * 0.3
        rms = torch.rand(B, M, L, device=DEV, generator=gen) + 0.5
        zeros = torch.zeros(B, M, D, dtype=dtype, device=DEV)
        states = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        scan.fm_scan_forward(g, x, zeros, states, plain=plain)
        groups = lib.fmscan_reduced_groups(B, D)
        assert groups == ((D + 7) // 8 if B * ((D + 7) // 8) >= 512 else (D + 3) // 4)
        for recover in (False, True):
            # with rms in place of the saved states, the kernel takes them to be states_n * rms
            states_n = (states.float() / rms.unsqueeze(2)).to(dtype) if recover else states
            saved = (states_n.float() * rms.unsqueeze(2)).to(dtype) if recover else states
            G = (co.unsqueeze(2) * og.float().unsqueeze(1) - cs.unsqueeze(2) * states_n.float()).to(dtype)
            want_tok = torch.empty(B, D, L, dtype=dtype, device=DEV)
            want_part = torch.empty(B, M, groups, L, device=DEV)
            assert lib.fmscan_backward_reduced(P(g), P(G), P(zeros), P(want_tok), P(saved), P(x), P(want_part), None,
                                               None, B, M, D, L, code, flags, st) == 0
            got_tok, got_part = torch.empty_like(want_tok), torch.empty_like(want_part)
            assert lib.fmscan_backward_layer(P(g), P(states_n), P(co), P(cs), P(og), P(zeros), P(got_tok),
                                             None if recover else P(states), P(rms) if recover else None, P(x),
                                             P(got_part), None, None, B, M, D, L, code, flags, st) == 0, \
                lib.fmscan_last_error()
            tag = f"{(B, M, D, L)} {dtype} plain={plain} recover={recover}"
            # G rounded to the storage type on one side, made in float32 on the other: 2 * TOL
            check(tag + " d_tokens", got_tok, want_tok.double().cpu().numpy(), 2 * TOL[dtype])
            check(tag + " gate gradient", got_part.sum(dim=2), want_part.sum(dim=2).double().cpu().numpy(), 2 * TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_slots_dealt_to_several_blocks(scan, dtype):
    """fmscan_backward_reduced_split and fmscan_backward_layer_split (few batch elements: the slots of
    each dealt to `split` blocks, the token gradient left as float32 partial sums) against the unsplit
    calls on the same inputs: the gate-gradient partials and the initial state's gradient are the same
    numbers (equal bits where both calls form groups of the same size), the token gradient is the
    unsplit one before its rounding. Every divisor of M that leaves a wave a slot, and one that does not.
    The layer form also with its rows cut into segments (two passes: what arrives at a segment from the
    steps after it is composed from step pairs instead of carried along), 2 to 5 of them and no split at
    all: the same to float32 rounding."""
    lib = scan.module
    st = torch.cuda.current_stream().cuda_stream
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    P = lambda t: None if t is None else t.data_ptr()
    for (B, M, D, L), splits in [((1, 16, 20, 1032), (2, 4, 8)), ((3, 12, 9, 520), (2, 3, 6)), ((2, 8, 130, 40), (2,))]:
        gen = gpu_gen(B + M + D + L)
        g = torch.sigmoid(torch.randn(B, M, L, device=DEV, generator=gen) + 2).to(dtype)
        x = torch.randn(B, D, L, device=DEV, generator=gen).to(dtype)
        og = torch.randn(B, D, L, device=DEV, generator=gen).to(dtype)
        G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dtype)
        co = torch.randn(B, M, L, device=DEV, generator=gen)
        cs = torch.randn(B, M, L, device=DEV, generator=gen) * 0.3
        rms = torch.rand(B, M, L, device=DEV, generator=gen) + 0.5
        h0 = torch.randn(B, M, D, device=DEV, generator=gen).to(dtype)
        fpg = torch.randn(B, M, D, device=DEV, generator=gen).to(dtype)
        states = torch.empty(B, M, D, L, dtype=dtype, device=DEV)
        scan.fm_scan_forward(g, x, h0, states)
        states_n = (states.float() / rms.unsqueeze(2)).to(dtype)
        groups = lib.fmscan_reduced_groups(B, D)
        tok = [torch.empty(B, D, L, dtype=dtype, device=DEV) for _ in range(2)]
        part = [torch.empty(B, M, groups, L, device=DEV) for _ in range(2)]
        dh0 = [torch.empty_like(h0) for _ in range(2)]
        assert lib.fmscan_backward_reduced(P(g), P(G), P(fpg), P(tok[0]), P(states), P(x), P(part[0]), P(h0), P(dh0[0]),
                                           B, M, D, L, code, 0, st) == 0, lib.fmscan_last_error()
        assert lib.fmscan_backward_layer(P(g), P(states_n), P(co), P(cs), P(og), P(fpg), P(tok[1]), None, P(rms), P(x),
                                         P(part[1]), P(h0), P(dh0[1]), B, M, D, L, code, 0, st) == 0, lib.fmscan_last_error()
        for split in splits:
            gs = lib.fmscan_reduced_groups(B * split, D)
            tp = [torch.empty(B, D, split, L, device=DEV) for _ in range(2)]
            ps = [torch.empty(B, M, gs, L, device=DEV) for _ in range(2)]
            ds = [torch.empty_like(h0) for _ in range(2)]
            assert lib.fmscan_backward_reduced_split(P(g), P(G), P(fpg), P(tp[0]), P(states), P(x), P(ps[0]), P(h0),
                                                     P(ds[0]), B, M, D, L, split, 1, None, 0, code, 0,
                                                     st) == 0, lib.fmscan_last_error()
            assert lib.fmscan_backward_layer_split(P(g), P(states_n), P(co), P(cs), P(og), P(fpg), P(tp[1]), None, P(rms),
                                                   P(x), P(ps[1]), P(h0), P(ds[1]), B, M, D, L, split, 1, None, 0, code,
                                                   0, st) == 0, lib.fmscan_last_error()
            for k, form in enumerate(("plain call", "layer form")):
                tag = f"{(B, M, D, L)} {dtype} split={split} {form}"
                assert torch.equal(ds[k], dh0[k]), tag + " d_initial_state"
                if gs == groups:
                    assert torch.equal(ps[k], part[k]), tag + " gate-gradient partials"
                else:
                    check(tag + " gate gradient", ps[k].sum(dim=2), part[k].sum(dim=2).double().cpu().numpy(), 1e-5)
                summed = torch.empty(B, D, L, dtype=dtype, device=DEV)
                assert lib.fmscan_sum_groups(P(tp[k]), split, P(summed), B * D, L, code, st) == 0
                # the unsplit call rounds the same float32 sum, made in another order
                check(tag + " d_tokens", summed, tok[k].double().cpu().numpy(), TOL[dtype])
                check(tag + " d_tokens, before the rounding", tp[k].sum(dim=2), tok[k].double().cpu().numpy(), TOL[dtype])
        tile = 256 if dtype == torch.float32 else 512
        for split, segments in [(1, s) for s in range(2, min(5, (L + tile - 1) // tile) + 1)] + [(splits[0], 2)]:
            if segments > (L + tile - 1) // tile:
                continue
            gs = lib.fmscan_reduced_groups(B * split, D)
            tp1, ps1, ds1 = torch.empty(B, D, split, L, device=DEV), torch.empty(B, M, gs, L, device=DEV), torch.empty_like(h0)
            ws = torch.empty(B * M * D * segments * 8, dtype=torch.uint8, device=DEV)
            for saved, r in ((states, None), (None, rms)):  # the states at hand, or taken back from states_n * rms
                for t in (tp1, ps1):
                    t.fill_(float("nan"))
                assert lib.fmscan_backward_layer_split(P(g), P(states_n), P(co), P(cs), P(og), P(fpg), P(tp1), P(saved),
                                                       P(r), P(x), P(ps1), P(h0), P(ds1), B, M, D, L, split, segments,
                                                       P(ws), ws.numel(), code, 0, st) == 0, lib.fmscan_last_error()
                whole_tok, whole_part, whole_dh0 = torch.empty_like(tok[1]), torch.empty_like(part[1]), torch.empty_like(h0)
                assert lib.fmscan_backward_layer(P(g), P(states_n), P(co), P(cs), P(og), P(fpg), P(whole_tok), P(saved),
                                                 P(r), P(x), P(whole_part), P(h0), P(whole_dh0), B, M, D, L, code, 0,
                                                 st) == 0, lib.fmscan_last_error()
                tag = f"{(B, M, D, L)} {dtype} split={split} segments={segments} saved states {saved is not None}"
                check(tag + " d_tokens", tp1.sum(dim=2), whole_tok.double().cpu().numpy(), TOL[dtype])
                check(tag + " gate gradient", ps1.sum(dim=2), whole_part.sum(dim=2).double().cpu().numpy(),
                      1e-5 if dtype == torch.float32 else 1e-4)
                check(tag + " d_initial_state", ds1, whole_dh0.double().cpu().numpy(), TOL[dtype])
            # the call that is given the states' gradient as a tensor, cut the same way
            for t in (tp1, ps1):
                t.fill_(float("nan"))
            assert lib.fmscan_backward_reduced_split(P(g), P(G), P(fpg), P(tp1), P(states), P(x), P(ps1), P(h0), P(ds1),
                                                     B, M, D, L, split, segments, P(ws), ws.numel(), code, 0,
                                                     st) == 0, lib.fmscan_last_error()
            tag = f"{(B, M, D, L)} {dtype} split={split} segments={segments} plain call"
            check(tag + " d_tokens", tp1.sum(dim=2), tok[0].double().cpu().numpy(), TOL[dtype])
            check(tag + " gate gradient", ps1.sum(dim=2), part[0].sum(dim=2).double().cpu().numpy(),
                  1e-5 if dtype == torch.float32 else 1e-4)
            check(tag + " d_initial_state", ds1, dh0[0].double().cpu().numpy(), TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_layer_prepare_and_finish_kernels(scan, dtype):
    """The layer's small tensors: gates and read weights with time last, bit for bit as the
    reference's PyTorch lines form them; and the gradients of alpha and the two scales from those
    of gates (as partial sums) and read, against the same formulas in float64."""
    lib, st = scan.module, torch.cuda.current_stream().cuda_stream
    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    for (B, L, M, G) in [(2, 64, 3, 1), (1, 1000, 33, 2), (3, 130, 70, 3), (2, 2048, 32, 16), (1, 5, 1, 1)]:
        gen = torch.Generator().manual_seed(L + M)
        alpha = torch.softmax(torch.randn(B, L, M, generator=gen), -1).to(dtype).to(DEV)
        us = torch.rand(B, L, 1, generator=gen).to(dtype).to(DEV)
        osc = torch.randn(B, L, 1, generator=gen).to(dtype).to(DEV)
        gates, read = torch.empty(B, M, L, dtype=dtype, device=DEV), torch.empty(B, M, L, dtype=dtype, device=DEV)
        assert lib.fmscan_layer_prepare(alpha.data_ptr(), us.data_ptr(), osc.data_ptr(), gates.data_ptr(),
                                        read.data_ptr(), B, L, M, code, st) == 0
        a64, u64, o64 = (O.to_f64(t) for t in (alpha, us, osc))
        tag = f"{(B, L, M, G)} {dtype}"
        # bit for bit what the reference's lines give (fm_scan.py:116-119,130), evaluated by PyTorch on
        # CPU tensors of the storage type: the product is a tensor of its own, so the gates are
        # rounded twice; and the same from the oracle's layer, which the layer tests compare with
        a_c, u_c, o_c = alpha.cpu(), us.cpu(), osc.cpu()
        want_gates = 1.0 - (a_c * u_c).transpose(1, 2).contiguous()
        want_read = (a_c * o_c).transpose(1, 2).contiguous()
        assert torch.equal(gates.cpu(), want_gates), tag + " gates"
        assert torch.equal(read.cpu(), want_read), tag + " read"
        rounded = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(torch.float64).numpy()
        o_gates, _, o_read = O._layer_operands(a64, u64, o64, np.zeros((B, L, 1)), rounded)
        assert np.array_equal(gates.double().cpu().numpy(), o_gates), tag + " gates vs oracle"
        assert np.array_equal(read.double().cpu().numpy(), o_read), tag + " read vs oracle"
        partial = torch.randn(B, M, G, L, generator=gen).to(DEV)
        q = torch.randn(B, M, L, generator=gen).to(DEV)
        d_alpha, d_us, d_os = torch.empty_like(alpha), torch.empty_like(us), torch.empty_like(osc)
        assert lib.fmscan_layer_finish(partial.data_ptr(), G, q.data_ptr(), alpha.data_ptr(), us.data_ptr(),
                                       osc.data_ptr(), d_alpha.data_ptr(), d_us.data_ptr(), d_os.data_ptr(),
                                       B, L, M, code, st) == 0
        dg = np.transpose(O.to_f64(partial).sum(axis=2), (0, 2, 1))  # (B, L, M)
        dr = np.transpose(O.to_f64(q), (0, 2, 1))
        tol = 1e-5 if dtype == torch.float32 else 4e-3
        check(tag + " d_alpha", d_alpha, dr * o64 - dg * u64, tol)
        check(tag + " d_update_scale", d_us, -(dg * a64).sum(axis=2, keepdims=True), tol)
        check(tag + " d_output_scale", d_os, (dr * a64).sum(axis=2, keepdims=True), tol)


def test_scan_then_readout_equals_the_one_node_layer(scan):
    """fm_scan followed by fm_readout (two autograd nodes, a (B, M, D, L) gradient between them) and
    fm_layer (one node) are the same function: values and gradients within the storage type's
    rounding of each other."""
    B, M, D, L, dt = 2, 4, 24, 2048, torch.bfloat16
    gen = gpu_gen(17)
    mk = lambda *s: torch.randn(*s, device=DEV, generator=gen)
    g0, x0, h0, r0 = torch.sigmoid(mk(B, M, L) + 2).to(dt), mk(B, D, L).to(dt), mk(B, M, D).to(dt), mk(B, M, L).to(dt)
    w = mk(B, D, L).to(dt)
    grads = []
    for route in ("two nodes", "one node"):
        g, x, h, r = (t.clone().requires_grad_() for t in (g0, x0, h0, r0))
        if route == "two nodes":
            out, mem = scan.fm_readout(scan.fm_scan(g, x, h), r, True, 1e-5)
        else:
            out, mem = scan.fm_layer(g, x, h, r, True, 1e-5)
        out.backward(w)
        grads.append([out.detach(), mem.detach(), g.grad, x.grad, h.grad, r.grad])
    for a, b, name in zip(grads[0], grads[1], ("output", "memory states", "d_gates", "d_tokens", "d_initial_state",
                                               "d_read")):
        check(name, b, a.double().cpu().numpy(), 2e-2)  # two bfloat16 results against each other


def test_layer_keeps_no_second_copy_of_the_states(scan):
    """With the norm, backward works from the normalised states the layer returns (and inv_rms):
    the scanned states are not kept. Measured as allocated memory across the forward pass."""
    B, L, M, D, dt = 2, 4096, 8, 64, torch.bfloat16
    gen = gpu_gen(11)
    alpha = torch.softmax(torch.randn(B, L, M, device=DEV, generator=gen), -1).to(dt).requires_grad_()
    us = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt).requires_grad_()
    osc = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt).requires_grad_()
    inp = torch.randn(B, L, D, device=DEV, generator=gen).to(dt).requires_grad_()
    states_bytes = B * M * D * L * 2
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    out, mem = scan.fm_memory(alpha, us, osc, inp)
    torch.cuda.synchronize()
    held = torch.cuda.memory_allocated() - before
    assert states_bytes <= held < 1.5 * states_bytes, (held, states_bytes)
    out.sum().backward()  # and the gradients still come out
    assert all(t.grad is not None and torch.isfinite(t.grad.float()).all() for t in (alpha, us, osc, inp))


def test_swap_last_two_is_exact(scan):
    from fm_amd.scan.fm_scan import _swap_last_two

    for shape, dt in [((2, 5, 7), torch.float32), ((3, 64, 64), torch.bfloat16), ((1, 1000, 33), torch.float16),
                      ((2, 129, 2048), torch.bfloat16), ((1, 1, 1), torch.float32),
                      ((2, 130, 2048), torch.bfloat16), ((3, 2048, 32), torch.float16), ((1, 2, 2), torch.bfloat16),
                      ((2, 300, 258), torch.bfloat16), ((2, 136, 200), torch.bfloat16), ((1, 8, 8), torch.float16),
                      ((2, 2048, 128), torch.bfloat16), ((3, 72, 2056), torch.float16)]:
        t = torch.randn(*shape, device=DEV).to(dt)
        assert torch.equal(_swap_last_two(t), t.transpose(1, 2).contiguous()), (shape, dt)


def test_kernels_follow_the_current_stream(scan):
    """Every call reads torch's current stream when it is made (the reference extension does the
    same, fm_scan.cuh:271): work issued under a side stream is ordered there, not on the
    default stream."""
    B, L, M, D, dt = 2, 2048, 4, 32, torch.bfloat16
    gen = gpu_gen(23)
    alpha = torch.softmax(torch.randn(B, L, M, device=DEV, generator=gen), -1).to(dt)
    us = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt)
    osc = torch.rand(B, L, 1, device=DEV, generator=gen).to(dt)
    inp = torch.randn(B, L, D, device=DEV, generator=gen).to(dt)
    want_out, want_mem = scan.fm_memory(alpha, us, osc, inp)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        # a long-running kernel first: were the layer's kernels on another stream, they would
        # read `late` before it is written
        big = torch.randn(64 * 1024 * 1024, device=DEV)
        for _ in range(8):
            big = big * 1.0001
        late = (inp.float() + big[: inp.numel()].view_as(inp) * 0.0).to(dt)
        out, mem = scan.fm_memory(alpha, us, osc, late)
    side.synchronize()
    assert torch.equal(out, want_out) and torch.equal(mem, want_mem)


def test_calls_can_be_captured_in_a_graph(scan):
    """The entry points only enqueue kernels on the given stream (no allocation, no memset, no
    synchronisation), so a forward + backward pair can be captured once and replayed. Every
    replay is checked against the eager result, with eager work in between."""
    B, M, D, L, dt = 2, 4, 8, 4096, torch.bfloat16
    gen = gpu_gen(3)
    g = torch.rand(B, M, L, device=DEV, generator=gen).to(dt)
    x = torch.randn(B, D, L, device=DEV, generator=gen).to(dt)
    G = torch.randn(B, M, D, L, device=DEV, generator=gen).to(dt)
    z = torch.zeros(B, M, D, dtype=dt, device=DEV)
    out, dx, dg = (torch.empty(B, M, D, L, dtype=dt, device=DEV) for _ in range(3))

    def run():
        scan.fm_scan_forward(g, x, z, out)
        scan.fm_scan_backward(g, G, z, dx, out, x, dg)

    run()
    torch.cuda.synchronize()
    want = [t.clone() for t in (out, dx, dg)]
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()  # warm-up on the capturing stream
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run()
    for k in range(3):
        for t in (out, dx, dg):
            t.fill_(float(k))          # eager work between replays; also wipes the previous results
        x.mul_(1.0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref, name in zip((out, dx, dg), want, ("states", "token grad", "gate grad")):
            assert torch.equal(got, ref), (k, name)


# ----------------------------------------------------------------------------- errors on the GPU

def test_argument_errors_on_gpu(scan):
    g = torch.rand(2, 2, 64, device=DEV)
    x = torch.rand(2, 3, 64, device=DEV)
    z = torch.zeros(2, 2, 3, device=DEV)
    out = torch.empty(2, 2, 3, 64, device=DEV)
    with pytest.raises(RuntimeError, match="dtype"):
        scan.fm_scan_forward(g, x.half(), z, out)
    with pytest.raises(RuntimeError, match="contiguous"):
        scan.fm_scan_forward(g, torch.rand(2, 64, 3, device=DEV).transpose(1, 2), z, out)
    with pytest.raises(RuntimeError, match="Unsupported tensor dtype"):
        scan.fm_scan_forward(g.double(), x.double(), z.double(), out.double())
    with pytest.raises(RuntimeError, match="gates must be"):
        scan.fm_scan_forward(g[:, :1].contiguous(), x, z, out)
    with pytest.raises(RuntimeError, match="overlaps"):
        scan.fm_scan_forward(out.view(-1)[:256].view(2, 2, 64), x, z, out)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        scan.fm_scan_forward(g.cpu(), x, z, out)
    # the calls above launched nothing; a valid call still works afterwards
    scan.fm_scan_forward(g, x, z, out)
    check("states", out, C.forward_f64(g, x), 1e-5)
