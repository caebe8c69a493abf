"""Writes tests/golden/fm_scan_exact.json: small scan problems solved in exact
rational arithmetic, with exact derivatives from forward-mode differentiation.

Nothing from the reference is imported or executed: the recurrence is the one
stated in its sources (fm/scan/fm_pytorch.py:22,37: h_t = g_t h_{t-1} + (1 - g_t) x_t),
evaluated here with `fractions.Fraction`; derivatives come from dual numbers
(value, tangent) pushed through that same recurrence, one input at a time, so no
hand-derived gradient formula enters the expected values. Every stored number is
a dyadic rational that float64 holds exactly (checked on write).

The objective whose gradient is stored, per row (b, m, d):
    loss = sum_t G[t] * h[t] + first_prop_grad * h[L-1]
(first_prop_grad is the gradient that arrives from beyond the last step,
reference fm/scan/fm_scan.cuh:360). Row-level derivatives with respect to that
row's own copy of the gate / token sequence are the (B, M, D, L) tensors the
backward kernel writes; their sums over d / m are d_gates / d_tokens.

    python tests/golden/make_exact_vectors.py
"""
import json
import random
from fractions import Fraction as Fr
from pathlib import Path

OUT = Path(__file__).resolve().parent / "fm_scan_exact.json"


class Dual:
    """value + eps * tangent over the rationals."""

    __slots__ = ("v", "d")

    def __init__(self, v, d=Fr(0)):
        self.v, self.d = Fr(v), Fr(d)

    def __add__(self, o):
        return Dual(self.v + o.v, self.d + o.d)

    def __sub__(self, o):
        return Dual(self.v - o.v, self.d - o.d)

    def __mul__(self, o):
        return Dual(self.v * o.v, self.d * o.v + self.v * o.d)


ONE = Dual(1)


def row_states(g, x, h0, plain):
    """g, x: lists of Dual, h0: Dual -> list of Dual states."""
    h, out = h0, []
    for gt, xt in zip(g, x):
        h = gt * h + (xt if plain else (ONE - gt) * xt)
        out.append(h)
    return out


def row_loss_tangent(g, x, h0, G, fpg, plain, wrt, idx):
    """d loss / d (one input of the row), exactly."""
    gd = [Dual(v, 1 if (wrt == "g" and i == idx) else 0) for i, v in enumerate(g)]
    xd = [Dual(v, 1 if (wrt == "x" and i == idx) else 0) for i, v in enumerate(x)]
    hd = Dual(h0, 1 if wrt == "h0" else 0)
    hs = row_states(gd, xd, hd, plain)
    return sum((Fr(Gt) * h.d for Gt, h in zip(G, hs)), Fr(0)) + Fr(fpg) * hs[-1].d


def exact_float(q):
    f = float(q)
    assert Fr(f) == q, "not exactly representable in float64: %s" % q
    return f


def make_case(name, B, M, D, L, seed, plain, zero_state, special=None):
    rnd = random.Random(seed)
    # gates on a grid of eighths in [0, 1] (0 and 1 included: reset and hold), the rest on quarters
    gate = lambda: Fr(rnd.randint(0, 8), 8)
    val = lambda: Fr(rnd.randint(-8, 8), 4)
    g = [[[gate() for _ in range(L)] for _ in range(M)] for _ in range(B)]
    if special == "gates_above_one":  # the recurrence is not restricted to [0, 1]
        g = [[[Fr(rnd.randint(-12, 12), 8) for _ in range(L)] for _ in range(M)] for _ in range(B)]
    x = [[[val() for _ in range(L)] for _ in range(D)] for _ in range(B)]
    G = [[[[val() for _ in range(L)] for _ in range(D)] for _ in range(M)] for _ in range(B)]
    z = Fr(0)
    h0 = [[[z if zero_state else val() for _ in range(D)] for _ in range(M)] for _ in range(B)]
    fpg = [[[z if zero_state else val() for _ in range(D)] for _ in range(M)] for _ in range(B)]

    shape4 = lambda f: [[[f(b, m, d) for d in range(D)] for m in range(M)] for b in range(B)]
    states = shape4(lambda b, m, d: [h.v for h in row_states(
        [Dual(v) for v in g[b][m]], [Dual(v) for v in x[b][d]], Dual(h0[b][m][d]), plain)])
    grad = lambda wrt: shape4(lambda b, m, d: [row_loss_tangent(
        g[b][m], x[b][d], h0[b][m][d], G[b][m][d], fpg[b][m][d], plain, wrt, t) for t in range(L)])
    gate_grad, token_grad = grad("g"), grad("x")
    d_h0 = shape4(lambda b, m, d: row_loss_tangent(
        g[b][m], x[b][d], h0[b][m][d], G[b][m][d], fpg[b][m][d], plain, "h0", 0))

    def conv(a):
        return [conv(v) for v in a] if isinstance(a, list) else exact_float(a)

    return {"name": name, "B": B, "M": M, "D": D, "L": L, "plain": plain,
            "gates": conv(g), "tokens": conv(x), "out_grad": conv(G), "initial_state": conv(h0),
            "first_prop_grad": conv(fpg), "states": conv(states), "token_grad": conv(token_grad),
            "gate_grad": conv(gate_grad), "d_initial_state": conv(d_h0)}


def main():
    cases = [
        make_case("fm_zero_state", 2, 2, 3, 6, seed=1, plain=False, zero_state=True),
        make_case("fm_with_state", 2, 2, 3, 6, seed=2, plain=False, zero_state=False),
        make_case("fm_single_row", 1, 1, 1, 9, seed=3, plain=False, zero_state=False),
        make_case("fm_length_one", 2, 1, 2, 1, seed=4, plain=False, zero_state=False),
        make_case("plain_with_state", 2, 2, 2, 6, seed=5, plain=True, zero_state=False),
        make_case("fm_gates_outside_unit_interval", 1, 2, 2, 5, seed=6, plain=False, zero_state=False,
                  special="gates_above_one"),
        # rows of 8 float32 = 32 bytes: 16-byte vector access on the GPU, and M > 1 with D > 1 for the
        # backward kernel that sums over d and m itself
        make_case("fm_vector_rows", 2, 3, 2, 8, seed=7, plain=False, zero_state=False),
        make_case("plain_vector_rows", 1, 2, 3, 8, seed=8, plain=True, zero_state=False),
    ]
    OUT.write_text(json.dumps({"cases": cases}, indent=None, separators=(",", ":")) + "\n")
    print("wrote", OUT, OUT.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
