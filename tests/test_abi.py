"""The C-ABI library loads and exports exactly what include/fmscan.h declares; rejected
arguments come back as error codes with a message, before anything touches a GPU."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = (ROOT / "include" / "fmscan.h").read_text()


@pytest.fixture(scope="module")
def lib():
    from fm_amd import _lib

    return _lib.load()


def declared_functions():
    code = re.sub(r"/\*.*?\*/", "", HEADER, flags=re.S)
    return sorted(set(re.findall(r"\b(fmscan_[a-z0-9_]+)\s*\(", code)))


def test_header_declares_the_expected_entry_points():
    assert declared_functions() == ["fmscan_abi_version", "fmscan_backward", "fmscan_backward_layer",
                                    "fmscan_backward_layer_packed", "fmscan_backward_layer_split", "fmscan_backward_reduced",
                                    "fmscan_backward_reduced_packed", "fmscan_backward_reduced_split",
                                    "fmscan_build_id", "fmscan_forward",
                                    "fmscan_forward_normed", "fmscan_forward_normed_cut",
                                    "fmscan_forward_normed_max_d", "fmscan_forward_normed_pays",
                                    "fmscan_forward_normed_segments", "fmscan_forward_static",
                                    "fmscan_forward_sumsq", "fmscan_last_error", "fmscan_layer_finish",
                                    "fmscan_layer_prepare", "fmscan_readout_backward", "fmscan_readout_dot",
                                    "fmscan_readout_forward", "fmscan_readout_inv_rms", "fmscan_reduced_groups",
                                    "fmscan_reduced_packed_groups", "fmscan_reduced_pays", "fmscan_reduced_plan", "fmscan_reduced_split",
                                    "fmscan_sum_groups", "fmscan_sumsq_finish", "fmscan_sumsq_groups",
                                    "fmscan_swap_last_two", "fmscan_workspace_bytes"]


def test_every_declared_symbol_is_exported(lib):
    for name in declared_functions():
        assert hasattr(lib, name), name


def test_abi_version_matches_header(lib):
    want = int(re.search(r"#define\s+FMSCAN_ABI_VERSION\s+(\d+)", HEADER).group(1))
    assert lib.fmscan_abi_version() == want


def _const(name):
    return int(re.search(r"#define\s+%s\s+\(?(-?\w+)\)?" % name, HEADER).group(1), 0)


def test_python_constants_match_header():
    from fm_amd import _lib

    assert _lib.DTYPE_F32 == _const("FMSCAN_DTYPE_F32")
    assert _lib.DTYPE_F16 == _const("FMSCAN_DTYPE_F16")
    assert _lib.DTYPE_BF16 == _const("FMSCAN_DTYPE_BF16")
    assert _lib.FLAG_WAVES_SHIFT == _const("FMSCAN_FLAG_WAVES_SHIFT")
    assert _lib.FLAG_BLOCKS_SHIFT == _const("FMSCAN_FLAG_BLOCKS_SHIFT")
    assert _lib.FLAG_DEPTH_SHIFT == _const("FMSCAN_FLAG_DEPTH_SHIFT")
    assert _lib.FLAG_SEGMENTS_SHIFT == _const("FMSCAN_FLAG_SEGMENTS_SHIFT")
    assert _lib.ABI_VERSION == _const("FMSCAN_ABI_VERSION")
    assert _lib.FLAG_PLAIN == int(re.search(r"FMSCAN_FLAG_PLAIN\s+(0x[0-9a-f]+)u", HEADER).group(1), 16)


P = 1 << 32  # never dereferenced: every call below is rejected by the argument checks


def fwd(lib, g=P, x=2 * P, h0=None, out=3 * P, B=1, M=1, D=1, L=8, dtype=0, flags=0, ws=None, ws_bytes=0):
    return lib.fmscan_forward(g, x, h0, out, B, M, D, L, dtype, flags, ws, ws_bytes, None)


def bwd(lib, g=P, G=2 * P, fpg=None, dx=3 * P, h=4 * P, x=5 * P, dg=6 * P, h0=None, dh0=None, B=1, M=1,
        D=1, L=8, dtype=0, flags=0, ws=None, ws_bytes=0):
    return lib.fmscan_backward(g, G, fpg, dx, h, x, dg, h0, dh0, B, M, D, L, dtype, flags, ws, ws_bytes, None)


def test_rejected_arguments(lib):
    E_NULL, E_SHAPE, E_DTYPE, E_FLAGS, E_ALIAS, E_WORKSPACE, E_UNALIGNED = (
        _const("FMSCAN_E_" + n) for n in ("NULL", "SHAPE", "DTYPE", "FLAGS", "ALIAS", "WORKSPACE", "UNALIGNED"))
    assert fwd(lib, g=None) == E_NULL
    assert b"NULL" in lib.fmscan_last_error()
    assert fwd(lib, out=None) == E_NULL
    assert fwd(lib, L=0) == E_SHAPE
    assert fwd(lib, B=-1) == E_SHAPE
    assert fwd(lib, B=1 << 20, M=1 << 20, D=1 << 20) == E_SHAPE
    assert fwd(lib, dtype=3) == E_DTYPE
    assert b"dtype" in lib.fmscan_last_error()
    assert fwd(lib, flags=0x2) == E_FLAGS
    assert fwd(lib, flags=3 << 8) == E_FLAGS          # 3 waves per row is not offered
    assert fwd(lib, flags=5 << 16) == E_FLAGS         # prefetch depth 5 is not offered
    assert fwd(lib, flags=3 << 16) == E_FLAGS         # nor 3: the library holds depths 2 and 4
    assert fwd(lib, flags=1 << 28) == E_FLAGS         # unknown bit
    assert fwd(lib, L=1 << 16, flags=4 << 20) == E_WORKSPACE   # 4 segments asked for, no workspace
    assert b"workspace" in lib.fmscan_last_error()
    assert fwd(lib, L=1 << 16, flags=4 << 20, ws=7 * P, ws_bytes=8) == E_WORKSPACE  # too small
    assert bwd(lib, L=1 << 16, flags=4 << 20) == E_WORKSPACE
    assert bwd(lib, dh0=4 * P) == E_ALIAS             # initial_state_grad on top of cached_output
    red = lambda **k: lib.fmscan_backward_reduced(
        k.get("g", P), 2 * P, None, k.get("dx", 3 * P), 4 * P, 5 * P, k.get("part", 6 * P), None, None,
        2, 2, k.get("D", 2), k.get("L", 8), k.get("dtype", 0), k.get("flags", 0), None)
    assert red(part=None) == E_NULL
    assert red(flags=1 << 8) == E_FLAGS               # tuning flags do not apply here
    assert red(dx=4 * P) == E_ALIAS
    assert red(L=7) == _const("FMSCAN_E_UNALIGNED")
    assert red(g=P + 4) == _const("FMSCAN_E_UNALIGNED")
    lay = lambda **k: lib.fmscan_backward_layer(
        P, 2 * P, k.get("co", 7 * P), k.get("cs", 8 * P), k.get("og", 9 * P), None, k.get("dx", 3 * P),
        k.get("h", 4 * P), k.get("r", None), 5 * P, 6 * P, None, None, 2, 2, 2, 8, 0, 0, None)
    assert lay(co=None) == E_NULL
    assert lay(cs=None) == E_NULL
    assert lay(og=None) == E_NULL
    assert lay(h=None) == E_NULL                      # no saved states and no inv_rms to take them back with
    assert lay(h=None, r=3 * P) == E_ALIAS            # inv_rms under token_grad
    assert lay(dx=9 * P) == E_ALIAS                   # token_grad on top of the layer's out_grad
    # the same two with the slots of a batch element dealt to `split` blocks
    reds = lambda **k: lib.fmscan_backward_reduced_split(
        P, 2 * P, None, k.get("tp", 3 * P), 4 * P, 5 * P, 6 * P, None, None, 2, 8, 2, k.get("L", 8), k.get("split", 2),
        k.get("segments", 1), k.get("ws", None), k.get("ws_bytes", 0), 0, k.get("flags", 0), None)
    assert reds(split=3) == E_SHAPE                   # 3 does not divide M = 8
    assert reds(split=0) == E_SHAPE
    assert reds(tp=None) == E_NULL                    # the split token gradient has nowhere to go
    assert reds(tp=4 * P) == E_ALIAS                  # token_grad_partial on top of cached_output
    assert reds(L=4096, segments=4) == E_WORKSPACE and reds(L=4096, segments=4, ws=10 * P, ws_bytes=1 << 20, flags=1) == E_FLAGS
    lays = lambda **k: lib.fmscan_backward_layer_split(
        P, 2 * P, k.get("co", 7 * P), 8 * P, 9 * P, None, k.get("tp", 3 * P), 4 * P, None, 5 * P, 6 * P, None, None,
        2, 8, 2, k.get("L", 8), k.get("split", 4), k.get("segments", 1), k.get("ws", None), k.get("ws_bytes", 0), 0,
        k.get("flags", 0), None)
    assert lays(co=None) == E_NULL
    assert lays(split=5) == E_SHAPE
    assert lays(tp=9 * P) == E_ALIAS                  # token_grad_partial on top of the layer's out_grad
    assert lays(segments=2) == E_SHAPE                # one tile of float32: nothing to cut
    assert lays(L=4096, segments=0) == E_SHAPE and lays(L=4096, segments=256) == E_SHAPE
    assert lays(L=4096, segments=4) == E_WORKSPACE    # the segments' step pairs need a workspace
    assert lays(L=4096, segments=4, ws=10 * P, ws_bytes=64) == E_WORKSPACE
    assert lays(L=4096, segments=4, ws=10 * P, ws_bytes=1 << 20, flags=1) == E_FLAGS   # not in the plain form
    assert lays(L=4096, segments=4, ws=3 * P, ws_bytes=1 << 20) == E_ALIAS            # on top of token_grad_partial
    import ctypes
    def plan(*shape):
        sp, sg = ctypes.c_int64(-1), ctypes.c_int64(-1)
        return lib.fmscan_reduced_plan(*shape, ctypes.byref(sp), ctypes.byref(sg)), sp.value, sg.value
    assert plan(32, 32, 128, 2048, 2) == (0, 1, 1) and plan(4, 32, 128, 8192, 2) == (0, 4, 1)
    assert plan(2, 32, 128, 16384, 2) == (0, 8, 1)    # 64 pairs of (b, 4 d): the slots dealt out, no second read
    assert plan(1, 32, 128, 32768, 2) == (0, 1, 16) and plan(1, 16, 64, 65536, 2) == (0, 2, 16)
    assert plan(1, 32, 128, 2048, 2) == (0, 8, 1)     # four tiles: too short to cut
    assert plan(1, 32, 128, 2048, 9)[0] == E_DTYPE and plan(0, 32, 128, 2048, 2) == (E_SHAPE, 0, 0)
    # which split the library asks for: none where (b, group of 4 d) pairs fill the GPU or the slots are few,
    # else the smallest divisor of M that brings the pairs to 512 blocks, every wave of a block keeping a slot
    split = lib.fmscan_reduced_split
    assert split(32, 32, 128) == 1 and split(1, 7, 64) == 1 and split(0, 32, 128) == 0
    assert split(1, 32, 128) == 8 and split(2, 32, 128) == 8 and split(4, 32, 128) == 4 and split(8, 32, 128) == 4 and split(16, 32, 128) == 2
    assert split(1, 16, 64) == 4 and split(3, 12, 20) == 3
    # whether the kernels with the sums inside, or scan and norm in one kernel, are expected to pay
    pays = lib.fmscan_reduced_pays
    assert pays(32, 32, 128, 2048, 2) == 1 and pays(2, 32, 128, 16384, 2) == 1
    assert pays(1, 16, 64, 65536, 2) == 1 and pays(1, 16, 64, 2048, 2) == 0 and pays(4, 1, 64, 2048, 2) == 0
    # rows of up to 256 bytes: fmscan_backward packs several into a wave
    assert pays(512, 32, 128, 64, 2) == 0 and pays(256, 32, 128, 128, 2) == 0 and pays(128, 32, 128, 256, 2) == 1
    assert pays(256, 32, 128, 64, 0) == 0 and pays(256, 32, 128, 68, 0) == 1 and pays(256, 32, 128, 100, 2) == 0
    # the kernel with the sums inside for such rows: groups of the rows a wave holds, 0 where it does not apply
    pg = lib.fmscan_reduced_packed_groups
    assert pg(512, 32, 128, 64, 2) == 16 and pg(256, 32, 128, 128, 2) == 32 and pg(2048, 32, 128, 16, 2) == 4
    assert pg(512, 32, 128, 64, 0) == 32 and pg(128, 32, 128, 256, 2) == 0 and pg(512, 32, 128, 100, 2) == 0
    assert pg(8, 32, 128, 64, 2) == 0 and pg(0, 32, 128, 64, 2) == 0 and pg(512, 32, 128, 64, 9) == 0
    assert lib.fmscan_backward_reduced_packed(P, 2 * P, None, 3 * P, 4 * P, 5 * P, 6 * P, None, None,
                                              8, 32, 128, 64, 2, 0, None) == E_SHAPE   # too few rows for it
    assert lib.fmscan_backward_reduced_packed(P, 2 * P, None, 3 * P, 4 * P, 5 * P, 6 * P, None, None,
                                              512, 32, 128, 64, 2, 2, None) == E_FLAGS
    assert lib.fmscan_backward_reduced_packed(P, 2 * P, None, None, 4 * P, 5 * P, 6 * P, None, None,
                                              512, 32, 128, 64, 2, 0, None) == E_NULL
    assert lib.fmscan_backward_reduced_packed(P + 2, 2 * P, None, 3 * P, 4 * P, 5 * P, 6 * P, None, None,
                                              512, 32, 128, 64, 2, 0, None) == E_UNALIGNED
    assert lib.fmscan_forward_normed_pays(32, 32, 128) == 1 and lib.fmscan_forward_normed_pays(2, 32, 128) == 1
    assert lib.fmscan_forward_normed_pays(1, 32, 128) == 0 and lib.fmscan_forward_normed_pays(1, 8, 2048) == 1
    # scan and norm in one kernel with the sequence cut: no cut without a workspace, no more segments than tiles
    cutn = lambda **k: lib.fmscan_forward_normed_cut(
        P, 2 * P, None, 3 * P, 4 * P, 1, 2, 8, k.get("L", 4096), 0, 1e-6, k.get("segments", 4), k.get("ws", 5 * P),
        k.get("ws_bytes", 1 << 20), None)
    assert cutn(ws=None) == E_WORKSPACE
    assert cutn(ws_bytes=8) == E_WORKSPACE
    assert cutn(ws=5 * P + 4) == E_WORKSPACE
    assert cutn(segments=0) == E_SHAPE and cutn(segments=256) == E_SHAPE
    assert cutn(L=512, segments=3) == E_SHAPE         # two tiles of float32
    assert cutn(ws=3 * P) == E_ALIAS                  # the workspace on top of states_n
    segs = lib.fmscan_forward_normed_segments
    assert segs(32, 32, 128, 2048, 2) == 1 and segs(1, 32, 128, 32768, 2) == 8 and segs(2, 32, 128, 16384, 2) == 4
    assert segs(1, 8, 24, 2048, 2) == 1               # four tiles: too short to cut
    assert segs(1, 8, 24, 4104, 2) == 2 and segs(1, 8, 24, 4104, 0) == 4
    assert segs(1, 8, 200, 4104, 2) == 0 and segs(1, 8, 24, 4104, 7) == 0
    # groups of 8 rows where B * ceil(D / 8) fills the GPU twice over, of 4 otherwise
    assert lib.fmscan_reduced_groups(32, 128) == 16 and lib.fmscan_reduced_groups(1, 128) == 32
    assert lib.fmscan_reduced_groups(2, 9) == 3 and lib.fmscan_reduced_groups(512, 9) == 2 and lib.fmscan_reduced_groups(0, 9) == 0
    assert fwd(lib, out=P) == E_ALIAS                 # out on top of gates
    assert fwd(lib, out=2 * P + 16) == E_ALIAS        # out inside tokens
    assert bwd(lib, h=None) == E_NULL
    assert bwd(lib, x=None) == E_NULL                 # tokens are needed unless plain
    assert bwd(lib, L=0) == E_SHAPE
    assert bwd(lib, dtype=-1) == E_DTYPE
    assert bwd(lib, dx=4 * P) == E_ALIAS              # token_grad_out on top of cached_output
    assert bwd(lib, dg=3 * P) == E_ALIAS              # the two outputs on top of each other
    assert b"overlaps" in lib.fmscan_last_error()


def test_rows_times_segments_must_fit_a_grid(lib):
    """A requested cut that would need 2^31 or more blocks is rejected, not truncated."""
    rows, L, seg = 1 << 24, 1 << 16, 255
    need = rows * seg * 8
    Q = 1 << 44  # each tensor spans 2^41 bytes here
    assert fwd(lib, g=Q, x=2 * Q, out=3 * Q, B=rows, L=L, dtype=2, flags=seg << 20, ws=7 * Q,
               ws_bytes=need) == _const("FMSCAN_E_SHAPE")
    assert b"segments" in lib.fmscan_last_error()
    assert bwd(lib, g=Q, G=2 * Q, dx=3 * Q, h=4 * Q, x=5 * Q, dg=6 * Q, B=rows, L=L, dtype=2, flags=seg << 20,
               ws=7 * Q, ws_bytes=need) == _const("FMSCAN_E_SHAPE")
    assert lib.fmscan_workspace_bytes(rows, 1, 1, L, 2, seg << 20) == 0


def test_error_text_is_per_thread(lib):
    """Two threads issue rejected calls at the same time; each reads its own message afterwards
    (the calls are stateless apart from this per-thread text)."""
    import threading

    barrier = threading.Barrier(2)
    seen = {}

    def worker(name, kwargs, word):
        for _ in range(200):
            barrier.wait()
            rc = fwd(lib, **kwargs)
            barrier.wait()  # the other thread's call has failed too by now
            text = lib.fmscan_last_error()
            if rc >= 0 or word not in text:
                seen[name] = (rc, text)
                break
        else:
            seen[name] = "ok"

    a = threading.Thread(target=worker, args=("a", {"dtype": 7}, b"dtype"))
    b = threading.Thread(target=worker, args=("b", {"g": None}, b"NULL"))
    a.start(); b.start(); a.join(); b.join()
    assert seen == {"a": "ok", "b": "ok"}, seen


def test_build_id_matches_the_sources(lib):
    from fm_amd import build

    lib.fmscan_build_id.restype = ctypes.c_char_p
    assert lib.fmscan_build_id().decode() == build.source_id()


def test_rejected_readout_arguments(lib):
    E_NULL, E_SHAPE, E_DTYPE, E_ALIAS = (_const("FMSCAN_E_" + n) for n in ("NULL", "SHAPE", "DTYPE", "ALIAS"))
    dims = (2, 3, 4, 64)
    rms = lambda s=P, r=2 * P, dims=dims, dtype=2, eps=1e-6: lib.fmscan_readout_inv_rms(s, r, *dims, dtype, eps, None)
    assert rms(s=None) == E_NULL
    assert rms(dims=(2, 3, 0, 64)) == E_SHAPE
    assert rms(dims=(2, 3, 1 << 20, 64)) == E_SHAPE      # D beyond the grid
    assert rms(dtype=5) == E_DTYPE
    assert rms(eps=-1.0) == E_SHAPE
    assert rms(r=P + 64) == E_ALIAS
    fw = lambda s=P, r=2 * P, w=3 * P, so=4 * P, o=5 * P: lib.fmscan_readout_forward(s, r, w, so, o, *dims, 2, None)
    assert fw(w=None) == E_NULL
    assert fw(so=None) == E_NULL                        # the norm needs somewhere to put the states
    assert fw(o=P) == E_ALIAS
    assert fw(so=3 * P) == E_ALIAS                       # normalised states on top of read
    assert b"overlaps" in lib.fmscan_last_error()
    dot = lambda sn=P, og=2 * P, e=None, q=3 * P, qe=None, r=None, w=None, co=None, cs=None, rms=None: \
        lib.fmscan_readout_dot(sn, og, e, q, qe, r, w, co, cs, rms, *dims, 2, None)
    assert dot(q=None) == E_NULL
    assert dot(e=4 * P) == E_NULL                        # ext_grad without qe
    assert dot(e=4 * P, qe=3 * P) == E_ALIAS
    assert dot(co=5 * P) == E_NULL                       # coef_out without coef_self and read
    assert dot(w=6 * P, co=5 * P, cs=5 * P) == E_ALIAS
    assert dot(rms=7 * P) == E_NULL                      # rms_out without inv_rms
    prep = lambda a=P, u=2 * P, o=3 * P, g=4 * P, r=5 * P, M=3: lib.fmscan_layer_prepare(a, u, o, g, r, 2, 64, M, 2, None)
    assert prep(r=None) == E_NULL
    assert prep(M=0) == E_SHAPE
    assert prep(g=P) == E_ALIAS
    fin = lambda p=P, G=2, q=2 * P, a=3 * P, u=4 * P, o=5 * P, da=6 * P, du=7 * P, do=8 * P: \
        lib.fmscan_layer_finish(p, G, q, a, u, o, da, du, do, 2, 64, 3, 2, None)
    assert fin(q=None) == E_NULL
    assert fin(G=0) == E_SHAPE
    assert fin(du=6 * P) == E_ALIAS
    bw = lambda sn=P, r=2 * P, w=3 * P, og=4 * P, e=None, q=5 * P, qe=None, sg=6 * P: \
        lib.fmscan_readout_backward(sn, r, w, og, e, q, qe, sg, *dims, 2, None)
    assert bw(sg=None) == E_NULL
    assert bw(q=None) == E_NULL                          # the norm's gradient needs q
    assert bw(e=7 * P) == E_NULL                         # ... and qe when ext_grad is given
    assert bw(sg=P) == E_ALIAS
    sw = lambda src=P, dst=2 * P, es=2, R=5: lib.fmscan_swap_last_two(src, dst, 2, R, 7, es, None)
    assert sw(dst=None) == E_NULL
    assert sw(es=8) == E_DTYPE
    assert sw(R=0) == E_SHAPE
    assert sw(dst=P + 8) == E_ALIAS


def test_workspace_bytes(lib):
    """Two floats per segment, only for problems with very few rows (or on request)."""
    wb = lib.fmscan_workspace_bytes
    assert wb(16 * 2048, 1, 1, 16384, 2, 0) == 0          # many rows: never cut
    assert wb(4, 1, 1, 65536, 2, 0) == 4 * 32 * 8           # 4 rows of 128 tiles -> 32 segments of 4 tiles
    assert wb(4, 1, 1, 65536, 2, 1 << 20) == 0              # segments = 1: never cut
    assert wb(4, 1, 1, 65536, 2, 8 << 20) == 4 * 8 * 8      # 8 segments on request
    assert wb(1000, 1, 1, 65536, 2, 2 << 20) == 1000 * 2 * 8
    assert wb(4, 1, 1, 512, 2, 0) == 0                      # one tile per row: nothing to cut
    assert wb(4, 1, 1, 65536, 2, 4 << 8) == 0               # caller fixed the waves per row
    assert wb(0, 1, 1, 8, 0, 0) == 0                        # invalid problem


def test_streaming_probe_library_rejects_what_it_does_not_cover():
    """bench.py's bare streaming kernel lives in a library of its own, outside the package (bench.py builds it
    when it is not there); no GPU is needed to see it refuse."""
    import sys
    sys.path.insert(0, str(ROOT))
    import bench

    f = bench.load_probe().fmscan_probe_stream
    from fm_amd import build
    assert not hasattr(build, "PROBE_LIB") and not list((ROOT / "fm_amd").rglob("*probe*"))  # not in the product
    a, b = 1 << 20, 1 << 30
    assert f(None, b, 4, 1024, 2, 1, 2, 1, 0, None) == -1        # no input
    assert f(a, b, 4, 1000, 2, 1, 2, 1, 0, None) == -1           # a row is not whole steps
    assert f(a, b, 4, 1024, 2, 1, 2, 2, 0, None) == -1           # nor whole steps of two waves side by side
    assert f(a, b, 4, 1024, 1, 1, 2, 1, 0, None) == -1           # a stream count it has no kernel for
    assert f(a, b, 4, 1024, 3, 2, 3, 1, 0, None) == -1           # a prefetch depth it has no kernel for
    assert f(a, b, 4, 4096, 3, 2, 2, 3, 0, None) == -1           # three waves per row: not offered
    assert f(a, b, 4, 1024, 3, 2, 2, 1, 16, None) == -1          # a cap beyond 15 blocks
    assert f(a + 8, b, 4, 1024, 3, 2, 2, 1, 0, None) == -1       # not 16-byte aligned


def test_rejected_sum_groups_arguments(lib):
    f = lib.fmscan_sum_groups
    f.restype = ctypes.c_int
    f.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
                  ctypes.c_void_p]
    a, b = 1 << 30, 1 << 44
    assert f(None, 4, b, 8, 64, 2, None) == -1            # FMSCAN_E_NULL
    assert f(a, 0, b, 8, 64, 2, None) == -2               # FMSCAN_E_SHAPE: no group
    assert f(a, 4, b, 8, 64, 7, None) == -3               # FMSCAN_E_DTYPE
    assert f(a, 4, a + 64, 8, 64, 2, None) == -5          # FMSCAN_E_ALIAS: out inside partial
