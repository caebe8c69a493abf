#!/usr/bin/env python3
"""Benchmark of the Factorization-Memory scan on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg3]

One step = one forward scan + one backward scan over one batch of synthetic
input that is already resident in HBM, through the extension entry points
(`fm_scan_forward`, `fm_scan_backward`: ctypes -> C ABI -> HIP kernels) on
pre-allocated outputs. The default workload is the headline configuration:
bfloat16, (B, C, T) = (16, 2048, 16384), passed as B' = B*C rows with M = D = 1.

Prints one JSON line. `value` is the effective HBM bandwidth of the step:
algorithmic bytes (9 * element size per element: forward reads g, x and writes h;
backward reads g, dL/dh, h, x and writes the two gradients) divided by wall
time over K steps that hold nothing but the calls. `roofline` prices the backward
kernel, the dominant one, from HIP events recorded around it in a second pass of the
same K steps right after. `cpu_baseline` times the compiled CPU
port of the same scan (oracle/fmscan_cpu.c) on this host's cores on a bounded
row sample of the same workload.

The default run also carries `per_config`: the same step timed the same way on the other
benchmark configurations (cfg1, cfg2, cfg4, cfg5, cfg5 in float16) and on the layer, after the
headline's timed region (20 steps each; `--workload X` prints the full line for one of them).

`--workload layer` is a secondary measurement, the Factorization-Memory layer
around the scan (`fm_memory`: scan, RMS norm over D, read-out over M) at the
FM-native reading of configuration 5, (B, L, M, D) = (32, 2048, 32, 128) bfloat16:
one step = forward + backward through autograd; the line also carries each
kernel's own time and bandwidth from direct calls.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_HBM_GBPS = 8000.0  # MI355X HBM3E, published

METRIC = "fwd+bwd scan effective HBM GB/s (% of MI355X peak), bf16 B16 C2048 T16384"

# (B, C, T, dtype name, gate law)
WORKLOADS = {
    "cfg1": (2, 64, 1024, "float32"),
    "cfg2": (8, 1024, 4096, "float32"),
    "cfg3": (16, 2048, 16384, "bfloat16"),
    "cfg4": (4, 1024, 65536, "bfloat16"),
    "cfg5": (32, 4096, 2048, "bfloat16"),
    "cfg5f16": (32, 4096, 2048, "float16"),  # configuration 5 in its other 16-bit type
}

STORAGE = {"bfloat16": "bf16", "float32": "f32", "float16": "f16"}


def profiled_traffic(stem, kernel, copy_bytes):
    """HBM bytes per launch of `kernel` (parts of its name, joined by *) from the rocprofv3 counter
    summaries kept under profiles/:
    FETCH_SIZE + WRITE_SIZE (KiB per dispatch), each scaled by what the same counter reads in the
    same run for an elementwise copy of known size (torch.neg, `copy_bytes` read and written).
    Returns (bytes or None, what it was read from)."""
    total, used = 0.0, []
    for counter in ("fetch_size", "write_size"):
        path = ROOT / "profiles" / f"{stem}_pmc_{counter}.txt"
        if not path.exists():
            return None, f"profiles/{path.name} is not there"
        copy_kib, kernel_kib = None, None
        for line in path.read_text().splitlines():
            cols = line.split()
            if len(cols) < 6 or cols[-5].upper() != counter.upper():
                continue
            name, avg = " ".join(cols[:-5]), float(cols[-3])
            if "neg_kernel" in name:  # the probe's copy (the row with four launches)
                copy_kib = avg if int(cols[-4]) >= 4 else copy_kib
            elif all(part in name for part in kernel.split("*")):
                kernel_kib = avg
        if not copy_kib or kernel_kib is None:
            return None, f"profiles/{path.name} has no row for {kernel} or for the copy"
        total += kernel_kib * (copy_bytes / 1024.0 / copy_kib) * 1024.0
        used.append(f"profiles/{path.name}")
    return int(total), " + ".join(used)


PROBE_SRC = ROOT / "bench_stream_probe.hip"
PROBE_LIB = ROOT / "bench_stream_probe.so"


def build_probe(verbose=False):
    """Compiles the bare streaming kernel this benchmark compares the scan kernels with into a small
    library of its own, beside this file. The product library (fm_amd) does not contain it."""
    import subprocess

    from fm_amd import build as hip_build

    tmp = PROBE_LIB.with_suffix(".so.tmp%d" % os.getpid())
    cmd = [hip_build.hipcc_path(), *hip_build.HIPCC_FLAGS, "-shared", "-o", str(tmp), str(PROBE_SRC)]
    if verbose:
        print("[bench] " + " ".join(cmd), flush=True)
    try:
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode:
            raise RuntimeError("hipcc failed on bench_stream_probe.hip:\n" + res.stderr)
        os.replace(tmp, PROBE_LIB)
    finally:
        tmp.unlink(missing_ok=True)
    return PROBE_LIB


def load_probe():
    """The streaming probe, built first when it is missing or older than its source."""
    import ctypes

    if not PROBE_LIB.exists() or PROBE_LIB.stat().st_mtime < PROBE_SRC.stat().st_mtime:
        build_probe()
    lib = ctypes.CDLL(str(PROBE_LIB))
    lib.fmscan_probe_stream.restype = ctypes.c_int
    lib.fmscan_probe_stream.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                        ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                        ctypes.c_void_p]
    return lib


def streaming_copy(torch, rows, row_bytes, fwd_ms, bwd_ms, reps=5):
    """What a bare streaming kernel with the scan kernels' access pattern reaches on the same shape.

    `bench_stream_probe.so` (bench_stream_probe.hip, beside this file) walks `rows` rows of `row_bytes` bytes,
    reading 2 tensors and writing 1 (the forward scan's streams) or reading 3 and writing 2 (the backward
    scan's), with no arithmetic. It has the scan kernels' three knobs (waves side by side on a row, cap on
    the blocks a compute unit holds, tiles of loads in flight) and is swept over all of them: `best` is the
    fastest combination, `untuned` a wave per row with no cap (the better of the two depths). The published
    8 TB/s is not reachable by any kernel; this is the second reference point for kernels with these streams.
    Timed with events on the current stream."""
    if row_bytes % 1024:
        return None
    lib = load_probe()
    tensor = rows * row_bytes
    src = torch.ones(3 * tensor, dtype=torch.uint8, device="cuda")
    dst = torch.empty(2 * tensor, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    out = {}
    for name, reads, writes in (("forward_streams", 2, 1), ("backward_streams", 3, 2)):
        best, untuned = None, None
        for waves in (1, 2, 4, 8):
            if row_bytes % (1024 * waves):
                continue
            for cap in (0, 1, 2, 4):
                for depth in (2, 4):
                    def launch():
                        rc = lib.fmscan_probe_stream(src.data_ptr(), dst.data_ptr(), rows, row_bytes, reads, writes,
                                                     depth, waves, cap, stream)
                        if rc:
                            raise RuntimeError(f"fmscan_probe_stream returned {rc}")
                    for _ in range(2):
                        launch()
                    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    a.record()
                    for _ in range(reps):
                        launch()
                    b.record()
                    b.synchronize()
                    ms = a.elapsed_time(b) / reps
                    if best is None or ms < best[0]:
                        best = (ms, waves, cap, depth)
                    if waves == 1 and cap == 0 and (untuned is None or ms < untuned):
                        untuned = ms
        gbps = lambda ms: round((reads + writes) * tensor / (ms * 1e-3) / 1e9, 1)
        out[name] = {"reads": reads, "writes": writes,
                     "best": {"ms": round(best[0], 4), "GBps": gbps(best[0]), "waves_per_row": best[1],
                              "blocks_per_cu": best[2] or "no cap", "depth": best[3]},
                     "untuned": {"ms": round(untuned, 4), "GBps": gbps(untuned)}}
    # the scan kernels on the bytes they move, over the best bare kernel with the same streams
    out["forward_kernel_over_copy"] = round(out["forward_streams"]["best"]["ms"] / fwd_ms, 3)
    out["backward_kernel_over_copy"] = round(out["backward_streams"]["best"]["ms"] / bwd_ms, 3)
    return out


def make_inputs(torch, name, device):
    B, Cn, T, dtn = WORKLOADS[name]
    dt = getattr(torch, dtn)
    rows = B * Cn
    gen = torch.Generator(device=device).manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=device, generator=gen)
    ru = lambda *s: torch.rand(*s, device=device, generator=gen)
    if name == "cfg5f16":
        name = "cfg5"
    if name == "cfg1":
        g = torch.sigmoid(rn(rows, 1, T) + 2.0)
        x = rn(rows, 1, T)
    elif name == "cfg2":
        g = 0.9 + 0.1 * ru(rows, 1, T)
        x = rn(rows, 1, T)
    elif name == "cfg3":
        g = 1.0 - torch.exp(-torch.nn.functional.softplus(rn(rows, 1, T)))
        x = rn(rows, 1, T)
    elif name == "cfg4":
        g = 0.99 + 0.01 * ru(rows, 1, T)
        g[ru(rows, 1, T) < 0.01] = 0.0
        x = 0.1 * rn(rows, 1, T)
    else:
        g = torch.exp(-torch.exp(-6.0 * ru(1, Cn, 1))).expand(B, Cn, T).reshape(rows, 1, T)
        x = rn(rows, 1, T) * rn(rows, 1, T) / 128.0
    G = rn(rows, 1, 1, T)
    return g.to(dt).contiguous(), x.to(dt).contiguous(), G.to(dt).contiguous()


def cpu_baseline(torch, g, x, G, budget_s=12.0):
    """Times the CPU port on the first rows of the workload (at most 1/8 of them)."""
    sys.path.insert(0, str(ROOT / "oracle"))
    import fmscan_cpu as C

    rows, _, T = g.shape
    n = max(1, min(rows, max(rows // 8, 128)))
    gc, xc, Gc = g[:n].cpu().contiguous(), x[:n].cpu().contiguous(), G[:n].cpu().contiguous()
    out = torch.empty(n, 1, 1, T, dtype=g.dtype)
    dx, dg = torch.empty_like(out), torch.empty_like(out)
    threads = C.max_threads()

    def one_pass():
        C.port_forward(gc, xc, None, out)
        C.port_backward(gc, Gc, None, dx, out, xc, dg)

    one_pass()  # warm up: thread pool, page faults of the outputs
    passes, t0 = 0, time.perf_counter()
    while True:
        one_pass()
        passes += 1
        el = time.perf_counter() - t0
        if (el >= budget_s and passes >= 3) or el >= 2.5 * budget_s:
            break
    s = g.element_size()
    gbps = 9 * s * n * T * passes / el / 1e9
    return {"value": round(gbps, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "elements_per_s": round(n * T * passes / el, 1),
            "sample": f"first {n} of {rows} rows x T={T} ({g.dtype}), fwd+bwd, {passes} passes in "
                      f"{el:.1f} s, C port oracle/fmscan_cpu.c with OpenMP over rows"}


def reference_cpu_path(torch, g, x, G):
    """Config 1 only: the per-timestep PyTorch form (the counterpart of the reference's CPU path,
    fm/scan/fm_pytorch.py: a Python loop over t, backward by autograd) on the host cores."""
    from fm.scan.fm_pytorch import fm_scan_pytorch

    gc = g.float().cpu().requires_grad_()
    xc = x.float().cpu().requires_grad_()
    Gc = G.float().cpu()
    t0 = time.perf_counter()
    states = fm_scan_pytorch(gc, xc)
    t1 = time.perf_counter()
    states.backward(Gc)
    t2 = time.perf_counter()
    n = states.numel()
    return {"value": round(36 * n / (t2 - t0) / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(),
            "kind": "per-timestep torch loop with autograd (fm_amd/scan/fm_pytorch.py)",
            "elements_per_s": round(n / (t2 - t0), 1), "fwd_s": round(t1 - t0, 3), "bwd_s": round(t2 - t1, 3)}


def scan_buffers(torch, g, x, G, waves_per_row=0):
    """Pre-allocated outputs of one workload and the step over them: one forward scan and one
    backward scan through the extension entry points, optionally with events around each."""
    from fm.scan.fm_scan import fm_scan_backward, fm_scan_forward

    rows, _, T = g.shape
    zeros = torch.zeros(rows, 1, 1, dtype=g.dtype, device=g.device)
    out = torch.empty(rows, 1, 1, T, dtype=g.dtype, device=g.device)
    dx, dg = torch.empty_like(out), torch.empty_like(out)

    def step(ev=None):
        if ev:
            ev[0].record()
        fm_scan_forward(g, x, zeros, out, waves_per_row=waves_per_row)
        if ev:
            ev[1].record()
        fm_scan_backward(g, G, zeros, dx, out, x, dg, waves_per_row=waves_per_row)
        if ev:
            ev[2].record()

    return zeros, out, dx, dg, step


def time_steps(torch, step, steps, warmup):
    """(wall seconds of `steps` steps that hold nothing but the calls, forward kernel ms, backward
    kernel ms). The split between the two kernels comes from a pass of its own right after: the
    kernels run on torch's current stream, so torch events bracket them (kept out of the timed steps,
    where they would be extra work in the stream)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    for k in range(steps):
        step(events[k])
    torch.cuda.synchronize()
    fwd_ms = sum(e[0].elapsed_time(e[1]) for e in events) / steps
    bwd_ms = sum(e[1].elapsed_time(e[2]) for e in events) / steps
    return elapsed, fwd_ms, bwd_ms


def per_config(torch, dev, skip, steps, warmup):
    """Every benchmark configuration but `skip` (the headline, timed before), and the layer: the same
    step, the same timing, fewer fields. Effective GB/s prices a step at 9 element sizes per element
    (forward 3, backward 6), moved GB/s at the 8 the kernels move."""
    out = {}
    for name, (B, Cn, T, dtn) in WORKLOADS.items():
        if name == skip:
            continue
        g, x, G = make_inputs(torch, name, dev)
        buffers = scan_buffers(torch, g, x, G)
        elapsed, fwd_ms, bwd_ms = time_steps(torch, buffers[-1], steps, warmup)
        s, N = g.element_size(), B * Cn * T
        ms = elapsed * 1e3 / steps
        out[name] = {"workload": f"(B,C,T)=({B},{Cn},{T}) {dtn}", "ms_per_step": round(ms, 4),
                     "GBps": round(9 * s * N / ms / 1e6, 1), "pct_of_peak": round(9 * s * N / ms / 1e6 / PEAK_HBM_GBPS * 100, 2),
                     "moved_GBps": round(8 * s * N / ms / 1e6, 1), "elements_per_s": round(N / ms * 1e3, 1),
                     "fwd_ms": round(fwd_ms, 4), "bwd_ms": round(bwd_ms, 4),
                     "fwd_frac_of_peak": round(3 * s * N / fwd_ms / 1e6 / PEAK_HBM_GBPS, 4),
                     "bwd_frac_of_peak": round(6 * s * N / bwd_ms / 1e6 / PEAK_HBM_GBPS, 4),
                     "bwd_frac_of_moved_bytes": round(5 * s * N / bwd_ms / 1e6 / PEAK_HBM_GBPS, 4)}
        del g, x, G, buffers
        torch.cuda.empty_cache()
        copy = streaming_copy(torch, B * Cn, T * s, fwd_ms, bwd_ms)
        if copy:  # the best bare streaming kernel with the same streams on this shape (see streaming_copy)
            out[name]["best_copy_GBps"] = {"forward_streams": copy["forward_streams"]["best"]["GBps"],
                                           "backward_streams": copy["backward_streams"]["best"]["GBps"]}
            out[name]["fwd_kernel_over_copy"] = copy["forward_kernel_over_copy"]
            out[name]["bwd_kernel_over_copy"] = copy["backward_kernel_over_copy"]
        torch.cuda.empty_cache()
    # the layer: ten launches and PyTorch's allocator per step, so the steps and warm-up of `--workload layer`
    step, N, name = layer_step(torch, dev)
    layer_warmup, layer_steps = max(warmup, 10), max(steps, 50)
    for _ in range(layer_warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(layer_steps):
        step()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) * 1e3 / layer_steps
    out["layer"] = {"workload": name, "steps": layer_steps, "warmup": layer_warmup, "ms_per_step": round(ms, 4),
                    "Gelem_per_s": round(N / ms / 1e6, 2)}
    return out


LAYER = (32, 2048, 32, 128, "bfloat16")  # B, L, M, D


def layer_inputs(torch, dev):
    B, L, M, D, dtn = LAYER
    dt = getattr(torch, dtn)
    gen = torch.Generator(device=dev).manual_seed(0)
    rn = lambda *sh: torch.randn(*sh, device=dev, generator=gen)
    alpha = torch.softmax(rn(B, L, M), -1).to(dt).requires_grad_()
    us = torch.rand(B, L, 1, device=dev, generator=gen).to(dt).requires_grad_()
    osc = torch.rand(B, L, 1, device=dev, generator=gen).to(dt).requires_grad_()
    inp = rn(B, L, D).to(dt).requires_grad_()
    w_out = rn(B, L, D).to(dt)
    return alpha, us, osc, inp, w_out, gen


def layer_step(torch, dev):
    """(step, elements of the states, name): fm_memory forward + backward through autograd."""
    import fm.scan.fm_scan as S

    B, L, M, D, dtn = LAYER
    alpha, us, osc, inp, w_out, _ = layer_inputs(torch, dev)
    leaves = (alpha, us, osc, inp)

    def step():
        out, _ = S.fm_memory(alpha, us, osc, inp)
        out.backward(w_out)
        for t in leaves:
            t.grad = None

    return step, B * M * D * L, f"fm_memory (B,L,M,D)=({B},{L},{M},{D}) {dtn}, mem_norm, fwd+bwd via autograd"


# (B, L, M, D) of the layer off its benchmark shape: the same count of state elements, or half of it, with
# fewer batch elements and longer rows, where the fused kernels' blocks (one per batch element and group of
# channels, or per slot, for the whole sequence) become few
LAYER_SHAPES = [(32, 2048, 32, 128), (8, 8192, 32, 128), (4, 8192, 32, 128), (2, 16384, 32, 128), (1, 32768, 32, 128),
                (1, 65536, 16, 64), (1, 8192, 32, 2048), (64, 1024, 16, 64),
                # short sequences, many batch elements: rows of at most 256 bytes go several to a wave
                (256, 256, 32, 128), (256, 128, 32, 128), (512, 64, 32, 128), (1024, 32, 32, 128), (2048, 16, 32, 128)]


def run_layer_shapes(torch, args) -> int:
    """`--layer-shapes`: the layer's step (fm_memory forward + backward, bfloat16, loss on the output) over
    LAYER_SHAPES, with the routes the library names for each shape. A table on stderr, one JSON line on stdout."""
    import fm.scan.fm_scan as S

    dev = torch.device("cuda", 0)
    dt = torch.bfloat16
    lib = S.module
    rows = []
    shapes = [tuple(int(v) for v in args.layer_shape.split(","))] if args.layer_shape else LAYER_SHAPES
    for (B, L, M, D) in shapes:
        gen = torch.Generator(device=dev).manual_seed(0)
        rn = lambda *sh: torch.randn(*sh, device=dev, generator=gen)
        alpha = torch.softmax(rn(B, L, M), -1).to(dt).requires_grad_()
        us = torch.rand(B, L, 1, device=dev, generator=gen).to(dt).requires_grad_()
        osc = torch.rand(B, L, 1, device=dev, generator=gen).to(dt).requires_grad_()
        inp = rn(B, L, D).to(dt).requires_grad_()
        w_out = rn(B, L, D).to(dt)
        leaves = (alpha, us, osc, inp)
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]

        def step(record=False):
            if record:
                ev[0].record()
            out, _ = S.fm_memory(alpha, us, osc, inp)
            if record:
                ev[1].record()
            out.backward(w_out)
            if record:
                ev[2].record()
            for t in leaves:
                t.grad = None

        for _ in range(5):
            step()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(20):
                step()
            torch.cuda.synchronize()
            ms = (time.perf_counter() - t0) * 1e3 / 20
            best = ms if best is None else min(best, ms)
        fwd = bwd = None
        for _ in range(5):
            step(True)
            torch.cuda.synchronize()
            f, b = ev[0].elapsed_time(ev[1]), ev[1].elapsed_time(ev[2])
            fwd, bwd = (f if fwd is None else min(fwd, f)), (b if bwd is None else min(bwd, b))
        n = B * M * D * L
        from fm_amd.scan.fm_scan import _reduced_plan
        plan = _reduced_plan(B, M, D, L, 2)  # (split, segments) of the layer's backward kernel
        rows.append({"shape": [B, L, M, D], "elements": n, "ms_per_step": round(best, 4), "fwd_ms": round(fwd, 4),
                     "bwd_ms": round(bwd, 4), "Gelem_per_s": round(n / best / 1e6, 1),
                     "sequence_cut_into": int(lib.fmscan_forward_normed_segments(B, M, D, L, 2)),  # 0: D beyond one block
                     "scan_and_norm_in_one_kernel": bool(lib.fmscan_forward_normed_segments(B, M, D, L, 2) > 1
                                                         or lib.fmscan_forward_normed_pays(B, M, D)),
                     "slots_dealt_to_blocks": plan[0], "backward_cut_into": plan[1],
                     "groups_of_d": int(lib.fmscan_reduced_groups(B * plan[0], D)),
                     "several_rows_to_a_wave": bool(lib.fmscan_reduced_packed_groups(B, M, D, L, 2) > 0)})
        del alpha, us, osc, inp, w_out
        torch.cuda.empty_cache()
    print(f"{'(B, L, M, D)':>24s} {'elements':>11s} {'step ms':>8s} {'fwd':>7s} {'bwd':>7s} {'Gelem/s':>8s}  routes",
          file=sys.stderr)
    for r in rows:
        print(f"{str(tuple(r['shape'])):>24s} {r['elements']:11d} {r['ms_per_step']:8.3f} {r['fwd_ms']:7.3f} "
              f"{r['bwd_ms']:7.3f} {r['Gelem_per_s']:8.1f}  "
              f"{'scan + norm in one kernel' if r['scan_and_norm_in_one_kernel'] else 'scan, norm, read-out apart'}"
              f"{', sequence cut in %d' % r['sequence_cut_into'] if r['sequence_cut_into'] > 1 else ''}; "
              f"backward: slots of a batch element in {r['slots_dealt_to_blocks']} block(s), "
              f"{'rows cut in %d, ' % r['backward_cut_into'] if r['backward_cut_into'] > 1 else ''}{r['groups_of_d']} groups of d"
              if not r["several_rows_to_a_wave"] else
              f"{str(tuple(r['shape'])):>24s} {r['elements']:11d} {r['ms_per_step']:8.3f} {r['fwd_ms']:7.3f} "
              f"{r['bwd_ms']:7.3f} {r['Gelem_per_s']:8.1f}  short rows: several to a wave in scan + norm, read-out, dot and backward",
              file=sys.stderr)
    print(json.dumps({"metric": "fm_memory layer forward+backward, elements of the (B,M,D,L) states per second",
                      "unit": "Gelem/s", "dtype": "f32", "storage_dtype": "bf16", "data": "synthetic",
                      "shapes": rows}), flush=True)
    return 0


def run_layer(torch, args) -> int:
    import fm.scan.fm_scan as S

    dev = torch.device("cuda", 0)
    B, L, M, D, dtn = LAYER
    dt = getattr(torch, dtn)
    alpha, us, osc, inp, w_out, gen = layer_inputs(torch, dev)
    rn = lambda *sh: torch.randn(*sh, device=dev, generator=gen)
    leaves = (alpha, us, osc, inp)

    def step():
        out, _ = S.fm_memory(alpha, us, osc, inp)
        out.backward(w_out)
        for t in leaves:
            t.grad = None

    ms_per_step = 0.0
    if not args.probe:
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ms_per_step = (time.perf_counter() - t0) * 1e3 / args.steps

    # every kernel on its own, through the same Python entry points, HIP events around each
    N, s = B * M * D * L, alpha.element_size()
    gates = torch.rand(B, M, L, device=dev, generator=gen).to(dt)
    tokens = rn(B, D, L).to(dt)
    read = rn(B, M, L).to(dt)
    og = rn(B, D, L).to(dt)
    G = rn(B, M, D, L).to(dt)
    zeros = torch.zeros(B, M, D, dtype=dt, device=dev)
    states = torch.empty(B, M, D, L, dtype=dt, device=dev)
    lib, st = S.module, torch.cuda.current_stream().cuda_stream
    inv = torch.empty(B, M, L, device=dev)
    q = torch.empty_like(inv)
    rms = torch.full_like(inv, 1.5)  # 1 / inv_rms (float32): takes the scanned states back from the normalised ones
    normed, sg = torch.empty_like(states), torch.empty_like(states)
    out = torch.empty(B, D, L, dtype=dt, device=dev)
    coef, dtok = rn(B, M, L), torch.empty(B, D, L, dtype=dt, device=dev)  # coefficient vectors are float32
    groups = lib.fmscan_reduced_groups(B, D)  # of 8 (or 4) consecutive d
    partial = torch.empty(B, M, groups, L, device=dev)  # float32
    partial_bytes = 4 * B * M * groups * L
    code = {"float32": 0, "float16": 1, "bfloat16": 2}[dtn]
    P = lambda t: t.data_ptr()
    calls = {
        # what fm_memory runs, forward: scan and norm in one kernel, then the read-out of the normalised states
        "scan_forward_normed_kernel": (s * N, lambda: lib.fmscan_forward_normed(
            P(gates), P(tokens), None, P(normed), P(inv), B, M, D, L, code, 1e-6, st)),
        "readout_forward_kernel (read-out alone)": (s * N, lambda: lib.fmscan_readout_forward(
            P(normed), None, P(read), None, P(out), B, M, D, L, code, st)),
        # backward, with only the output in the loss: the dot products, then the scan's backward kernel in
        # the form that makes the states' gradient itself (no readout_backward_kernel, no G) and takes the
        # scanned states back from the normalised ones (reads one (B,M,D,L) tensor)
        "rowdot_kernel (dot)": (s * N, lambda: lib.fmscan_readout_dot(P(normed), P(og), None, P(q), None, None, None, None, None, None, B, M, D, L, code, st)),
        "scan_backward_reduced_kernel (layer form)": (s * N + partial_bytes, lambda: lib.fmscan_backward_layer(
            P(gates), P(normed), P(coef), P(coef), P(og), P(zeros), P(dtok), None, P(rms), P(tokens), P(partial),
            None, None, B, M, D, L, code, 0, st)),
        # the same steps as separate kernels (what runs for D beyond one block's rows, or with the
        # returned memory states in the loss)
        "scan_forward_kernel": (s * N, lambda: S.fm_scan_forward(gates, tokens, zeros, states)),
        "rowdot_kernel (inv_rms)": (s * N, lambda: lib.fmscan_readout_inv_rms(P(states), P(inv), B, M, D, L, code, 1e-6, st)),
        "readout_forward_kernel": (2 * s * N, lambda: lib.fmscan_readout_forward(
            P(states), P(inv), P(read), P(normed), P(out), B, M, D, L, code, st)),
        "readout_backward_kernel": (2 * s * N, lambda: lib.fmscan_readout_backward(
            P(normed), P(inv), P(read), P(og), None, P(q), None, P(sg), B, M, D, L, code, st)),
        "scan_backward_reduced_kernel": (2 * s * N + partial_bytes, lambda: lib.fmscan_backward_reduced(
            P(gates), P(G), P(zeros), P(dtok), P(states), P(tokens), P(partial), None, None, B, M, D, L, code, 0, st)),
    }
    if args.probe:  # for rocprofv3 --pmc: a copy of known size, then every kernel a few times
        for _ in range(4):
            torch.neg(states, out=sg)
        for _, call in calls.values():
            for _ in range(4):
                call()
        torch.cuda.synchronize()
        print(f"probe: torch.neg reads and writes {states.numel() * s} bytes each; algorithmic bytes: "
              + ", ".join(f"{k} {v[0]}" for k, v in calls.items()))
        return 0

    kernels = {}
    for name, (nbytes, call) in calls.items():
        for _ in range(3):
            call()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        ev[0].record()
        for _ in range(10):
            call()
        ev[1].record()
        torch.cuda.synchronize()
        ms = ev[0].elapsed_time(ev[1]) / 10
        kernels[name] = {"ms": round(ms, 4), "algorithmic_bytes": nbytes, "GBps": round(nbytes / ms / 1e6, 1)}
    dom = kernels["scan_backward_reduced_kernel (layer form)"]
    traffic, traffic_from = profiled_traffic(f"layer_kernels_B{B}_L{L}_M{M}_D{D}_{STORAGE[dtn]}",
                                             "scan_backward_reduced_kernel*, 2, 0>", s * N)
    result = {
        "metric": "fm_memory layer forward+backward, elements of the (B,M,D,L) states per second",
        "value": round(N / (ms_per_step * 1e-3) / 1e9, 2), "unit": "Gelem/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "storage_dtype": STORAGE[dtn], "data": "synthetic",
        "config": {"workload": f"layer: fm_memory (B,L,M,D)=({B},{L},{M},{D}) {dtn}, mem_norm, fwd+bwd via autograd",
                   "elements": N},
        "kernels": kernels,
        "roofline": {"kernel": "scan_backward_reduced_kernel (layer form)", "bound": "hbm", "achieved": dom["GBps"],
                     "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": round(dom["GBps"] / PEAK_HBM_GBPS, 4),
                     "algorithmic_bytes": dom["algorithmic_bytes"], "traffic": traffic, "traffic_from": traffic_from},
    }
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = layer_cpu_baseline(torch, alpha, us, osc, inp, w_out)
    print(json.dumps(result), flush=True)
    return 0


def layer_cpu_baseline(torch, alpha, us, osc, inp, w_out, batch=16):
    """The float64 numpy oracle of the layer (forward, then the gradients of the read-out and of
    the scan) on the first `batch` batch elements of the same inputs: one core, sequential in t."""
    sys.path.insert(0, str(ROOT / "oracle"))
    import numpy as np

    import fm_scan_oracle as O

    a, u, o, x, w = (O.to_f64(t.detach()[:batch]) for t in (alpha, us, osc, inp, w_out))
    t0 = time.perf_counter()
    write = np.ascontiguousarray(np.transpose(a * u, (0, 2, 1)))
    tokens = np.ascontiguousarray(np.transpose(x, (0, 2, 1)))
    read = np.ascontiguousarray(np.transpose(a * o, (0, 2, 1)))
    gates = 1.0 - write
    states = O.forward(gates, tokens)
    out, normed, _ = O.readout_forward(states, read, True, 1e-6)
    state_grad, read_grad = O.readout_backward(np.transpose(w, (0, 2, 1)), None, read, states, True, 1e-6)
    O.backward(gates, tokens, state_grad, states=states)
    el = time.perf_counter() - t0
    n = states.size
    return {"value": round(n / el / 1e9, 4), "unit": "Gelem/s", "cores": 1, "kind": "port",
            "sample": f"first {batch} of {alpha.shape[0]} batch elements ({n} elements of the states), forward + "
                      f"backward once in {el:.1f} s, float64 numpy oracle oracle/fm_scan_oracle.py"}


GRID_ROWS = (256, 2048, 16384, 131072)
GRID_L = (1024, 4096, 16384, 65536)
GRID_NATIVE = ((32, 32, 64, 2048), (8, 16, 64, 16384), (4, 32, 1024, 4096), (1, 32, 1024, 8192))  # (B, M, D, L)
# (B, M, D, L, dtype): rows of at most 1 KiB, which the scan calls put several to a wave; fold mapping
# (M = D = 1) of 2^27 elements at every length, lengths that are not whole 16-byte vectors, and
# Factorization-Memory shapes of the benchmark's slots and channels with short sequences
SHORT_ROW_SHAPES = [
    (4194304, 1, 1, 32, "bfloat16"), (2097152, 1, 1, 64, "bfloat16"), (1048576, 1, 1, 128, "bfloat16"),
    (524288, 1, 1, 256, "bfloat16"), (262144, 1, 1, 512, "bfloat16"), (1048576, 1, 1, 64, "float32"),
    (524288, 1, 1, 256, "float32"), (1342177, 1, 1, 100, "bfloat16"), (262144, 1, 1, 500, "bfloat16"),
    (1048576, 1, 1, 33, "float32"),
    (512, 32, 128, 64, "bfloat16"), (256, 32, 128, 128, "bfloat16"), (128, 32, 128, 256, "bfloat16"),
    (64, 32, 128, 512, "bfloat16"), (128, 32, 128, 128, "float32"),
]


def run_short_rows(torch, args) -> int:
    """`--short-rows`: fmscan_forward and fmscan_backward on SHORT_ROW_SHAPES, the library's choice (several
    rows to a wave) against the general kernels asked for by flag (a row to a wave). A table on stderr, one
    JSON line on stdout; for the shapes with shared gates and tokens also FM_Scan.backward's two routes.
    GB/s counts streams of the size of the (B,M,D,L) tensor: 3 forward and 6 backward in the
    fold mapping (the metric's model), 1 and 4 where gates and tokens are shared (states written; two tensors read
    and two written), for both columns alike."""
    import fm.scan.fm_scan as S

    dev = torch.device("cuda", 0)

    def timed(call, reps):
        for _ in range(3):
            call()
        best = None
        for _ in range(3):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                call()
            b.record()
            b.synchronize()
            ms = a.elapsed_time(b) / reps
            best = ms if best is None else min(best, ms)
        return best

    rows = []
    for (B, M, D, L, dtn) in SHORT_ROW_SHAPES:
        dt = getattr(torch, dtn)
        gen = torch.Generator(device=dev).manual_seed(1)
        g = (0.5 + 0.5 * torch.rand(B, M, L, device=dev, generator=gen)).to(dt)
        x = torch.randn(B, D, L, device=dev, generator=gen).to(dt)
        G = torch.randn(B, M, D, L, device=dev, generator=gen).to(dt)
        z = torch.zeros(B, M, D, dtype=dt, device=dev)
        out = torch.empty(B, M, D, L, dtype=dt, device=dev)
        dx, dg = torch.empty_like(out), torch.empty_like(out)
        nbytes = B * M * D * L * g.element_size()
        r = {"shape": [B, M, D, L], "storage_dtype": STORAGE[dtn]}
        for name, kw in (("packed", {}), ("row_per_wave", {"waves_per_row": 1})):
            f = timed(lambda: S.fm_scan_forward(g, x, z, out, **kw), 20)
            b = timed(lambda: S.fm_scan_backward(g, G, z, dx, out, x, dg, **kw), 20)
            fold = M == 1 and D == 1
            r[name] = {"fwd_ms": round(f, 4), "bwd_ms": round(b, 4),
                       "fwd_GBps": round((3 if fold else 1) * nbytes / f / 1e6, 1),
                       "bwd_GBps": round((6 if fold else 4) * nbytes / b / 1e6, 1)}
        if M > 1 and D > 1:  # FM_Scan.backward's routes: the sums inside the kernel, or two tensors and two sums
            code = {"float32": 0, "float16": 1, "bfloat16": 2}[dtn]
            r["sums_inside"] = ("packed" if S.module.fmscan_reduced_packed_groups(B, M, D, L, code) > 0 else "a row per wave")
            r["sums_inside_ms"] = round(timed(lambda: S.fm_scan_backward_reduced(g, G, z, out, x), 10), 4)

            def two():
                S.fm_scan_backward(g, G, z, dx, out, x, dg)
                return dg.sum(dim=2), dx.sum(dim=1)

            r["two_tensors_and_sums_ms"] = round(timed(two, 10), 4)
        rows.append(r)
        del g, x, G, out, dx, dg
        torch.cuda.empty_cache()
    print(f"{'(B, M, D, L)':>26s} {'dtype':>5s} | {'fwd ms':>8s} {'GB/s':>7s} {'bwd ms':>8s} {'GB/s':>7s} | a row per wave: "
          f"{'fwd ms':>8s} {'GB/s':>7s} {'bwd ms':>8s} {'GB/s':>7s}", file=sys.stderr)
    for r in rows:
        p, o = r["packed"], r["row_per_wave"]
        print(f"{str(tuple(r['shape'])):>26s} {r['storage_dtype']:>5s} | {p['fwd_ms']:8.4f} {p['fwd_GBps']:7.0f} "
              f"{p['bwd_ms']:8.4f} {p['bwd_GBps']:7.0f} |                 {o['fwd_ms']:8.4f} {o['fwd_GBps']:7.0f} "
              f"{o['bwd_ms']:8.4f} {o['bwd_GBps']:7.0f}", file=sys.stderr)
    print("\nbackward with the sums over slots and channels (FM_Scan.backward): inside the kernel | "
          "fmscan_backward, then two torch sums", file=sys.stderr)
    for r in rows:
        if "sums_inside_ms" in r:
            print(f"{str(tuple(r['shape'])):>26s} {r['storage_dtype']:>5s} | {r['sums_inside_ms']:8.4f} ms "
                  f"({r['sums_inside']}) | {r['two_tensors_and_sums_ms']:8.4f} ms", file=sys.stderr)
    print(json.dumps({"metric": "fmscan_forward / fmscan_backward on rows of at most 1 KiB, GB/s",
                      "unit": "GB/s", "dtype": "f32", "data": "synthetic", "shapes": rows}), flush=True)
    return 0


GRID_MAX_ELEMENTS = 1 << 31  # per tensor; larger cells of the grid are left out
GRID_DEPTHS = (2, 4)


def run_grid(torch, args) -> int:
    """The library's choice of kernel variant against every variant a caller can ask for, off the
    benchmark shapes: rows x L x {bfloat16, float32} in the fold mapping (M = D = 1), and a few
    Factorization-Memory shapes with shared gate and token rows. Forward and backward kernels apart,
    HIP events around `reps` launches after 3 untimed ones. One text line per cell and direction:
    time and fraction of peak of the library's choice (on the metric's bytes, forward 3 and backward 6
    element sizes per element, and on the bytes moved, 3 and 5), the best override (waves per row /
    resident blocks per compute unit / prefetch depth), and how far the choice is behind it."""
    from fm.scan.fm_scan import fm_scan_backward, fm_scan_forward

    dev = torch.device("cuda", 0)
    overrides = [(w, b, d) for w in (1, 2, 4, 8) for b in (1, 2, 4, 8) for d in GRID_DEPTHS]
    raw = open(args.grid_raw, "w") if args.grid_raw else None

    def timed(call):
        """ms per launch: the better of two rounds of launches that fill about 3 ms each (5 to 100)."""
        for _ in range(3):
            call()
        best, reps = None, 5
        for _ in range(3):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            for _ in range(reps):
                call()
            b.record()
            b.synchronize()
            ms = a.elapsed_time(b) / reps
            best = ms if best is None else min(best, ms)
            reps = max(5, min(100, int(3.0 / ms)))
        return best

    print("# python bench.py --grid   (fold mapping: (rows, 1, L) gates and tokens; native: (B, M, D, L))")
    print("# frac = of 8 TB/s on the metric's bytes / on the bytes moved; behind = library's time / best override's - 1")
    print(f"# {'shape':<26} {'dtype':<9} {'dir':<4} {'lib ms':>9} {'frac':>6} {'moved':>6}   {'best override (w/b/d)':<22} {'ms':>9} {'behind':>7}")
    worst = []
    cells = [((r, 1, 1, L), dtn) for dtn in ("bfloat16", "float32") for r in GRID_ROWS for L in GRID_L]
    cells += [(shape, "bfloat16") for shape in GRID_NATIVE]
    for (B, M, D, L), dtn in cells:
        dt = getattr(torch, dtn)
        N = B * M * D * L
        if N > GRID_MAX_ELEMENTS:
            print(f"# {str((B, M, D, L)):<26} {dtn:<9} left out: more than 2^31 elements per tensor")
            continue
        gen = torch.Generator(device=dev).manual_seed(N % 9973)
        g = (0.5 + 0.5 * torch.rand(B, M, L, device=dev, generator=gen)).to(dt)
        x = torch.randn(B, D, L, device=dev, generator=gen).to(dt)
        G = torch.randn(B, M, D, L, device=dev, generator=gen).to(dt)
        zeros = torch.zeros(B, M, D, dtype=dt, device=dev)
        out = torch.empty(B, M, D, L, dtype=dt, device=dev)
        dx, dg = torch.empty_like(out), torch.empty_like(out)
        s = g.element_size()
        small = (B * M + B * D) * L  # gates and tokens
        for direction in ("fwd", "bwd"):
            if direction == "fwd":
                run = lambda **kw: fm_scan_forward(g, x, zeros, out, **kw)
                metric_bytes = moved_bytes = s * (N + small)
                if M == 1 and D == 1:
                    metric_bytes = moved_bytes = 3 * s * N
            else:
                run = lambda **kw: fm_scan_backward(g, G, zeros, dx, out, x, dg, **kw)
                metric_bytes, moved_bytes = s * (4 * N + small), s * (3 * N + small)
                if M == 1 and D == 1:
                    metric_bytes, moved_bytes = 6 * s * N, 5 * s * N
            lib_ms = timed(lambda: run())
            best, best_ms = None, None
            for (w, b, d) in overrides:
                ms = timed(lambda: run(waves_per_row=w, blocks_per_cu=b, depth=d))
                if raw:
                    raw.write(json.dumps({"shape": [B, M, D, L], "dtype": dtn, "dir": direction, "w": w, "b": b, "d": d,
                                          "ms": round(ms, 5)}) + "\n")
                if best_ms is None or ms < best_ms:
                    best, best_ms = (w, b, d), ms
            lib_ms = min(lib_ms, timed(lambda: run()))  # once more, after the sweep: the better of two
            if raw:
                raw.write(json.dumps({"shape": [B, M, D, L], "dtype": dtn, "dir": direction, "w": 0, "b": 0, "d": 0,
                                      "ms": round(lib_ms, 5)}) + "\n")
                raw.flush()
            behind = lib_ms / best_ms - 1.0
            print(f"  {str((B, M, D, L)):<26} {dtn:<9} {direction:<4} {lib_ms:9.4f} {metric_bytes / lib_ms / 1e6 / PEAK_HBM_GBPS:6.3f} "
                  f"{moved_bytes / lib_ms / 1e6 / PEAK_HBM_GBPS:6.3f}   {'%d/%d/%d' % best:<22} {best_ms:9.4f} {100 * behind:6.1f}%", flush=True)
            if behind > 0.07:
                worst.append(((B, M, D, L), dtn, direction, round(100 * behind, 1)))
        del g, x, G, zeros, out, dx, dg
        torch.cuda.empty_cache()
    print(f"# cells where the library's choice is more than 7 % behind the best override: {worst if worst else 'none'}")
    return 0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", default="cfg3", choices=sorted(WORKLOADS) + ["layer"])
    ap.add_argument("--waves-per-row", type=int, default=0, help="0 = library's choice")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-per-config", action="store_true",
                    help="headline workload only: leave out the `per_config` object (the other benchmark "
                         "configurations and the layer, timed after the headline)")
    ap.add_argument("--grid", action="store_true",
                    help="no benchmark line: a text table of the library's choice of kernel variant against "
                         "every override, over a grid of shapes off the benchmark configurations")
    ap.add_argument("--grid-raw", default="", help="with --grid: also write every timing, one JSON object a line, to this file")
    ap.add_argument("--layer-shape", default="", metavar="B,L,M,D",
                    help="with --layer-shapes: this one shape instead of the list")
    ap.add_argument("--layer-shapes", action="store_true",
                    help="the layer's step over shapes with fewer batch elements and longer rows than the "
                         "benchmark's, with the routes the library takes for each; a table on stderr")
    ap.add_argument("--short-rows", action="store_true",
                    help="the two scan calls on rows of at most 1 KiB (several rows to a wave) against the "
                         "general kernels asked for by flag; a table on stderr")
    ap.add_argument("--graph", action="store_true",
                    help="also capture one step in a HIP graph and time its replays (what a launch-bound "
                         "caller, e.g. the small configuration 1, gets without the per-call Python cost)")
    ap.add_argument("--probe", action="store_true",
                    help="for rocprofv3 --pmc runs: a few launches of an elementwise copy of known "
                         "size (torch.neg, reads and writes one tensor), then of the two scan "
                         "kernels; no timing, no JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU; rows are independent, so more GPUs would "
              "each run the same kernels on a slice of the rows. Use --gpus 1.", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the scan has no CPU path to benchmark", file=sys.stderr)
        return 1
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    if args.grid:
        return run_grid(torch, args)
    if args.layer_shapes:
        return run_layer_shapes(torch, args)
    if args.short_rows:
        return run_short_rows(torch, args)
    if args.workload == "layer":
        return run_layer(torch, args)
    B, Cn, T, dtn = WORKLOADS[args.workload]
    rows = B * Cn
    W = args.waves_per_row
    if args.probe:
        g, x, G = make_inputs(torch, args.workload, dev)
        zeros, out, dx, dg, step = scan_buffers(torch, g, x, G, W)
        for _ in range(4):
            torch.neg(out, out=dx)
        for _ in range(4):
            step()
        torch.cuda.synchronize()
        print(f"probe: torch.neg reads and writes {out.numel() * out.element_size()} bytes each; "
              f"forward algorithmic bytes {3 * g.element_size() * rows * T}, "
              f"backward {6 * g.element_size() * rows * T}")
        return 0

    g, x, G = make_inputs(torch, args.workload, dev)
    zeros, out, dx, dg, step = scan_buffers(torch, g, x, G, W)
    elapsed, fwd_ms, bwd_ms = time_steps(torch, step, args.steps, args.warmup)
    s = g.element_size()
    N = rows * T
    ms_per_step = elapsed * 1e3 / args.steps
    value = 9 * s * N / (ms_per_step * 1e-3) / 1e9
    bwd_bytes = 6 * s * N   # the byte model of the metric: g, dL/dh, h, x read; two gradients written
    bwd_moved = 5 * s * N   # what the kernel moves: it makes h again from g and x instead of reading it
    achieved = bwd_bytes / (bwd_ms * 1e-3) / 1e9
    stem = f"scan_kernels_{args.workload.replace('f16', '')}_{STORAGE[dtn]}"
    traffic, traffic_from = profiled_traffic(stem, "scan_backward_kernel", s * N)
    result = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",  # the arithmetic type; tensors are stored as storage_dtype
        "storage_dtype": STORAGE[dtn],
        "data": "synthetic",
        "config": {"workload": f"{args.workload}: (B,C,T)=({B},{Cn},{T}) {dtn}, fwd+bwd, passed as "
                               f"{rows} rows with M=D=1, FM form h=g*h+(1-g)*x",
                   "bytes_per_element": 9 * s, "elements": N,
                   "bytes_moved_per_element": 8 * s,
                   "note": "value prices the step at the metric's 9 element sizes per element (forward 3, backward "
                           "6); the backward kernel makes the states again from gates and tokens instead of "
                           "reading them, so 8 are moved"},
        "pct_of_peak": round(100 * value / PEAK_HBM_GBPS, 2),
        "elements_per_s": round(N / (ms_per_step * 1e-3), 1),
        "fwd_ms": round(fwd_ms, 4),
        "bwd_ms": round(bwd_ms, 4),
        "fwd_GBps": round(3 * s * N / (fwd_ms * 1e-3) / 1e9, 1),
        "moved_GBps": round(8 * s * N / (ms_per_step * 1e-3) / 1e9, 1),
        "roofline": {"kernel": "scan_backward_kernel", "bound": "hbm", "achieved": round(achieved, 1),
                     "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": round(achieved / PEAK_HBM_GBPS, 4),
                     "algorithmic_bytes": bwd_bytes, "moved_bytes": bwd_moved,
                     "frac_of_moved_bytes": round(bwd_moved / (bwd_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 4),
                     "traffic": traffic, "traffic_from": traffic_from,
                     "timed_by": "events around each kernel in a second pass of the same steps, right after the "
                                 "timed one (inside the timed steps the events cost 6 us each)"},
    }
    result["streaming_copy"] = streaming_copy(torch, rows, T * s, fwd_ms, bwd_ms)
    if args.graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            step()
        for _ in range(args.warmup):
            graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            graph.replay()
        torch.cuda.synchronize()
        graph_ms = (time.perf_counter() - t0) * 1e3 / args.steps
        result["graph_replay"] = {"ms_per_step": round(graph_ms, 4),
                                  "GBps": round(9 * s * N / (graph_ms * 1e-3) / 1e9, 1)}
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(torch, g, x, G)
        if args.workload == "cfg1":
            result["reference_cpu_path"] = reference_cpu_path(torch, g, x, G)
    if args.workload == "cfg3" and not args.no_per_config:
        # the other configurations and the layer, after the headline's timed region and with its tensors freed
        del g, x, G, zeros, out, dx, dg, step
        torch.cuda.empty_cache()
        result["per_config"] = per_config(torch, dev, args.workload, steps=20, warmup=5)
    print(json.dumps(result), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
