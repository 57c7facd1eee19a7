#!/usr/bin/env python3
"""Benchmark of the fp32 matrix-product path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one batch of synthetic input: one fp32 GEMM
C = A.B with M = N = K = 8192 (the size the headline metric is quoted on), operands resident in
HBM before the timed region.  Prints ONE JSON line with the whole-job throughput in TFLOP/s,
the roofline of the dominant kernel (fp32 MFMA peak 157.3 TFLOP/s) measured with HIP events on the
stream the kernel runs on, and a CPU baseline (the C++ restatement of the reference's CPU matmul,
timed on this host's cores on a bounded sample of the same workload).

`extra.rows` carries one entry per product of every benchmark configuration — the square sweep with
a row-major and a transposed-view A, the attention-shaped batched products and their gradients, the
broadcast-batched case with its backward, the GPT-2-shaped linear layers (forward, dX, dW), mv, vm,
the skinny product and the CBOW logits with their gradient: microseconds per launch (HIP events,
median of three groups of back-to-back launches after a warm-up), TFLOP/s and GB/s on the
algorithmic flop and bytes, the roof that bounds it (the larger of flop / 157.3 TFLOP/s and
bytes / 8 TB/s), the fraction of that roof, and the relative Frobenius error of the whole result
against fp64.  Products whose operands and result would fit the chip's 256 MB memory-side cache are
timed over several copies of their buffers in rotation, so that every launch reads from HBM.
`extra` also holds the MLP training step in ms on GPU and CPU and the shader clock under load.

A full run (neither `--no-cpu` nor `--no-extra`) only coordinates in the process started from the command line: the headline,
the rows and the CPU baseline with the MLP step are measured by three child processes, one after the other, and their
results are merged into the one line.  A failure in a row then costs that row and the ones behind it, not the headline;
after a child that died of a signal nothing more is started on the GPU.  A run with `--no-cpu` or `--no-extra` (one thing
measured, typically under a profiler, which follows one program: `rocprofv3 ... -- python3 bench.py --rows cbow --no-cpu`)
and any run with `--single-process` measure in the process itself.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3  # 256 CU x 2.4 GHz x 256 flop/clk/CU
PEAK_HBM_GBPS = 8000.0
MALL_BYTES = 256e6             # memory-side cache: a working set below this would be served from it
MLP_LOSS_TOLERANCE = 1e-4      # |loss on the GPU - loss on the CPU| per training step of the MNIST-shaped MLP

# HBM bytes per 8192^3 launch of the headline kernel = FETCH_SIZE x its copy-calibration factor +
# WRITE_SIZE x its factor, read from the two counter summaries under profiles/ (None when absent)
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemm_mfma_256x128_square8192.md")


def measured_traffic_bytes():
    """`traffic_bytes_per_launch: <number>` line of the committed counter summary for the headline kernel."""
    try:
        with open(TRAFFIC_PROFILE) as f:
            for line in f:
                if line.lower().startswith("traffic_bytes_per_launch:"):
                    return float(line.split(":", 1)[1].split()[0])
    except OSError:
        pass
    return None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=8192, help="M=N=K of the square GEMM (default: the headline size)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the per-configuration rows and the MLP-step measurement")
    ap.add_argument("--clock-probe-rounds", type=int, default=50000, help="length of the shader-clock probe (rounds of four MFMAs per wavefront)")
    ap.add_argument("--mlp-fused-tail", action="store_true",
                    help="also time the MLP step with its last two layers, loss, backward and update fused into one launch, with the first layer's "
                    "gradient and update fused as well, and with the first layer's forward as one launch too (mlp_fused_tail knob 1, 2 and 3)")
    ap.add_argument("--tune", default="", help="comma-separated name=value overrides of the kernel selection (tenmo_hip_set_tuning) for the rows, "
                    "e.g. gemm_panel=1,gemm_smallk=0: the same committed rows under another kernel choice")
    ap.add_argument("--sweep", default="", help="semicolon-separated lists in the form of --tune: the chosen rows (--rows) are timed once more "
                    "under each list, in this process, and reported under extra.sweep")
    ap.add_argument("--rows", default="", help="comma-separated substrings: only the rows whose name contains one of them")
    ap.add_argument("--adjacent", action="store_true",
                    help="also time the adjacent operators (cross-entropy, SGD step, convolution) into `extra`; off by default")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy, the known-size kernel against which FETCH_SIZE/WRITE_SIZE are scaled")
    ap.add_argument("--single-process", action="store_true",
                    help="measure everything in this process.  A full run (no --no-cpu, no --no-extra) otherwise only coordinates: the "
                    "headline, the rows and the CPU / MLP leg each run in a child process of their own, so that a failure in an "
                    "additional measurement cannot take the headline with it")
    ap.add_argument("--phase", default="", help=argparse.SUPPRESS)            # headline | rows | cpu: what a child process measures
    ap.add_argument("--worker-launcher", default="", help=argparse.SUPPRESS)  # how to start a child (tests: a wrapper around this file)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the reference has no multi-GPU path and every "
              "configuration fits one MI355X); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        return 2
    # (a run that leaves out the CPU leg or the rows is a measurement of one thing, typically under a profiler: one process)
    if not args.single_process and not args.phase and not args.no_cpu and not args.no_extra:
        return coordinate(args)
    phases = {args.phase} if args.phase else {"headline", "rows", "cpu"}
    out, rc = measure(args, phases)
    print(json.dumps(out), flush=True)
    return rc


def coordinate(args) -> int:
    """Runs the phases in child processes and prints the one line.  This process never touches the GPU."""
    import shlex
    import subprocess

    launcher = shlex.split(args.worker_launcher) if args.worker_launcher else [sys.executable, os.path.abspath(__file__)]
    passed = [a for a in sys.argv[1:]]

    def child(phase):
        """(dict printed by the child or None, how it ended)"""
        proc = subprocess.Popen(launcher + passed + ["--phase", phase], stdout=subprocess.PIPE, text=True, cwd=ROOT)  # stderr passes through
        last = None
        partial_rows = []
        for line in proc.stdout:
            line = line.strip()
            if not line.startswith("{"):
                continue
            try:
                obj = json.loads(line)
            except ValueError:
                continue
            if "row_done" in obj:
                partial_rows.append(obj["row_done"])
            else:
                last = obj
        code = proc.wait()
        return last, partial_rows, code

    out, _, code = child("headline")
    if out is None:
        print("bench.py: the headline measurement ended with status %d and printed no result" % code, file=sys.stderr)
        return code or 1
    extra = out.pop("extra", {})
    gates = out.pop("gates", {})
    ok = code == 0
    gpu_alive = True
    if not args.no_extra:
        got, partial_rows, code = child("rows")
        if got is not None:
            extra.update(got.get("extra", {}))
            gates.update({k: v for k, v in got.get("gates", {}).items() if k != "max_rel_err_vs_fp64"})
            gates["max_rel_err_vs_fp64"] = max(gates.get("max_rel_err_vs_fp64", 0.0), got.get("gates", {}).get("max_rel_err_vs_fp64", 0.0))
        else:  # the child died: keep what it had finished, name where it stopped, start nothing more on the GPU
            extra["rows"] = partial_rows
            extra["rows_error"] = "the process measuring the rows ended with status %d after %d rows" % (code, len(partial_rows))
            gpu_alive = code >= 0 and code not in (124, 134, 137, 139)
        ok = ok and code == 0 and got is not None
    if not args.no_cpu:
        got, _, code = child("cpu" if gpu_alive else "cpu-only")
        if got is not None:
            if "cpu_baseline" in got:
                out["cpu_baseline"] = got["cpu_baseline"]
            extra.update(got.get("extra", {}))
            gates.update({k: v for k, v in got.get("gates", {}).items() if k == "mlp_loss_ok"})
        else:
            extra["cpu_baseline_error"] = "the process measuring the CPU baseline and the MLP step ended with status %d" % code
        ok = ok and code == 0 and got is not None
    if extra:
        out["extra"] = extra
    gates["rel_err_ok"] = gates.get("max_rel_err_vs_fp64", 1.0) <= 1e-5
    gates["measurements_ok"] = ok and not any(k.endswith("_error") for k in extra)
    out["gates"] = gates
    print(json.dumps(out), flush=True)
    return 0 if gates["rel_err_ok"] and gates.get("mlp_loss_ok", True) and gates["measurements_ok"] else 1


def measure(args, phases):
    """The phases in this process: (the result dict, exit status)."""
    import numpy as np
    import torch

    from tenmo_amd import _lib

    if phases == {"cpu-only"}:  # (after a GPU failure in another phase: the CPU baseline alone, nothing of this process touches the GPU)
        return measure_more(args, phases, {}, 0.0, None, _lib, torch, np)
    _lib.init(0)
    L = _lib.load()
    cus = C.c_int()
    name = C.create_string_buffer(128)
    L.tenmo_hip_device_info(C.byref(cus), name, 128)
    if "headline" not in phases:
        return measure_more(args, phases, {}, 0.0, L, _lib, torch, np)

    if args.pmc_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    S = args.size
    gen = torch.Generator(device="cuda")
    gen.manual_seed(8192)
    A = torch.randn((S, S), generator=gen, device="cuda", dtype=torch.float32)
    B = torch.randn((S, S), generator=gen, device="cuda", dtype=torch.float32)
    Cc = torch.empty((S, S), device="cuda", dtype=torch.float32)

    def step():
        _lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, S, 1, B.data_ptr(), 0, S, 1, Cc.data_ptr(), S, S, S,
                                        0, None, None, None, 0, 0))

    # the first launches after start-up run while the clocks still ramp (9.0, 8.1, 7.6, 7.4 ms ... 7.2 ms in a
    # kernel trace): bring the device to its steady state before the W warm-up steps the caller asked for
    for _ in range(10):
        step()
    for _ in range(args.warmup):
        step()
    _lib.check(L.tenmo_hip_sync())
    torch.cuda.synchronize()
    # wall clock around exactly K steps, synchronised on both sides; HIP events on the library's
    # stream bracket the same launches for the per-launch kernel duration
    t0 = time.perf_counter()
    _lib.check(L.tenmo_hip_timer_begin())
    for _ in range(args.steps):
        step()
    ev_ms = C.c_float()
    _lib.check(L.tenmo_hip_timer_end(C.byref(ev_ms)))
    _lib.check(L.tenmo_hip_sync())
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kernel_ms = ev_ms.value / args.steps
    flop = 2.0 * S * S * S
    value = flop / (wall_ms * 1e-3) / 1e12
    achieved = flop / (kernel_ms * 1e-3) / 1e12
    # shader clock under a full matrix-core load, right behind the timed launches
    mhz = C.c_float()
    _lib.check(L.tenmo_hip_clock_probe(args.clock_probe_rounds, C.byref(mhz)))

    # accuracy gate on the timed result: the whole matrix against fp64
    rel_err = rel_fro_vs_fp64(torch, Cc, A, B)

    out = {
        "metric": "fp32 GEMM TFLOP/s (M=N=K=%d) + %% fp32-MFMA peak (1 GPU); MLP train-step ms vs CPU" % S,
        "value": round(value, 3),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "square fp32 GEMM C=A.B, M=N=K=%d, A and B row-major N(0,1), inputs resident in HBM" % S,
                   "device": name.value.decode(), "compute_units": cus.value},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 3), "peak": PEAK_FP32_MFMA_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": measured_traffic_bytes() if S == 8192 else None,
                     "kernel_ms": round(kernel_ms, 4), "effective_mhz": round(mhz.value, 1)},
        "rel_fro_error_vs_fp64": rel_err,
    }
    del A, B, Cc
    torch.cuda.empty_cache()
    # the headline so far, on stderr: a run that is cut short in the additional measurements still shows it (stdout carries
    # the one complete line at the end)
    print("bench headline (the complete line follows on stdout): " + json.dumps(out), file=sys.stderr, flush=True)
    return measure_more(args, phases, out, rel_err, L, _lib, torch, np)


def measure_more(args, phases, out, rel_err, L, _lib, torch, np):
    """The additional measurements (phases "rows" and "cpu") on top of the headline dict `out`."""
    S = args.size
    gen = torch.Generator(device="cuda") if phases != {"cpu-only"} else None
    mhz = C.c_float()
    # The headline line is printed whatever becomes of the additional measurements: an exception in one of them is
    # recorded under its name and the others still run.
    extra = {}
    worst = rel_err
    failed = False

    def attempt(name, fn):
        nonlocal failed
        try:
            return fn()
        except Exception as e:  # noqa: BLE001
            failed = True
            extra[name + "_error"] = "%s: %s" % (type(e).__name__, e)
            return None

    if not args.no_extra and "rows" in phases:
        only = [s for s in args.rows.split(",") if s]

        def rows_under(tune_list):
            """The rows timed with the kernel selection overridden by `tune_list` ("name=value,...", may be empty)."""
            tuned = [kv.split("=", 1) for kv in tune_list.split(",") if "=" in kv]
            for name_, value_ in tuned:
                _lib.check(L.tenmo_hip_set_tuning(name_.strip().encode(), int(value_)))
            try:
                return {n.strip(): int(v) for n, v in tuned}, config_rows(L, _lib, torch, only, announce=phases == {"rows"})
            finally:
                for name_, _ in tuned:
                    L.tenmo_hip_set_tuning(name_.strip().encode(), -1 if name_.strip() != "mlp_fused_tail" else 0)

        got = attempt("rows", lambda: rows_under(args.tune))
        if got is not None:
            if got[0]:
                extra["tune"] = got[0]
            rows = got[1]
            extra["rows"] = rows
            worst = max([worst] + [r["rel_err_vs_fp64"] for r in rows])
            extra["rows_max_rel_err_vs_fp64"] = worst
        for i, tune_list in enumerate(t for t in args.sweep.split(";") if t.strip()):
            got = attempt("sweep%d" % i, lambda: rows_under(tune_list))
            if got is not None:
                extra.setdefault("sweep", []).append({"tune": got[0], "rows": [
                    {k: r[k] for k in ("name", "us", "frac", "rel_err_vs_fp64")} for r in got[1]]})
                worst = max([worst] + [r["rel_err_vs_fp64"] for r in got[1]])

        def clock_after_rows():
            _lib.check(L.tenmo_hip_clock_probe(args.clock_probe_rounds, C.byref(mhz)))
            return round(mhz.value, 1)

        after = attempt("effective_mhz_after_rows", clock_after_rows)
        if after is not None:
            extra["effective_mhz_after_rows"] = after
    if args.adjacent and "rows" in phases:
        extra.update(attempt("adjacent", lambda: adjacent_operators(L, _lib, torch)) or {})
    if not args.no_cpu and ("cpu" in phases or "cpu-only" in phases):
        def cpu_leg():
            # the same operands as the headline's (the same seeded generator; on the host when the GPU is not to be used any more)
            if gen is None:
                host = torch.Generator()
                host.manual_seed(8192)
                return cpu_gemm_baseline(torch.randn((S, S), generator=host), torch.randn((S, S), generator=host), S, np)
            gen.manual_seed(8192)
            A = torch.randn((S, S), generator=gen, device="cuda", dtype=torch.float32)
            B = torch.randn((S, S), generator=gen, device="cuda", dtype=torch.float32)
            return cpu_gemm_baseline(A, B, S, np)

        baseline = attempt("cpu_baseline", cpu_leg)
        if baseline is not None:
            out["cpu_baseline"] = baseline
        if not args.no_extra and "cpu" in phases:
            extra.update(attempt("mlp_step", lambda: mlp_step_times(_lib, torch, np, args.mlp_fused_tail)) or {})
    if extra:
        out["extra"] = extra
    # the gates: every product within 1e-5 of fp64 (relative Frobenius error), the MLP's loss curve within 1e-4 of the CPU
    # run at every one of its steps, and no additional measurement failed
    mlp_ok = extra.get("mlp_max_abs_loss_diff", 0.0) <= MLP_LOSS_TOLERANCE
    out["gates"] = {"max_rel_err_vs_fp64": worst, "rel_err_ok": worst <= 1e-5, "mlp_loss_ok": mlp_ok, "measurements_ok": not failed}
    return out, (0 if worst <= 1e-5 and mlp_ok and not failed else 1)


def rel_fro_vs_fp64(torch, got, A, B):
    """||got - A.B||_F / ||A.B||_F with the product accumulated in fp64 from the same fp32 operands (views welcome);
    large results go through in slabs of rows so that the fp64 temporaries stay small."""
    M = got.shape[-2]
    slab = max(1, min(M, int(2 ** 27 // max(1, got.shape[-1] * max(1, got.numel() // (got.shape[-1] * M))))))
    num = den = 0.0
    for r0 in range(0, M, slab):
        ref = torch.matmul(A[..., r0:r0 + slab, :].double(), B.double())
        d = got[..., r0:r0 + slab, :].double() - ref
        num += float((d * d).sum())
        den += float((ref * ref).sum())
    return math.sqrt(num / den) if den > 0 else math.sqrt(num)


def hip_time_us(L, _lib, fns, est_us):
    """Microseconds per launch: the launches `fns` (one per buffer copy, used in rotation) back to back between two
    HIP events on the library's stream; median of three such groups after a warm-up."""
    def run(n):
        for i in range(n):
            fns[i % len(fns)]()
    run(max(3, len(fns)))
    _lib.check(L.tenmo_hip_sync())
    iters = int(min(200, max(10, 4000.0 / max(est_us, 1.0))))
    iters = (iters + len(fns) - 1) // len(fns) * len(fns)
    groups = []
    for _ in range(3):
        _lib.check(L.tenmo_hip_timer_begin())
        run(iters)
        ms = C.c_float()
        _lib.check(L.tenmo_hip_timer_end(C.byref(ms)))
        groups.append(ms.value * 1e3 / iters)
    return sorted(groups)[1]


def config_rows(L, _lib, torch, only, announce=False):
    """One row per product of the benchmark configurations (see the module docstring).  `announce`: print every finished row
    as a line of its own at once (a child process does: its parent then has the rows that were done if it dies later)."""
    rows = []
    gen = torch.Generator(device="cuda")

    def randn(shape, seed, std=1.0):
        gen.manual_seed(seed)
        t = torch.randn(shape, generator=gen, device="cuda", dtype=torch.float32)
        return t * std if std != 1.0 else t

    def view(t):
        return _lib.make_view(t.data_ptr(), 0, tuple(t.shape), tuple(t.stride()))

    def wanted(name):
        if only and not any(s in name for s in only):
            return False
        print("bench row: " + name, file=sys.stderr, flush=True)  # a run that dies names the row it died in
        return True

    def finish_row(name, cfg, shape, us, flop, nbytes, rel_err, copies):
        t_mfma, t_hbm = flop / (PEAK_FP32_MFMA_TFLOPS * 1e12) * 1e6, nbytes / (PEAK_HBM_GBPS * 1e9) * 1e6
        roof = max(t_mfma, t_hbm)
        rows.append({"name": name, "cfg": cfg, "shape": shape, "us": round(us, 2),
                     "tflops": round(flop / us / 1e6, 2), "gbps": round(nbytes / us / 1e3, 1),
                     "bound": "mfma" if t_mfma >= t_hbm else "hbm", "roof_us": round(roof, 2), "frac": round(roof / us, 4),
                     "rel_err_vs_fp64": rel_err, "buffer_copies": copies})
        if announce:
            print(json.dumps({"row_done": rows[-1]}), flush=True)

    def copies_for(nbytes):
        # enough copies of the buffers that a rotation through them exceeds the memory-side cache twice over
        return 1 if nbytes >= 2 * MALL_BYTES else int(min(12, math.ceil(2 * MALL_BYTES / nbytes)))

    def gemm_row(name, cfg, make_a, make_b, out_shape):
        """make_a / make_b: seed -> operand tensor (any torch view; broadcast batch dims have extent 1 or are absent)."""
        if not wanted(name):
            return
        a0, b0 = make_a(0), make_b(0)
        M, K, N = a0.shape[-2], a0.shape[-1], b0.shape[-1]
        batch = 1
        for d in out_shape[:-2]:
            batch *= d
        flop = 2.0 * M * N * K * batch
        nbytes = 4.0 * (a0.numel() + b0.numel() + batch * M * N)
        n = copies_for(nbytes)
        As, Bs = [a0] + [make_a(i) for i in range(1, n)], [b0] + [make_b(i) for i in range(1, n)]
        Cs = [torch.empty(out_shape, device="cuda", dtype=torch.float32) for _ in range(n)]
        views = [(view(a), view(b)) for a, b in zip(As, Bs)]
        fns = [(lambda av=av, bv=bv, c=c: _lib.check(L.tenmo_hip_matmul_nd(C.byref(av), C.byref(bv), c.data_ptr(), 0)))
               for (av, bv), c in zip(views, Cs)]
        us = hip_time_us(L, _lib, fns, max(flop / 100e6, nbytes / 4e6))
        err = rel_fro_vs_fp64(torch, Cs[0], As[0], Bs[0])
        finish_row(name, cfg, "[%s].[%s]" % ("x".join(map(str, a0.shape)), "x".join(map(str, b0.shape))), us, flop, nbytes, err, n)
        del As, Bs, Cs
        torch.cuda.empty_cache()

    # ---- config 2: square sweep, A row-major and A as a transposed view (storage [K, M], strides (1, M)) ----
    for S in (1024, 2048, 4096, 8192):
        gemm_row("square%d" % S, 2, lambda i, S=S: randn((S, S), 100 + i), lambda i, S=S: randn((S, S), 200 + i), (S, S))
        gemm_row("square%d_At" % S, 2, lambda i, S=S: randn((S, S), 100 + i).t(), lambda i, S=S: randn((S, S), 200 + i), (S, S))

    # ---- config 3: attention-shaped broadcast-batched products, Q K V dO = [8,12,1024,64], P dS = [8,12,1024,1024] ----
    bh, T, D = (8, 12), 1024, 64
    gemm_row("attn_qkt", 3, lambda i: randn(bh + (T, D), 300 + i), lambda i: randn(bh + (T, D), 310 + i).transpose(-1, -2), bh + (T, T))
    gemm_row("attn_pv", 3, lambda i: torch.softmax(randn(bh + (T, T), 320 + i), -1), lambda i: randn(bh + (T, D), 330 + i), bh + (T, D))
    gemm_row("attn_dP=dO.Vt", 3, lambda i: randn(bh + (T, D), 340 + i), lambda i: randn(bh + (T, D), 330 + i).transpose(-1, -2), bh + (T, T))
    gemm_row("attn_dV=Pt.dO", 3, lambda i: torch.softmax(randn(bh + (T, T), 320 + i), -1).transpose(-1, -2), lambda i: randn(bh + (T, D), 340 + i), bh + (T, D))
    gemm_row("attn_dQ=dS.K", 3, lambda i: randn(bh + (T, T), 350 + i), lambda i: randn(bh + (T, D), 310 + i), bh + (T, D))
    gemm_row("attn_Qt.dS", 3, lambda i: randn(bh + (T, D), 300 + i).transpose(-1, -2), lambda i: randn(bh + (T, T), 350 + i), bh + (D, T))
    # README case A[32,512,768] . B[1,768,768] and its backward
    gemm_row("bcast_fwd", 3, lambda i: randn((32, 512, 768), 360 + i), lambda i: randn((1, 768, 768), 370 + i), (32, 512, 768))
    gemm_row("bcast_dA=dC.Bt", 3, lambda i: randn((32, 512, 768), 380 + i), lambda i: randn((1, 768, 768), 370 + i).transpose(-1, -2), (32, 512, 768))
    if wanted("bcast_dB"):
        # dB = sum over the 32 batches of A_b^T . dC_b through the backward entry (+= into the gradbox of B)
        nb, M, K, N = 32, 512, 768, 768
        flop, nbytes = 2.0 * nb * M * K * N, 4.0 * (2 * nb * M * K + K * N)
        n = copies_for(nbytes)
        As = [randn((nb, M, K), 360 + i) for i in range(n)]
        dCs = [randn((nb, M, N), 380 + i) for i in range(n)]
        Bw = randn((1, K, N), 370)
        gBs = [torch.zeros((1, K, N), device="cuda") for _ in range(n)]
        bv = view(Bw)
        fns = [(lambda av=view(a), dc=dc, g=g: _lib.check(L.tenmo_hip_matmul_backward(C.byref(av), C.byref(bv), dc.data_ptr(), None, g.data_ptr(), 0)))
               for a, dc, g in zip(As, dCs, gBs)]
        us = hip_time_us(L, _lib, fns, flop / 100e6)
        gBs[0].zero_()
        fns[0]()
        err = rel_fro_vs_fp64(torch, gBs[0][0], As[0].reshape(-1, K).t(), dCs[0].reshape(-1, N))
        finish_row("bcast_dB=sum_b(At.dC)", 3, "sum_32 [768x512].[512x768]", us, flop, nbytes, err, n)
        del As, dCs, gBs
        torch.cuda.empty_cache()

    # ---- config 4: GPT-2-small linear layers, 8192 tokens: forward, dX = dY.W^T(view), dW = X^T(view).dY ----
    Tk = 8192
    for nm, din, dout in (("qkv", 768, 2304), ("proj", 768, 768), ("up", 768, 3072), ("down", 3072, 768), ("lmhead", 768, 50257)):
        gemm_row("gpt2_%s_fwd" % nm, 4, lambda i, din=din: randn((Tk, din), 400 + i), lambda i, din=din, dout=dout: randn((din, dout), 410 + i, 0.02), (Tk, dout))
        gemm_row("gpt2_%s_dX" % nm, 4, lambda i, dout=dout: randn((Tk, dout), 420 + i), lambda i, din=din, dout=dout: randn((din, dout), 410 + i, 0.02).t(), (Tk, din))
        gemm_row("gpt2_%s_dW" % nm, 4, lambda i, din=din: randn((Tk, din), 400 + i).t(), lambda i, dout=dout: randn((Tk, dout), 420 + i), (din, dout))

    # ---- config 5: memory-bound products ----
    n16 = 16384
    if wanted("mv") or wanted("vm"):
        W = randn((n16, n16), 500)
        x = randn((n16,), 501)
        o = torch.empty((n16,), device="cuda")
        nbytes = (n16 * n16 + 2 * n16) * 4.0
        mv = lambda: _lib.check(L.tenmo_hip_mv_f32(W.data_ptr(), 0, n16, 1, x.data_ptr(), 0, 1, o.data_ptr(), n16, n16, 0, None, None, None, 0, 0))
        vm = lambda: _lib.check(L.tenmo_hip_vm_f32(x.data_ptr(), 0, 1, W.data_ptr(), 0, n16, 1, o.data_ptr(), n16, n16, 0, None, None, None, 0, 0))
        for nm, fn, ref in (("mv16384", mv, lambda: W.double() @ x.double()), ("vm16384", vm, lambda: x.double() @ W.double())):
            if not wanted(nm[:2]):
                continue
            us = hip_time_us(L, _lib, [fn], 160.0)
            r = ref()
            err = float((o.double() - r).norm() / r.norm())
            finish_row(nm, 5, "[16384x16384] x [16384]", us, 2.0 * n16 * n16, nbytes, err, 1)
        del W, x, o
        torch.cuda.empty_cache()
    gemm_row("skinny_4x768x50257", 5, lambda i: randn((4, 768), 510 + i), lambda i: randn((768, 50257), 520 + i), (4, 50257))
    gemm_row("cbow_logits", 5, lambda i: randn((256, 100), 530 + i), lambda i: randn((100, 50000), 540 + i), (256, 50000))
    gemm_row("cbow_At.dC", 5, lambda i: randn((256, 100), 530 + i).t(), lambda i: randn((256, 50000), 550 + i), (100, 50000))

    # ---- last (the one row whose kernels are younger than the others): config 4, the whole backward of a Linear layer ----
    if wanted("gpt2_up_linear_backward"):
        # the whole backward of the MLP-up Linear layer in one call: dX += dY.W^T, dW += X^T.dY, db += column sums of dY
        # (the bias gradient comes out of the dW launch: dY is streamed twice, not three times)
        din, dout = 768, 3072
        flop = 2 * 2.0 * Tk * din * dout
        nbytes = 4.0 * (2 * Tk * din + 2 * din * dout + Tk * dout + dout)
        n = copies_for(nbytes)
        Xs = [randn((Tk, din), 400 + i) for i in range(n)]
        dYs = [randn((Tk, dout), 420 + i) for i in range(n)]
        Wt = randn((din, dout), 410, 0.02)
        gXs = [torch.zeros((Tk, din), device="cuda") for _ in range(n)]
        gWs = [torch.zeros((din, dout), device="cuda") for _ in range(n)]
        gbs = [torch.zeros((dout,), device="cuda") for _ in range(n)]
        wv = view(Wt)
        fns = [(lambda xv=view(x), dy=dy, gx=gx, gw=gw, gb=gb: _lib.check(L.tenmo_hip_linear_backward(C.byref(xv), C.byref(wv), dy.data_ptr(), gx.data_ptr(),
                                                                                                      gw.data_ptr(), gb.data_ptr(), 0)))
               for x, dy, gx, gw, gb in zip(Xs, dYs, gXs, gWs, gbs)]
        us = hip_time_us(L, _lib, fns, flop / 100e6)
        for t in (gXs[0], gWs[0], gbs[0]):
            t.zero_()
        fns[0]()
        errs = [rel_fro_vs_fp64(torch, gXs[0], dYs[0], Wt.t()), rel_fro_vs_fp64(torch, gWs[0], Xs[0].t(), dYs[0]),
                float((gbs[0].double() - dYs[0].double().sum(0)).norm() / dYs[0].double().sum(0).norm())]
        finish_row("gpt2_up_linear_backward(dX,dW,db)", 4, "[8192x3072].[3072x768] + [768x8192].[8192x3072] + colsum", us, flop, nbytes, max(errs), n)
        del Xs, dYs, gXs, gWs, gbs
        torch.cuda.empty_cache()
    return rows


def adjacent_operators(L, _lib, torch):
    """Cross-entropy over GPT-2-sized logits, an SGD step on 2^28 parameters and one convolution layer, forward and
    backward: microseconds per call and fractions of the HBM peak on algorithmic bytes (TFLOP/s for the convolution)."""
    def hip_time(fn, iters, warm=3):
        for _ in range(warm):
            fn()
        _lib.check(L.tenmo_hip_sync())
        _lib.check(L.tenmo_hip_timer_begin())
        for _ in range(iters):
            fn()
        ms = C.c_float()
        _lib.check(L.tenmo_hip_timer_end(C.byref(ms)))
        return ms.value / iters

    res = {}
    M, Cn = 8192, 50257
    x = torch.randn(M, Cn, device="cuda")
    t = torch.randint(0, Cn, (M,), device="cuda")
    sm = torch.empty_like(x)
    rows = torch.empty(M, device="cuda")
    tot = torch.zeros(1, device="cuda")
    val = torch.zeros(1, dtype=torch.int32, device="cuda")
    up = torch.ones(1, device="cuda")
    fwd = lambda soft: _lib.check(L.tenmo_hip_cross_entropy_forward_f32(x.data_ptr(), t.data_ptr(), 1, M, Cn, -100, 0.0, soft, rows.data_ptr(),
                                                                        tot.data_ptr(), val.data_ptr(), 0))
    by = M * Cn * 4.0
    ms = hip_time(lambda: fwd(None), 10)
    res["ce_8192x50257_loss_only_us"] = round(ms * 1e3, 1)
    res["ce_8192x50257_loss_only_frac_hbm_peak"] = round(by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)
    ms = hip_time(lambda: fwd(sm.data_ptr()), 10)
    res["ce_8192x50257_forward_us"] = round(ms * 1e3, 1)
    res["ce_8192x50257_forward_frac_hbm_peak"] = round(2 * by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)
    g = x  # the logits are no longer needed: their storage takes the gradient
    ms = hip_time(lambda: _lib.check(L.tenmo_hip_cross_entropy_backward_f32(sm.data_ptr(), t.data_ptr(), 1, up.data_ptr(), M, Cn, -100, 0.0, 2, M,
                                                                            g.data_ptr(), 0, 0)), 10)
    res["ce_8192x50257_backward_us"] = round(ms * 1e3, 1)
    res["ce_8192x50257_backward_frac_hbm_peak"] = round(2 * by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)
    del x, sm, g
    n = 1 << 28
    p = torch.randn(n, device="cuda")
    gr = torch.randn(n, device="cuda")
    ms = hip_time(lambda: _lib.check(L.tenmo_hip_sgd_step_f32(p.data_ptr(), gr.data_ptr(), None, n, 0.01, 0.0, 0.0, 0)), 10)
    res["sgd_2p28_us"] = round(ms * 1e3, 1)
    res["sgd_2p28_frac_hbm_peak"] = round(12.0 * n / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)
    del p, gr
    nb, ci, h, w, co, k = 128, 64, 34, 34, 128, 3
    img = torch.randn(nb, ci, h, w, device="cuda")
    ker = torch.randn(co, ci, k, k, device="cuda")
    bias = torch.randn(co, device="cuda")
    ho, wo = h - k + 1, w - k + 1
    out = torch.empty(nb, co, ho, wo, device="cuda")
    flop = 2.0 * nb * co * ho * wo * ci * k * k
    ms = hip_time(lambda: _lib.check(L.tenmo_hip_conv2d_forward_f32(img.data_ptr(), nb, ci, h, w, ker.data_ptr(), co, k, k, bias.data_ptr(), 1, 1,
                                                                    out.data_ptr(), 0)), 10)
    res["conv_128x64x34x34_k3_to_128_forward_us"] = round(ms * 1e3, 1)
    res["conv_128x64x34x34_k3_to_128_forward_tflops"] = round(flop / (ms * 1e-3) / 1e12, 1)
    gi, gk, gb = torch.empty_like(img), torch.empty_like(ker), torch.empty_like(bias)
    ms = hip_time(lambda: _lib.check(L.tenmo_hip_conv2d_backward_f32(img.data_ptr(), nb, ci, h, w, ker.data_ptr(), co, k, k, 1, 1, out.data_ptr(),
                                                                     gi.data_ptr(), gk.data_ptr(), gb.data_ptr(), 0, 0)), 10)
    res["conv_128x64x34x34_k3_to_128_backward_us"] = round(ms * 1e3, 1)
    res["conv_128x64x34x34_k3_to_128_backward_tflops"] = round(2 * flop / (ms * 1e-3) / 1e12, 1)
    return res


def cpu_gemm_baseline(A, B, S, np):
    """The restated reference CPU matmul (tenmo/matmul_cpu.mojo, path 1a) on this host's physical
    cores.  The sample is bounded to roughly 10-30 s: whole GEMMs while they fit, otherwise the
    first row tiles of one (a row tile is the reference's unit of parallel work)."""
    from oracle import oracle as O

    cores = O.num_physical_cores()
    tile_m = 128 if S > 256 else (64 if S > 64 else 32)
    all_tiles = (S + tile_m - 1) // tile_m
    a = A.cpu().numpy().reshape(1, S, S)
    b = B.cpu().numpy()
    out = np.empty((1, S, S), np.float32)
    # probe: one row tile per thread
    probe_tiles = min(cores, all_tiles)
    t0 = time.perf_counter()
    O.mmnd(a, b, cores, work_item_limit=probe_tiles, out=out)
    probe = time.perf_counter() - t0
    est_full = probe * all_tiles / probe_tiles
    if est_full <= 12.0:
        reps = max(1, min(3, int(25.0 / max(est_full, 1e-3))))
        best = min(_timed(lambda: O.mmnd(a, b, cores, out=out)) for _ in range(reps))
        tiles, what = all_tiles, "the whole GEMM, best of %d" % reps
    else:
        tiles = max(probe_tiles, min(all_tiles, int(all_tiles * 15.0 / est_full) // probe_tiles * probe_tiles))
        best = _timed(lambda: O.mmnd(a, b, cores, work_item_limit=tiles, out=out))
        what = "the first %d of %d row tiles of the same GEMM" % (tiles, all_tiles)
    rows = min(S, tiles * tile_m)
    flop = 2.0 * rows * S * S
    return {"value": round(flop / best / 1e12, 5), "unit": "TFLOP/s", "cores": cores, "kind": "port",
            "sample": "%s (%d rows x %d columns, K=%d), %.1f s, %d threads, fp32 SIMD width %d"
                      % (what, rows, S, S, best, cores, O.simd_width())}


def _timed(fn):
    t0 = time.perf_counter()
    fn()
    return time.perf_counter() - t0


def mlp_step_times(_lib, torch, np, fused_tail=False):
    """MNIST-shaped MLP 784->128->32->10, batch 64, SGD lr 0.01: ms per training step on the GPU (inputs
    already on the device) and on the CPU restatement, and the largest per-step loss difference.  With
    `fused_tail` the same 20 steps once more with the last two layers, the loss, their backward and their
    update as one launch."""
    from oracle import oracle as O
    from tenmo_amd import rng as R
    from tenmo_amd.net import MLP

    dims, seed, lr, batch = [784, 128, 32, 10], 2024, 0.01, 64
    Ws, bs = R.xavier_mlp(dims, seed)
    gpu, cpu = MLP(dims, Ws, bs, batch), O.MLP(dims, Ws, bs, batch)
    batches = [R.mnist_like_batch(batch, seed, s) for s in range(30)]
    dev = [(torch.from_numpy(x).cuda(), torch.from_numpy(y).cuda()) for x, y in batches]
    worst = 0.0
    gl = []
    for xd, yd in dev:  # 30 training steps on fresh batches, loss by loss against the CPU run: the parity gate (and the warm-up)
        gl.append(float(gpu.step_device(xd, yd, lr, sync=True).item()))
    t0 = time.perf_counter()
    cl = [cpu.step(x, y, lr) for x, y in batches]
    cpu_ms = (time.perf_counter() - t0) * 1e3 / len(batches)
    worst = max(abs(a - b) for a, b in zip(gl, cl))
    L = _lib.load()
    _lib.check(L.tenmo_hip_sync())
    t0 = time.perf_counter()
    for xd, yd in dev[10:]:
        gpu.step_device(xd, yd, lr, sync=False)
    _lib.check(L.tenmo_hip_sync())
    gpu_ms = (time.perf_counter() - t0) * 1e3 / 20
    # the same 20 steps replayed from the captured graph (parameters keep training; timing only)
    gpu.step_device(*dev[0], lr, sync=True, graph=True)
    t0 = time.perf_counter()
    for xd, yd in dev[10:]:
        gpu.step_device(xd, yd, lr, sync=False, graph=True)
    _lib.check(L.tenmo_hip_sync())
    graph_ms = (time.perf_counter() - t0) * 1e3 / 20
    fused = {}
    if fused_tail:
        # 1: the last two layers, loss, backward and update in one launch; 2: also the first layer's gradient with its update; 3: also its forward
        for level, key in ((1, "mlp_step_ms_gpu_fused_tail"), (2, "mlp_step_ms_gpu_fused_tail_and_first"), (3, "mlp_step_ms_gpu_three_launches")):
            L.tenmo_hip_set_tuning(b"mlp_fused_tail", level)
            try:
                first = float(gpu.step_device(*dev[0], lr, sync=True).item())
                t0 = time.perf_counter()
                for xd, yd in dev[10:]:
                    gpu.step_device(xd, yd, lr, sync=False)
                _lib.check(L.tenmo_hip_sync())
                fused[key] = round((time.perf_counter() - t0) * 1e3 / 20, 4)
                fused[key.replace("mlp_step_ms_gpu", "mlp") + "_first_loss"] = first
            finally:
                L.tenmo_hip_set_tuning(b"mlp_fused_tail", 0)
    return {**fused, "mlp_step_ms_gpu": round(gpu_ms, 4), "mlp_step_ms_gpu_graph": round(graph_ms, 4), "mlp_step_ms_cpu": round(cpu_ms, 4), "mlp_cpu_cores": O.num_physical_cores(),
            "mlp_max_abs_loss_diff": worst, "mlp_parity_steps": len(batches), "mlp_loss_tolerance": MLP_LOSS_TOLERANCE}


if __name__ == "__main__":
    sys.exit(main())
