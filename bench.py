#!/usr/bin/env python3
"""Benchmark of the fp32 matrix-product path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one pass of the hot path over one batch of synthetic input: one fp32 GEMM
C = A.B with M = N = K = 8192 (the size the headline metric is quoted on), operands resident in
HBM before the timed region.  Prints ONE JSON line with the whole-job throughput in TFLOP/s,
the roofline of the dominant kernel (fp32 MFMA peak 157.3 TFLOP/s) measured with HIP events on the
stream the kernel runs on, and a CPU baseline (the C++ restatement of the reference's CPU matmul,
timed on this host's cores on a bounded sample of the same workload).  The `extra` object carries
the other headline figures: mv / vm bandwidth at 16384^2 and the MLP training step in ms on GPU
and CPU.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3  # 256 CU x 2.4 GHz x 256 flop/clk/CU
PEAK_HBM_GBPS = 8000.0

# Bytes moved between L2 and the memory fabric per 8192^3 launch, from two rocprofv3 --pmc runs
# (FETCH_SIZE 2.965e6 KiB scaled by 2.0, WRITE_SIZE 2.621e5 KiB scaled by 1.0; the scale factors are
# what the same counters read for a plain 1 GiB copy).  Only valid for the default size.
MEASURED_TRAFFIC_BYTES = 6.3e9


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--size", type=int, default=8192, help="M=N=K of the square GEMM (default: the headline size)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extra", action="store_true", help="skip the mv/vm and MLP-step side measurements")
    ap.add_argument("--adjacent", action="store_true",
                    help="also time the adjacent operators (cross-entropy, SGD step, convolution) into `extra`; off by default")
    ap.add_argument("--attention", action="store_true",
                    help="also time the attention-shaped batched products (Q.K^T, P.V, P^T.dO, Q^T.dS at [8,12,1024,64]) into `extra`; off by default")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy, the known-size kernel against which FETCH_SIZE/WRITE_SIZE are scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU (the reference has no multi-GPU path and every "
              "configuration fits one MI355X); --gpus %d is not supported" % args.gpus, file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from tenmo_amd import _lib

    _lib.init(0)
    L = _lib.load()
    cus = C.c_int()
    name = C.create_string_buffer(128)
    L.tenmo_hip_device_info(C.byref(cus), name, 128)

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

    # accuracy gate on the timed result: sampled rows against fp64
    rows = torch.tensor([0, S // 3, S - 1], device="cuda")
    ref = (A[rows].double() @ B.double()).cpu().numpy()
    got = Cc[rows].cpu().numpy()
    rel_err = float(np.linalg.norm(got - ref) / np.linalg.norm(ref))

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
                     "frac": round(achieved / PEAK_FP32_MFMA_TFLOPS, 4), "traffic": MEASURED_TRAFFIC_BYTES if S == 8192 else None,
                     "kernel_ms": round(kernel_ms, 4)},
        "rel_fro_error_vs_fp64": rel_err,
    }

    extra = {}
    if not args.no_extra:
        extra.update(side_measurements(L, _lib, torch, np))
    if args.adjacent:
        extra.update(adjacent_operators(L, _lib, torch))
    if args.attention:
        extra.update(attention_products(L, _lib, torch))
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_gemm_baseline(A, B, S, np)
        if not args.no_extra:
            extra.update(mlp_step_times(_lib, torch, np))
    if extra:
        out["extra"] = extra
    print(json.dumps(out), flush=True)
    return 0 if rel_err <= 1e-5 else 1


def hip_time(L, _lib, fn, iters, warm=3):
    for _ in range(warm):
        fn()
    _lib.check(L.tenmo_hip_sync())
    _lib.check(L.tenmo_hip_timer_begin())
    for _ in range(iters):
        fn()
    ms = C.c_float()
    _lib.check(L.tenmo_hip_timer_end(C.byref(ms)))
    return ms.value / iters


def side_measurements(L, _lib, torch, np):
    """mv / vm at 16384^2 (HBM-bound): GB/s of algorithmic bytes and fraction of the 8 TB/s peak."""
    n = 16384
    gen = torch.Generator(device="cuda")
    gen.manual_seed(16384)
    W = torch.randn((n, n), generator=gen, device="cuda", dtype=torch.float32)
    x = torch.randn((n,), generator=gen, device="cuda", dtype=torch.float32)
    out = torch.empty((n,), device="cuda", dtype=torch.float32)
    mv = lambda: _lib.check(L.tenmo_hip_mv_f32(W.data_ptr(), 0, n, 1, x.data_ptr(), 0, 1, out.data_ptr(), n, n, 0, None, None, None, 0, 0))
    vm = lambda: _lib.check(L.tenmo_hip_vm_f32(x.data_ptr(), 0, 1, W.data_ptr(), 0, n, 1, out.data_ptr(), n, n, 0, None, None, None, 0, 0))
    nbytes = (n * n + 2 * n) * 4.0
    res = {}
    for nm, fn in (("mv", mv), ("vm", vm)):
        ms = hip_time(L, _lib, fn, 30)
        gbps = nbytes / (ms * 1e-3) / 1e9
        res["%s_16384_us" % nm] = round(ms * 1e3, 2)
        res["%s_16384_gbps" % nm] = round(gbps, 1)
        res["%s_16384_frac_hbm_peak" % nm] = round(gbps / PEAK_HBM_GBPS, 4)
    return res


def attention_products(L, _lib, torch):
    """The broadcast-batched products of attention at Q, K, V = [8, 12, 1024, 64]: S = Q.K^T (K as a transposed view),
    O = P.V, dV = P^T.dO and Q^T.dS, each 12.88 GFLOP and 453 MB of algorithmic traffic; time, TFLOP/s and the
    relative Frobenius error of one batch against fp64."""
    Bn, H, T, D = 8, 12, 1024, 64
    gen = torch.Generator(device="cuda")
    gen.manual_seed(64)
    Q, K, V = (torch.randn((Bn, H, T, D), generator=gen, device="cuda", dtype=torch.float32) for _ in range(3))
    S = torch.empty((Bn, H, T, T), device="cuda", dtype=torch.float32)
    O = torch.empty((Bn, H, T, D), device="cuda", dtype=torch.float32)
    O2 = torch.empty((Bn, H, D, T), device="cuda", dtype=torch.float32)
    bs, st, pst = (Bn, H), (H * T * D, T * D), (H * T * T, T * T)

    def gemm(A, B, Cc, M, N, Kk, a_rs, a_cs, b_rs, b_cs, ab, bb):
        _lib.check(L.tenmo_hip_gemm_f32(A.data_ptr(), 0, a_rs, a_cs, B.data_ptr(), 0, b_rs, b_cs, Cc.data_ptr(), M, N, Kk,
                                        2, _lib.i64(bs), _lib.i64(ab), _lib.i64(bb), 0, 0))

    cases = (
        ("qkt", lambda: gemm(Q, K, S, T, T, D, D, 1, 1, D, st, st), lambda: (S[1, 2], Q[1, 2].double() @ K[1, 2].double().T)),
        ("pv", lambda: gemm(S, V, O, T, D, T, T, 1, D, 1, pst, st), lambda: (O[1, 2], S[1, 2].double() @ V[1, 2].double())),
        ("ptdo", lambda: gemm(S, V, O, T, D, T, 1, T, D, 1, pst, st), lambda: (O[1, 2], S[1, 2].double().T @ V[1, 2].double())),
        ("qtds", lambda: gemm(Q, S, O2, D, T, T, 1, D, T, 1, st, pst), lambda: (O2[1, 2], Q[1, 2].double().T @ S[1, 2].double())),
    )
    flop = 96 * 2.0 * T * T * D
    res = {}
    for nm, fn, check in cases:
        ms = hip_time(L, _lib, fn, 20)
        got, ref = check()
        res["attn_%s_us" % nm] = round(ms * 1e3, 1)
        res["attn_%s_tflops" % nm] = round(flop / (ms * 1e-3) / 1e12, 1)
        res["attn_%s_rel_err" % nm] = float((got.double() - ref).norm() / ref.norm())
    return res


def adjacent_operators(L, _lib, torch):
    """Cross-entropy over GPT-2-sized logits, an SGD step on 2^28 parameters and one convolution layer, forward and
    backward: microseconds per call and fractions of the HBM peak on algorithmic bytes (TFLOP/s for the convolution)."""
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
    ms = hip_time(L, _lib, lambda: fwd(None), 10)
    res["ce_8192x50257_loss_only_us"] = round(ms * 1e3, 1)
    res["ce_8192x50257_loss_only_frac_hbm_peak"] = round(by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)
    ms = hip_time(L, _lib, lambda: fwd(sm.data_ptr()), 10)
    res["ce_8192x50257_forward_us"] = round(ms * 1e3, 1)
    res["ce_8192x50257_forward_frac_hbm_peak"] = round(2 * by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)
    g = x  # the logits are no longer needed: their storage takes the gradient
    ms = hip_time(L, _lib, lambda: _lib.check(L.tenmo_hip_cross_entropy_backward_f32(sm.data_ptr(), t.data_ptr(), 1, up.data_ptr(), M, Cn, -100, 0.0, 2, M,
                                                                                     g.data_ptr(), 0, 0)), 10)
    res["ce_8192x50257_backward_us"] = round(ms * 1e3, 1)
    res["ce_8192x50257_backward_frac_hbm_peak"] = round(2 * by / (ms * 1e-3) / 1e9 / PEAK_HBM_GBPS, 3)
    del x, sm, g
    n = 1 << 28
    p = torch.randn(n, device="cuda")
    gr = torch.randn(n, device="cuda")
    ms = hip_time(L, _lib, lambda: _lib.check(L.tenmo_hip_sgd_step_f32(p.data_ptr(), gr.data_ptr(), None, n, 0.01, 0.0, 0.0, 0)), 10)
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
    ms = hip_time(L, _lib, lambda: _lib.check(L.tenmo_hip_conv2d_forward_f32(img.data_ptr(), nb, ci, h, w, ker.data_ptr(), co, k, k, bias.data_ptr(), 1, 1,
                                                                             out.data_ptr(), 0)), 10)
    res["conv_128x64x34x34_k3_to_128_forward_us"] = round(ms * 1e3, 1)
    res["conv_128x64x34x34_k3_to_128_forward_tflops"] = round(flop / (ms * 1e-3) / 1e12, 1)
    gi, gk, gb = torch.empty_like(img), torch.empty_like(ker), torch.empty_like(bias)
    ms = hip_time(L, _lib, lambda: _lib.check(L.tenmo_hip_conv2d_backward_f32(img.data_ptr(), nb, ci, h, w, ker.data_ptr(), co, k, k, 1, 1, out.data_ptr(),
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


def mlp_step_times(_lib, torch, np):
    """MNIST-shaped MLP 784->128->32->10, batch 64, SGD lr 0.01: ms per training step on the GPU (inputs
    already on the device) and on the CPU restatement, and the largest per-step loss difference."""
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
    for xd, yd in dev[:10]:  # warm-up steps double as the parity check
        gl.append(float(gpu.step_device(xd, yd, lr, sync=True).item()))
    cl = [cpu.step(x, y, lr) for x, y in batches[:10]]
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
    t0 = time.perf_counter()
    for x, y in batches[10:]:
        cpu.step(x, y, lr)
    cpu_ms = (time.perf_counter() - t0) * 1e3 / 20
    return {"mlp_step_ms_gpu": round(gpu_ms, 4), "mlp_step_ms_gpu_graph": round(graph_ms, 4), "mlp_step_ms_cpu": round(cpu_ms, 4), "mlp_cpu_cores": O.num_physical_cores(),
            "mlp_max_abs_loss_diff_first10": worst}


if __name__ == "__main__":
    sys.exit(main())
