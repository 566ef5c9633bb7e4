#!/usr/bin/env python3
"""Benchmark of the SGEMM / ABFT-SGEMM / SAXPY / SDOT path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one SGEMM launch at M=N=K=6144 (alpha=1, beta=0), the size the headline metric is quoted on; operands
are seeded synthetic data generated on the device, resident in HBM before the timed region.  One JSON line is
printed: `value` is the SGEMM rate in GFLOP/s, `roofline` prices the SGEMM kernel against the FP32 MFMA peak,
`cpu_baseline` times the CPU oracle's restatement of the reference's cpu_gemm on the host, and `extras` carries
the other parts of the metric (ABFT overhead and fault campaign at 4096^3, SAXPY/SDOT GB/s at 2^28, the rest of the
size sweep, rocBLAS/hipBLASLt through torch.matmul as a timed comparison only).
"""
from __future__ import annotations

import argparse
import re
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_FP32_MFMA_TFLOPS = 157.3   # 256 CU x 4 SIMD x 64 flop/clk x 2.4 GHz
PEAK_HBM_GBS = 8000.0


def profiled_traffic_bytes(summary):
    """HBM bytes per launch as the rocprofv3 summary under profiles/ states them (FETCH_SIZE and WRITE_SIZE of two
    --pmc runs, scaled by what the same counters read for a device copy of known size), or None without the file."""
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles", summary)
    try:
        text = open(path).read()
    except OSError:
        return None
    m = re.search(r"HBM traffic per launch:.*?=\s*([0-9.]+)\s*GB", text)
    return float(m.group(1)) * 1e9 if m else None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-extras", action="store_true", help="headline SGEMM line only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--ft-launches", type=int, default=1000, help="launches of the ABFT fault campaign")
    ap.add_argument("--kernel", default="all", choices=["all", "sgemm", "sgemm_1024", "sgemm_lowk", "sgemm_cm_nt", "ft_sgemm_cm_nt", "ft_sgemm", "ft_sgemm_fused", "ft_sgemm_wave", "offline_ft", "saxpy", "sdot", "copy",
                             "sgemv_n", "sgemv_t", "sgemm_deepk", "sgemm_1000", "sgemm_512", "sgemm_skinny", "ft_sgemm_skinny", "ft_sgemm_cadence",
                             "ft_sgemm_cadence_fused", "ft_sgemm_2048x1024", "ft_sgemm_weighted", "saxpy_tail", "sdot_tail"],
                    help="run one kernel only for --steps launches (for profiling with rocprofv3) and print a short line")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is a single-GPU library (no collectives); run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch

    from hpcdeepneuralnetworks_amd import blas

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    dev = "cuda"

    def timed(fn, steps, warmup):
        """Average ms per call over `steps` back-to-back launches on the current stream (HIP events on that stream)."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps

    def median_timed(fn, steps, warmup, batches=5):
        """Median over batches.  Short kernels get more calls: the clock sags within milliseconds of idling (allocating
        and filling the next operands is enough), so every measurement is preceded by at least 25 ms of the same
        call and each batch covers at least 8 ms."""
        per_call = max(timed(fn, 3, warmup), 1e-3)
        steps = min(max(steps, int(8.0 / per_call) + 1), 4000)
        lead = min(max(warmup, int(25.0 / per_call) + 1), 8000)
        return statistics.median(timed(fn, steps, lead if b == 0 else 1) for b in range(batches))

    def operands(M, N, K, seed):
        a = torch.empty(M, K, device=dev)
        b = torch.empty(K, N, device=dev)
        c = torch.empty(M, N, device=dev)
        blas.fill_uniform_matrix(a, M, K, seed)
        blas.fill_uniform_matrix(b, K, N, seed + 1)
        blas.fill_uniform_matrix(c, M, N, seed + 2)
        return a, b, c

    if args.kernel not in ("all", "sgemm"):
        # single-kernel mode for the profiler: same shapes as the full run
        if args.kernel == "sgemm_1024":
            # the reference's CPU-checkable configuration: M=N=K=1024, alpha=1, beta=0
            m = 1024
            a, b, c = operands(m, m, m, 10)
            fn = lambda: blas.sgemm(m, m, m, a, b, c, 1.0, 0.0)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel == "sgemm_lowk":
            # the low-K shape of the irregular set: 2048 tiles of 128x256, eight per persistent workgroup
            mm, kk = 8192, 256
            a, b, c = operands(mm, mm, kk, 10)
            fn = lambda: blas.sgemm(mm, mm, kk, a, b, c, 1.0, 0.0)
            work, unit = 2.0 * mm * mm * kk, "GFLOP/s"
        elif args.kernel in ("sgemm_deepk", "sgemm_1000", "sgemm_512", "sgemm_skinny"):
            # the shapes furthest from the roofline: deep K (split-K + ordered reduction), a ragged cube (edge kernel),
            # a cube for the 32x32 small-problem tile, the tall product with few columns
            mm, nn, kk = {"sgemm_deepk": (128, 128, 65536), "sgemm_1000": (1000, 1000, 1000), "sgemm_512": (512, 512, 512),
                          "sgemm_skinny": (16384, 64, 4096)}[args.kernel]
            a, b, c = operands(mm, nn, kk, 10)
            gws = blas.workspace(max(blas.sgemm_workspace_bytes(mm, nn, kk), 16))
            fn = lambda: blas.sgemm(mm, nn, kk, a, b, c, 1.0, 0.0, ws=gws)
            work, unit = 2.0 * mm * nn * kk, "GFLOP/s"
        elif args.kernel in ("ft_sgemm_skinny", "ft_sgemm_2048x1024"):
            # ABFT off the headline shape, with the class the library suggests
            mm, nn, kk = (16384, 64, 4096) if args.kernel == "ft_sgemm_skinny" else (2048, 2048, 1024)
            a, b, c = operands(mm, nn, kk, 20)
            cls = blas.ft_pick_class(mm, nn, kk)
            status = blas.ft_status_alloc(mm, nn, tile_class=cls)
            ft_ws = blas.workspace(blas.ft_workspace_bytes(mm, nn, kk))
            fn = lambda: blas.ft_sgemm(mm, nn, kk, a, b, c, 1.0, 0.0, tau=blas.ft_default_tau(kk), status=status, ws=ft_ws, tile_class=cls)
            work, unit = 2.0 * mm * nn * kk, "GFLOP/s"
        elif args.kernel == "ft_sgemm_weighted":
            # the reference's second scheme: two row sums of B, location from the ratio of the two residuals
            m = 4096
            a, b, c = operands(m, m, m, 20)
            status = blas.ft_status_alloc(m, m)
            ft_ws = blas.workspace(blas.ft_workspace_bytes(m, m, m))
            fn = lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=blas.ft_default_tau(m), status=status, ws=ft_ws,
                                       locator=blas.FT_LOCATE_WEIGHTED)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel in ("ft_sgemm_cadence", "ft_sgemm_cadence_fused"):
            # the reference's scheme: a verification every 256 values of k (ft_sgemm_huge.cuh:143)
            m = 4096
            a, b, c = operands(m, m, m, 20)
            status = blas.ft_status_alloc(m, m)
            ft_ws = blas.workspace(blas.ft_workspace_bytes(m, m, m)) if args.kernel == "ft_sgemm_cadence" else None
            fn = lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=blas.ft_default_tau(m), status=status, ws=ft_ws, check_interval=256)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel in ("saxpy_tail", "sdot_tail"):
            # the tail run of the vector configuration: n = 2^20 + 7 (latency-bound; the data fits in cache)
            nv = (1 << 20) + 7
            x = torch.empty(nv, device=dev)
            y = torch.empty(nv, device=dev)
            out = torch.zeros(1, device=dev)
            blas.fill_uniform(x, 30)
            blas.fill_uniform(y, 31)
            if args.kernel == "saxpy_tail":
                fn, work = (lambda: blas.saxpy(nv, 2.5, x, y)), 12.0 * nv
            else:
                fn, work = (lambda: blas.sdot(nv, x, y, out)), 8.0 * nv
            unit = "GB/s"
        elif args.kernel == "sgemm_cm_nt":
            # the reference family's column-major C = A * B^T at the headline size (square: the tensors serve as the
            # K x M, K x N and N x M buffers)
            m = 6144
            a, b, c = operands(m, m, m, 10)
            fn = lambda: blas.sgemm_cm_nt(m, m, m, a, b, c, 1.0, 0.0)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel == "ft_sgemm_cm_nt":
            m = 4096
            a, b, c = operands(m, m, m, 20)
            status = blas.ft_status_alloc(m, m)
            ft_ws = blas.workspace(blas.ft_cm_nt_workspace_bytes(m, m, m))
            fn = lambda: blas.ft_sgemm_cm_nt(m, m, m, a, b, c, 1.0, 0.0, ft_ws, tau=blas.ft_default_tau(m), status=status)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel == "ft_sgemm":
            m = 4096
            a, b, c = operands(m, m, m, 20)
            status = blas.ft_status_alloc(m, m)
            ft_ws = blas.workspace(blas.ft_workspace_bytes(m, m, m))
            fn = lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=blas.ft_default_tau(m), status=status, ws=ft_ws)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel in ("ft_sgemm_fused", "ft_sgemm_wave"):
            m = 4096
            a, b, c = operands(m, m, m, 20)
            wave = args.kernel == "ft_sgemm_wave"
            status = blas.ft_status_alloc(m, m, granularity=1 if wave else 0)
            ft_ws = blas.workspace(blas.ft_workspace_bytes(m, m, m)) if wave else None
            fn = lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=blas.ft_default_tau(m), status=status, ws=ft_ws,
                                       granularity=1 if wave else 0)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel == "offline_ft":
            m = 4096
            a, b, c = operands(m, m, m, 20)
            ows = blas.workspace(blas.offline_ft_workspace_bytes(m, m, m))
            res = torch.zeros(2 * (m // 256), device=dev)
            fn = lambda: blas.offline_ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, res, ows)
            work, unit = 2.0 * m ** 3, "GFLOP/s"
        elif args.kernel in ("sgemv_n", "sgemv_t"):
            mv = 16384
            am = torch.empty(mv, mv, device=dev)
            blas.fill_uniform_matrix(am, mv, mv, 40)
            xv = torch.empty(mv, device=dev)
            yv = torch.empty(mv, device=dev)
            blas.fill_uniform(xv, 41)
            gws = blas.workspace(max(blas.sgemv_workspace_bytes(mv, mv), 4))
            trans = args.kernel == "sgemv_t"
            fn = lambda: blas.sgemv(trans, mv, mv, 1.0, am, xv, 0.0, yv, ws=gws)
            work, unit = 4.0 * mv * mv, "GB/s"
        else:
            nv = 1 << 28
            x = torch.empty(nv, device=dev)
            y = torch.empty(nv, device=dev)
            out = torch.zeros(1, device=dev)
            blas.fill_uniform(x, 30)
            blas.fill_uniform(y, 31)
            if args.kernel == "saxpy":
                fn, work = (lambda: blas.saxpy(nv, 2.5, x, y)), 12.0 * nv
            elif args.kernel == "sdot":
                fn, work = (lambda: blas.sdot(nv, x, y, out)), 8.0 * nv
            else:
                z = torch.empty_like(x)
                fn, work = (lambda: z.copy_(x)), 8.0 * nv
            unit = "GB/s"
        ms = timed(fn, args.steps, args.warmup)
        print(json.dumps({"kernel": args.kernel, "steps": args.steps, "ms_per_step": round(ms, 4),
                          "value": round(work / ms / 1e6, 1), "unit": unit}))
        return 0
    if args.kernel == "sgemm":
        args.no_extras = args.no_cpu = True

    # ---------------- headline: SGEMM 6144^3, exactly K timed steps between two synchronisations
    n = 6144
    a, b, c = operands(n, n, n, 1)
    flop = 2.0 * n * n * n
    for _ in range(args.warmup):
        blas.sgemm(n, n, n, a, b, c, 1.0, 0.0)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        blas.sgemm(n, n, n, a, b, c, 1.0, 0.0)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kern_ms = e0.elapsed_time(e1) / args.steps
    gflops = flop / (wall_ms * 1e-3) / 1e9
    achieved_tflops = flop / (kern_ms * 1e-3) / 1e12

    result = {
        "metric": "sgemm_fp32_gflops_6144",
        "value": round(gflops, 1),
        "unit": "GFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic (seeded counter-based uniform[-1,1), generated on the device)",
        "config": {
            "workload": "SGEMM row-major FP32 M=N=K=6144, lda=ldb=ldc=6144, alpha=1, beta=0 "
                        "(largest size of the square sweep, the size the metric is quoted on)",
            "timing": "back-to-back launches, no per-launch sync (the reference syncs around every launch)",
        },
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved_tflops, 2),
            "peak": PEAK_FP32_MFMA_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(achieved_tflops / PEAK_FP32_MFMA_TFLOPS, 4),
            "traffic": profiled_traffic_bytes("sgemm_persistent_kernel_6144cube.md"),
            "kernel": "sgemm_persistent_kernel<192,256> (one launch = 2*6144^3 flop)",
            "kernel_ms": round(kern_ms, 4),
        },
    }

    extras = {}
    if not args.no_extras:
        st, wu = max(args.steps // 2, 10), 3
        # reference-style timing: device sync before and after every launch (kernel/sgemm/sgemm.cu:161-359)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            torch.cuda.synchronize()
            blas.sgemm(n, n, n, a, b, c, 1.0, 0.0)
            torch.cuda.synchronize()
        extras["sgemm_6144_sync_bracketed_gflops"] = round(flop * 10 / (time.perf_counter() - t0) / 1e9, 1)
        ms = median_timed(lambda: blas.sgemm(n, n, n, a, b, c, 1.0, 1.0), st, wu)
        extras["sgemm_6144_beta1_gflops"] = round(flop / ms / 1e6, 1)
        ms = median_timed(lambda: torch.matmul(a, b, out=c), st, wu)
        extras["rocblas_via_torch_6144_gflops"] = round(flop / ms / 1e6, 1)
        del a, b, c

        # square sizes of the sweep: without a workspace (no split of any kind) and with the optional workspace
        # (the tiles left over after the last full round of CUs are then split along K), hipBLASLt beside them
        sweep = {}
        for m in (1024, 2048, 3072, 4096, 5120):
            a, b, c = operands(m, m, m, 10)
            ws = blas.workspace(max(blas.sgemm_workspace_bytes(m, m, m), 4))
            ms = median_timed(lambda: blas.sgemm(m, m, m, a, b, c, 1.0, 0.0), st, wu)
            ms_ws = median_timed(lambda: blas.sgemm(m, m, m, a, b, c, 1.0, 0.0, ws=ws), st, wu)
            ms_lt = median_timed(lambda: torch.matmul(a, b, out=c), st, wu)
            sweep[str(m)] = {"no_workspace": round(2.0 * m ** 3 / ms / 1e6, 1), "workspace": round(2.0 * m ** 3 / ms_ws / 1e6, 1),
                             "hipblaslt_via_torch": round(2.0 * m ** 3 / ms_lt / 1e6, 1)}
            del a, b, c, ws
        extras["sgemm_square_gflops"] = sweep

        # irregular / skinny shapes (split-K with a caller-provided workspace where the library chooses it)
        irregular = {}
        for (M, N, K) in ((8192, 8192, 256), (16384, 64, 4096), (128, 128, 65536), (6000, 6000, 6000), (3001, 3001, 3001), (1000, 1000, 1000)):
            a, b, c = operands(M, N, K, 15)
            ws = blas.workspace(max(blas.sgemm_workspace_bytes(M, N, K), 4))
            ms = median_timed(lambda: blas.sgemm(M, N, K, a, b, c, 1.0, 0.0, ws=ws), st, wu)
            irregular[f"{M}x{N}x{K}"] = round(2.0 * M * N * K / ms / 1e6, 1)
            del a, b, c, ws
        extras["sgemm_irregular_gflops"] = irregular

        # the reference family's column-major C = A * B^T (kernel/ft_sgemm/sgemm.cu:111) on its own buffers: plain SGEMM
        # and the ABFT entry point both read the K-major operands in place (no transposed copy)
        cm = {}
        for m in (1024, 4096, 6144):
            a, b, c = operands(m, m, m, 17)   # square: the same tensors serve as the K x M, K x N and N x M buffers
            ws = blas.workspace(max(blas.sgemm_workspace_bytes(m, m, m), 4))
            ms = median_timed(lambda: blas.sgemm_cm_nt(m, m, m, a, b, c, 1.0, 0.0, ws=ws), st, wu)
            ms_lt = median_timed(lambda: torch.matmul(b.t(), a, out=c), st, wu)   # C^T = B^T^T A^T on the same memory
            cm[str(m)] = {"sgemm_cm_nt_gflops": round(2.0 * m ** 3 / ms / 1e6, 1), "hipblaslt_via_torch_tn_gflops": round(2.0 * m ** 3 / ms_lt / 1e6, 1)}
            if m == 4096:
                ft_ws_cm = blas.workspace(blas.ft_cm_nt_workspace_bytes(m, m, m))
                status_cm = blas.ft_status_alloc(m, m)
                ms_ft = median_timed(lambda: blas.ft_sgemm_cm_nt(m, m, m, a, b, c, 1.0, 0.0, ft_ws_cm, status=status_cm), st, wu)
                cm[str(m)]["ft_sgemm_cm_nt_gflops"] = round(2.0 * m ** 3 / ms_ft / 1e6, 1)
                cm[str(m)]["ft_overhead_pct_vs_sgemm_cm_nt"] = round((ms_ft - ms) / ms * 100.0, 2)
                del ft_ws_cm, status_cm
            del a, b, c, ws
        extras["column_major_a_bt"] = cm

        # ---- ABFT at 4096^3: overhead vs plain SGEMM and the seeded single-fault campaign
        m = 4096
        a, b, c = operands(m, m, m, 20)
        status = blas.ft_status_alloc(m, m)
        tau = blas.ft_default_tau(m)
        ms_plain = median_timed(lambda: blas.sgemm(m, m, m, a, b, c, 1.0, 0.0), st, wu)
        ms_plain_same_tile = median_timed(lambda: blas.sgemm(m, m, m, a, b, c, 1.0, 0.0, tile=0, split_k=1), st, wu)  # 256x128, the ABFT tile
        ft_ws = blas.workspace(blas.ft_workspace_bytes(m, m, m))
        # with the workspace: checksum vectors pre-encoded by one small kernel (timed as part of the call)
        ms_ft = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status, ws=ft_ws), st, wu)
        # without: every workgroup encodes them in its main loop
        ms_ft_fused = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status), st, wu)
        extras["abft_4096"] = {
            "sgemm_gflops": round(2.0 * m ** 3 / ms_plain / 1e6, 1),
            "sgemm_same_tile_gflops": round(2.0 * m ** 3 / ms_plain_same_tile / 1e6, 1),
            "ft_sgemm_gflops": round(2.0 * m ** 3 / ms_ft / 1e6, 1),
            "overhead_pct_vs_sgemm": round((ms_ft - ms_plain) / ms_plain * 100.0, 2),
            "overhead_pct_vs_same_tile_sgemm": round((ms_ft - ms_plain_same_tile) / ms_plain_same_tile * 100.0, 2),
            "no_workspace_ft_sgemm_gflops": round(2.0 * m ** 3 / ms_ft_fused / 1e6, 1),
            "no_workspace_overhead_pct_vs_sgemm": round((ms_ft_fused - ms_plain) / ms_plain * 100.0, 2),
            "tau": tau,
        }
        # checksum granularity and verification cadence (the reference's block- / warp- / thread-level study and its
        # verification every 256 k): time over plain SGEMM at the same size, the reference's own figures beside it
        status_w = blas.ft_status_alloc(m, m, granularity=blas.FT_GRAN_WAVE)
        ms_wave = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status_w, ws=ft_ws,
                                                     granularity=blas.FT_GRAN_WAVE), st, wu)
        status_w1 = blas.ft_status_alloc(m, m, tile_class=1, granularity=blas.FT_GRAN_WAVE)  # 64x64 wave tiles of the 128x128 class
        ms_wave1 = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status_w1, ws=ft_ws, tile_class=1,
                                                      granularity=blas.FT_GRAN_WAVE), st, wu)
        ms_cad = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status, ws=ft_ws, check_interval=256), st, wu)
        ms_cad_fused = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status, check_interval=256), st, wu)
        # the reference's second scheme: two row sums of B (weights [1, 1, ...] and [1, 2, ...]), location from their ratio
        ms_weighted = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status, ws=ft_ws,
                                                         locator=blas.FT_LOCATE_WEIGHTED), st, wu)
        pct = lambda t: round((t - ms_plain) / ms_plain * 100.0, 2)
        extras["abft_granularity_4096"] = {
            "weighted_locator_256x128_overhead_pct": pct(ms_weighted),
            "tile_256x128_overhead_pct": pct(ms_ft), "wave_tile_128x32_overhead_pct": pct(ms_wave),
            "wave_tile_64x64_of_128x128_class_overhead_pct": pct(ms_wave1),
            "tile_verify_every_256k_overhead_pct": pct(ms_cad), "tile_verify_every_256k_no_workspace_overhead_pct": pct(ms_cad_fused),
            "wave_tile_gflops": round(2.0 * m ** 3 / ms_wave / 1e6, 1),
            "reference_T4_block_warp_thread_overhead_pct": [13.49, 27.52, 45.13],    # 4761.49 / {4195.57, 3733.88, 3280.92} - 1
            "reference_A100_block_warp_thread_overhead_pct": [11.27, 13.20, 68.07],  # 17885.44 / {16073.50, 15800.36, 10641.73} - 1
            "note": "time over plain SGEMM at 4096^3; reference: fig/ABFT_GEMM/T4/fig12_step_wise_abft_plot.py:30-31, "
                    "A100/fig17_step_wise_abft_plot.py:28-29 against sgemm_huge (performance.py:22 / :21), other hardware",
        }
        ntiles = blas.ft_num_tiles(m, m)
        blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, status=status, ws=ft_ws)
        clean = blas.ft_status_numpy(status)
        c_clean = c.clone()
        rng = np.random.default_rng(2024)
        detected = located = corrected = false_pos = 0
        worst_fix = 0.0
        t0 = time.perf_counter()
        for _ in range(args.ft_launches):
            tile, i, j = int(rng.integers(ntiles)), int(rng.integers(blas.FT_TILE_M)), int(rng.integers(blas.FT_TILE_N))
            delta = float(np.float32((1 if rng.integers(2) else -1) * 10.0 ** rng.uniform(-2, 2)))
            blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=tau, fault=(tile, i, j, delta), status=status, ws=ft_ws)
            s = blas.ft_status_numpy(status)
            hit = s["flag"][tile] != 0
            detected += int(hit)
            located += int(s["flag"][tile] == 1 and s["row"][tile] == i and s["col"][tile] == j)
            others = np.delete(s["flag"], tile)
            false_pos += int(np.count_nonzero(others))
            # corrected = the whole product has the bits of the fault-free one again (the located accumulator is
            # computed again in the matrix cores' summation order)
            fix_err = 0.0 if torch.equal(c, c_clean) else float((c - c_clean).abs().max())
            corrected += int(s["flag"][tile] == 1 and fix_err == 0.0)
            worst_fix = max(worst_fix, fix_err)
        extras["abft_4096"].update({
            "campaign_launches": args.ft_launches,
            "detection_rate": detected / max(args.ft_launches, 1),
            "location_rate": located / max(args.ft_launches, 1),
            "correction_rate": corrected / max(args.ft_launches, 1),
            "false_positive_tiles": false_pos,
            "fault_free_flags": int(np.count_nonzero(clean["flag"])),
            "fault_free_max_residual": float(clean["max_clean_residual"].max()),
            "correction_criterion": "C bit-identical to the fault-free product",
            "worst_abs_error_after_correction": worst_fix,
            "campaign_seconds": round(time.perf_counter() - t0, 2),
        })
        del a, b, c, c_clean

        # ---- ABFT on a smaller problem: the tile class the library suggests (more, smaller checksum tiles)
        m, kk = 2048, 1024
        a, b, c = operands(m, m, kk, 25)
        cls = blas.ft_pick_class(m, m, kk)
        status_s = blas.ft_status_alloc(m, m, tile_class=cls)
        status_0 = blas.ft_status_alloc(m, m)
        ft_ws_s = blas.workspace(blas.ft_workspace_bytes(m, m, kk))
        ms_plain = median_timed(lambda: blas.sgemm(m, m, kk, a, b, c, 1.0, 0.0), st, wu)
        tau_s = blas.ft_default_tau(kk)
        ms_cls = median_timed(lambda: blas.ft_sgemm(m, m, kk, a, b, c, 1.0, 0.0, tau=tau_s, status=status_s, ws=ft_ws_s, tile_class=cls), st, wu)
        ms_c0 = median_timed(lambda: blas.ft_sgemm(m, m, kk, a, b, c, 1.0, 0.0, tau=tau_s, status=status_0, ws=ft_ws_s), st, wu)
        ms_scaled = median_timed(lambda: blas.ft_sgemm(m, m, kk, a, b, c, 1.0, 0.0, tau=0.0, status=status_s, ws=ft_ws_s, tile_class=cls), st, wu)
        extras["abft_2048x2048x1024"] = {
            "picked_tile_class": cls, "picked_tile": list(blas.ft_tile(cls)),
            "sgemm_gflops": round(2.0 * m * m * kk / ms_plain / 1e6, 1),
            "ft_sgemm_gflops": round(2.0 * m * m * kk / ms_cls / 1e6, 1),
            "overhead_pct_vs_sgemm": round((ms_cls - ms_plain) / ms_plain * 100.0, 2),
            "class0_256x128_ft_sgemm_gflops": round(2.0 * m * m * kk / ms_c0 / 1e6, 1),
            "default_data_scaled_threshold_overhead_pct_vs_sgemm": round((ms_scaled - ms_plain) / ms_plain * 100.0, 2),
        }
        del a, b, c

        # ---- ABFT on a product with few columns (one of the irregular shapes): the 64-column tile classes
        m, n_, kk = 16384, 64, 4096
        a, b, c = operands(m, n_, kk, 27)
        cls = blas.ft_pick_class(m, n_, kk)
        status_s = blas.ft_status_alloc(m, n_, tile_class=cls)
        status_1 = blas.ft_status_alloc(m, n_, tile_class=1)
        ft_ws_s = blas.workspace(blas.ft_workspace_bytes(m, n_, kk))
        gws = blas.workspace(max(blas.sgemm_workspace_bytes(m, n_, kk), 4))
        ms_plain = median_timed(lambda: blas.sgemm(m, n_, kk, a, b, c, 1.0, 0.0, ws=gws), st, wu)
        tau_s = blas.ft_default_tau(kk)
        ms_cls = median_timed(lambda: blas.ft_sgemm(m, n_, kk, a, b, c, 1.0, 0.0, tau=tau_s, status=status_s, ws=ft_ws_s, tile_class=cls), st, wu)
        ms_c1 = median_timed(lambda: blas.ft_sgemm(m, n_, kk, a, b, c, 1.0, 0.0, tau=tau_s, status=status_1, ws=ft_ws_s, tile_class=1), st, wu)
        ms_w = median_timed(lambda: blas.ft_sgemm(m, n_, kk, a, b, c, 1.0, 0.0, tau=tau_s, status=status_s, ws=ft_ws_s, tile_class=cls,
                                                  locator=blas.FT_LOCATE_WEIGHTED), st, wu)
        extras["abft_16384x64x4096"] = {
            "weighted_locator_overhead_pct_vs_sgemm": round((ms_w - ms_plain) / ms_plain * 100.0, 2),
            "picked_tile_class": cls, "picked_tile": list(blas.ft_tile(cls)),
            "sgemm_gflops": round(2.0 * m * n_ * kk / ms_plain / 1e6, 1),
            "ft_sgemm_gflops": round(2.0 * m * n_ * kk / ms_cls / 1e6, 1),
            "overhead_pct_vs_sgemm": round((ms_cls - ms_plain) / ms_plain * 100.0, 2),
            "class1_128x128_ft_sgemm_gflops": round(2.0 * m * n_ * kk / ms_c1 / 1e6, 1),
            "note": "one tile wide: the row checksums (a pre-pass over B only) are the screen, the column references are "
                    "formed when a row is flagged, nothing of A is summed in the loop; the tiles are split along K, two "
                    "workgroups per CU",
        }
        del a, b, c

        # ---- ABFT overhead across the square sweep (workspace variant, the tile class the library suggests)
        sweep = {}
        for m in (2048, 3001, 3072, 5120, 6000, 6144):  # (3001, 6000: ragged tiles on the last tile row and column)
            a, b, c = operands(m, m, m, 26)
            cls = blas.ft_pick_class(m, m, m)
            status_s = blas.ft_status_alloc(m, m, tile_class=cls)
            ft_ws_s = blas.workspace(blas.ft_workspace_bytes(m, m, m))
            ms_plain = median_timed(lambda: blas.sgemm(m, m, m, a, b, c, 1.0, 0.0), 10, 5, batches=3)
            ms_ft = median_timed(lambda: blas.ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, tau=blas.ft_default_tau(m), status=status_s, ws=ft_ws_s, tile_class=cls), 10, 5, batches=3)
            sweep[str(m)] = {"tile_class": cls, "sgemm_gflops": round(2.0 * m ** 3 / ms_plain / 1e6, 1),
                             "ft_sgemm_gflops": round(2.0 * m ** 3 / ms_ft / 1e6, 1),
                             "overhead_pct_vs_sgemm": round((ms_ft - ms_plain) / ms_plain * 100.0, 2)}
            del a, b, c
        extras["abft_square_sweep"] = sweep

        # ---- SAXPY / SDOT at n = 2^28 (12 and 8 algorithmic bytes per element)
        nv = 1 << 28
        x = torch.empty(nv, device=dev)
        y = torch.empty(nv, device=dev)
        out = torch.zeros(1, device=dev)
        blas.fill_uniform(x, 30)
        blas.fill_uniform(y, 31)
        ms = median_timed(lambda: blas.saxpy(nv, 2.5, x, y), 20, 3)
        extras["saxpy_2p28"] = {"GBps": round(12.0 * nv / ms / 1e6, 1), "frac_hbm_peak": round(12.0 * nv / ms / 1e6 / PEAK_HBM_GBS, 4),
                                "us": round(ms * 1e3, 1)}
        # the same with y placed 1 MiB + 8 KiB further from x than the allocator put it (x and y otherwise sit exactly
        # 1 GiB apart, the worst case for HBM channel/bank interleaving): placement, not the kernel, moves the rate
        ybig = torch.empty(nv + (1 << 19), device=dev)
        ysk = ybig[(1 << 18) + 2048:(1 << 18) + 2048 + nv]
        ysk.copy_(y)
        ms = median_timed(lambda: blas.saxpy(nv, 2.5, x, ysk), 20, 3)
        extras["saxpy_2p28"]["GBps_y_skewed_by_1MiB_8KiB"] = round(12.0 * nv / ms / 1e6, 1)
        extras["saxpy_2p28"]["x_y_distance_bytes"] = [int(y.data_ptr() - x.data_ptr()), int(ysk.data_ptr() - x.data_ptr())]
        del ybig, ysk
        ms = median_timed(lambda: blas.sdot(nv, x, y, out), 20, 3)
        extras["sdot_2p28"] = {"GBps": round(8.0 * nv / ms / 1e6, 1), "frac_hbm_peak": round(8.0 * nv / ms / 1e6 / PEAK_HBM_GBS, 4),
                               "us": round(ms * 1e3, 1)}
        z = torch.empty_like(x)
        ms = median_timed(lambda: z.copy_(x), 20, 3)
        extras["device_copy_2p28_GBps"] = round(8.0 * nv / ms / 1e6, 1)
        del z
        # the tail run (n = 2^20 + 7): these kernels take 4 us, less than the host needs to issue a call from Python
        # (about 7 us), so the eager loop measures the host; the same call captured 50 times into a HIP graph and
        # replayed measures the device
        nt = (1 << 20) + 7

        def graph_timed(fn, calls=50, replays=40):
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            g = torch.cuda.CUDAGraph()
            with torch.cuda.stream(side):
                fn()
                torch.cuda.synchronize()
                with torch.cuda.graph(g, stream=side):
                    for _ in range(calls):
                        fn()
            torch.cuda.synchronize()
            for _ in range(5):
                g.replay()
            torch.cuda.synchronize()
            g0, g1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            g0.record()
            for _ in range(replays):
                g.replay()
            g1.record()
            torch.cuda.synchronize()
            return g0.elapsed_time(g1) / (replays * calls)

        dot_ws = blas.workspace(64 + 8 * 4096)   # hpcdnn_workspace_bytes(HPCDNN_OP_SDOT): the call's own scratch, no allocation under capture
        ms = median_timed(lambda: blas.saxpy(nt, 2.5, x, y), 50, 5)
        extras["saxpy_2p20_plus_7_GBps"] = round(12.0 * nt / ms / 1e6, 1)
        ms_g = graph_timed(lambda: blas.saxpy(nt, 2.5, x, y))
        extras["saxpy_2p20_plus_7"] = {"us_eager_python_loop": round(ms * 1e3, 2), "us_graph_replay": round(ms_g * 1e3, 2),
                                       "GBps_graph_replay": round(12.0 * nt / ms_g / 1e6, 1)}
        ms = median_timed(lambda: blas.sdot(nt, x, y, out, ws=dot_ws), 50, 5)
        extras["sdot_2p20_plus_7_GBps"] = round(8.0 * nt / ms / 1e6, 1)
        ms_g = graph_timed(lambda: blas.sdot(nt, x, y, out, ws=dot_ws))
        extras["sdot_2p20_plus_7"] = {"us_eager_python_loop": round(ms * 1e3, 2), "us_graph_replay": round(ms_g * 1e3, 2),
                                      "GBps_graph_replay": round(8.0 * nt / ms_g / 1e6, 1)}
        del x, y

        # ---- SGEMV (4 algorithmic bytes per matrix element) and the offline ABFT baseline built from it
        mv = 16384
        am = torch.empty(mv, mv, device=dev)
        blas.fill_uniform_matrix(am, mv, mv, 40)
        xv = torch.empty(mv, device=dev)
        yv = torch.empty(mv, device=dev)
        blas.fill_uniform(xv, 41)
        gws = blas.workspace(max(blas.sgemv_workspace_bytes(mv, mv), 4))
        ms_n = median_timed(lambda: blas.sgemv(False, mv, mv, 1.0, am, xv, 0.0, yv), 20, 3)
        ms_t = median_timed(lambda: blas.sgemv(True, mv, mv, 1.0, am, xv, 0.0, yv, ws=gws), 20, 3)
        extras["sgemv_16384"] = {"n_GBps": round(4.0 * mv * mv / ms_n / 1e6, 1), "t_GBps": round(4.0 * mv * mv / ms_t / 1e6, 1),
                                 "n_frac_hbm_peak": round(4.0 * mv * mv / ms_n / 1e6 / PEAK_HBM_GBS, 4),
                                 "t_frac_hbm_peak": round(4.0 * mv * mv / ms_t / 1e6 / PEAK_HBM_GBS, 4)}
        del am, xv, yv, gws
        m = 4096
        a, b, c = operands(m, m, m, 20)
        ows = blas.workspace(blas.offline_ft_workspace_bytes(m, m, m))
        res = torch.zeros(2 * (m // 256), device=dev)
        ms_plain = median_timed(lambda: blas.sgemm(m, m, m, a, b, c, 1.0, 0.0), st, wu)
        ms_off = median_timed(lambda: blas.offline_ft_sgemm(m, m, m, a, b, c, 1.0, 0.0, res, ows), st, wu)
        extras["offline_abft_4096"] = {"gflops": round(2.0 * m ** 3 / ms_off / 1e6, 1),
                                       "overhead_pct_vs_sgemm": round((ms_off - ms_plain) / ms_plain * 100.0, 2),
                                       "max_abs_residual_sum": float(res.abs().max())}
        del a, b, c, ows
        result["extras"] = extras

    # ---------------- CPU baseline: the oracle's restatement of the reference's cpu_gemm, one thread, bounded sample
    if not args.no_cpu:
        import oracle

        m = 1024
        ha = oracle.fill_uniform_matrix(m, m, 1)
        hb = oracle.fill_uniform_matrix(m, m, 2)
        hc = np.zeros((m, m), dtype=np.float32)
        runs = []
        for _ in range(3):  # about 12 s of CPU work in all
            t0 = time.perf_counter()
            oracle.cpu_gemm(1.0, 0.0, ha, hb, m, hc)
            runs.append(time.perf_counter() - t0)
        dt = statistics.median(runs)
        result["cpu_baseline"] = {
            "value": round(2.0 * m ** 3 / dt / 1e9, 3),
            "unit": "GFLOP/s",
            "cores": 1,
            "kind": "port",
            "sample": f"oracle cpu_gemm (naive i-j-k, float accumulator, reference utils/utils.cu:93-103) at "
                      f"M=N=K=1024 (the reference's CPU-runnable configuration), median of three runs, {dt:.2f} s each; "
                      f"host has {os.cpu_count()} logical CPUs",
        }
        result["cpu_baseline"]["openmp_threads"] = oracle.num_threads()
        if not args.no_extras:
            # the FP64-accumulated validator (OpenMP) on the same product, labelled apart: it is the checker of the parity
            # tests, not the reference's routine
            runs = []
            for _ in range(3):
                t0 = time.perf_counter()
                oracle.gemm_f64_rows(m, m, m, ha, m, hb, m, None, m, 1.0, 0.0)
                runs.append(time.perf_counter() - t0)
            dv = statistics.median(runs)
            result["cpu_baseline"]["fp64_validator_openmp_1024cube"] = {
                "GFLOPs": round(2.0 * m ** 3 / dv / 1e9, 2), "seconds": round(dv, 3), "threads": oracle.num_threads()}
            # SAXPY (fused multiply-add) and SDOT (double accumulate) at both sizes of the vector configuration, on one
            # thread and on the OpenMP pool; wall clock around each call, median of three
            vec = {}
            for label, nv in (("2p28", 1 << 28), ("2p20_plus_7", (1 << 20) + 7)):
                hx, hy = oracle.fill_uniform(nv, 3), oracle.fill_uniform(nv, 4)
                reps = 3 if nv > (1 << 24) else 15
                t = {"saxpy_1": [], "saxpy_omp": [], "sdot_1": [], "sdot_omp": []}
                for _ in range(reps):
                    t0 = time.perf_counter()
                    oracle.saxpy(2.5, hx, hy)
                    t1 = time.perf_counter()
                    oracle.saxpy_omp(2.5, hx, hy)
                    t2 = time.perf_counter()
                    oracle.sdot_f64_serial(hx, hy)
                    t3 = time.perf_counter()
                    oracle.sdot_f64(hx, hy)
                    t4 = time.perf_counter()
                    for key, d in zip(t, (t1 - t0, t2 - t1, t3 - t2, t4 - t3)):
                        t[key].append(d)
                md = {key: statistics.median(v) for key, v in t.items()}
                vec[label] = {
                    "n": nv,
                    "saxpy_GBps_1_thread": round(12.0 * nv / md["saxpy_1"] / 1e9, 2),
                    "saxpy_GBps_openmp": round(12.0 * nv / md["saxpy_omp"] / 1e9, 2),
                    "sdot_GBps_1_thread": round(8.0 * nv / md["sdot_1"] / 1e9, 2),
                    "sdot_GBps_openmp": round(8.0 * nv / md["sdot_omp"] / 1e9, 2),
                    "saxpy_ms_1_thread": round(md["saxpy_1"] * 1e3, 3), "sdot_ms_1_thread": round(md["sdot_1"] * 1e3, 3),
                }
                del hx, hy
            vec["openmp_threads"] = oracle.num_threads()
            result["cpu_baseline"]["vector"] = vec

    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
