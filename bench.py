#!/usr/bin/env python3
"""Benchmark of the quantized matmul path on one MI355X.

Default workload (the configuration the headline metric is quoted on): HQ4_G32 decode GEMV,
M = 1, K = 5120, N = 17408, fused activation FWHT, cold-streamed over a ring of weight copies
larger than the 256 MB Infinity Cache.  One step = one GEMV launch over one bank of the ring.

Prints ONE JSON line: metric/value (GB/s over the algorithmic bytes), the HBM roofline of the
kernel measured with HIP events on the launch stream, and the CPU baseline (the reference's
oracle form - dequantize the bank to fp32, then one fp32 product - restated in numpy and timed
on this box's host cores over a bounded sample).

Other workloads: --workload c1|c2|c3|c4_decode|c4_prefill|c5_qkv|c5_down (see WORKLOADS).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0      # MI355X HBM3E, published
MFMA_PEAK_TFLOPS = 2500.0  # MI355X dense f16/bf16 MFMA, published


def _fail(msg: str) -> None:
    print(msg, file=sys.stderr)
    sys.exit(2)


def cpu_baseline_gemv(blocks, x_rot16, bits, group, is_m5, algo_bytes_full, rows_sample):
    """Reference CPU oracle form on a row sample: dequant whole sample to fp32 (f16-rounded), then sgemv."""
    from oracle import qworacle as qo
    sample = blocks[:rows_sample]
    frac = sample.shape[0] / blocks.shape[0]
    reps, t_total = 0, 0.0
    while t_total < 10.0 and reps < 50:
        t0 = time.perf_counter()
        qo.cpu_oracle_gemv(sample, x_rot16, bits, group, is_m5)
        t_total += time.perf_counter() - t0
        reps += 1
    sec = t_total / reps
    try:
        import threadpoolctl
        cores = max(int(i.get("num_threads", 1)) for i in threadpoolctl.threadpool_info()) if threadpoolctl.threadpool_info() else 1
    except Exception:
        cores = 1
    return {"value": round(algo_bytes_full * frac / sec / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"{sample.shape[0]} of {blocks.shape[0]} rows, numpy dequant-to-fp32 + fp32 product, "
                      f"{reps} reps, {sec * 1e3:.1f} ms each"}


def run_gemv(args, fmt, n, k, m, label, outliers):
    from oracle import qworacle as qo
    from qwegn_amd import qwhip
    from tests import helpers as H

    dev = qwhip.Device(0)
    kind, bits, group, is_m5, rotate = H.FORMATS[fmt]
    blocks, w16 = H.make_bank(fmt, n, k, seed=0)
    x32 = H.make_x(m, k, 100, outliers=outliers)
    x16 = x32.astype(np.float16)
    bank_bytes = blocks.nbytes
    ring_n = max(2, int(np.ceil(args.ring_mb * 1e6 / bank_bytes))) if not args.hot else 1
    banks = [dev.put(blocks) for _ in range(ring_n)]
    views = [H.view_of(dev, b, fmt, n, k) for b in banks]
    xb = dev.put(x16)
    y16 = dev.alloc(m * n * 2)
    prerot = bool(rotate) and (args.prerot or m > 1)     # verify (m > 1) activations arrive rotated by their producer
    x_basis = H.x_in_basis(x16, fmt)
    if prerot:
        xb = dev.put(x_basis)
    flags = (args.variant << 8) | (args.rt << 12) | (qwhip.X_PREROTATED if prerot else 0)
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_gemv(st, C.byref(views[i % ring_n]), xb.ptr, qwhip.F16, m, flags, y16.ptr, None))

    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    t0 = time.perf_counter()
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    wall = time.perf_counter() - t0
    ms = e0.elapsed_ms(e1)
    us_per = ms * 1e3 / args.steps

    got = y16.download(np.float16, (m, n))
    err = qo.normalized_error(got, qo.matmul_ref_f64(x_basis, w16))
    if not err <= 2e-3:
        _fail(f"bench: output failed parity (normalized error {err:.3e})")

    algo_bytes = bank_bytes + m * k * 2 + m * n * 2
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    out = {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": m, "N": n, "K": k, "fused_fwht": bool(rotate) and not prerot,
                   "cache": "hot" if args.hot else f"cold ring of {ring_n} banks ({ring_n * bank_bytes / 1e6:.0f} MB)"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None,
                     "algorithmic_bytes": algo_bytes, "kernel_us": round(us_per, 3)},
        "normalized_error": err, "wall_ms_per_step": round(wall * 1e3 / args.steps, 6),
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_gemv(blocks, x_basis, bits, group, is_m5, algo_bytes,
                                                rows_sample=min(n, args.cpu_rows))
    return out


def run_gemm(args, fmt, n, k, m, label):
    """Prefill GEMM: X bf16 [m, k] in the container's basis -> Y bf16 [m, n]; one step = one launch."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip
    from tests import helpers as H

    dev = qwhip.Device(0)
    kind, bits, group, is_m5, rotate = H.FORMATS[fmt]
    blocks, w16 = H.make_bank(fmt, n, k, seed=0)
    x32 = H.make_x(m, k, 100)
    xbits = qo.f32_to_bf16_bits(x32)
    bank, xb, yb = dev.put(blocks), dev.put(xbits), dev.alloc(m * n * 2)
    ws = dev.alloc(m * k * 2)                      # f16 copy of the bf16 activations (one conversion pass per launch, timed)
    view = H.view_of(dev, bank, fmt, n, k)
    flags = qwhip.X_PREROTATED | (args.cfg << 8)
    lib, st = dev.lib, dev.stream.handle

    def launch():
        qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, qwhip.BF16, m, 0, yb.ptr, qwhip.BF16, 0, flags, ws.ptr, ws.nbytes))

    for _ in range(args.warmup):
        launch()
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for _ in range(args.steps):
        launch()
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    # parity on a row sample (full-size parity is a test)
    rows = np.arange(0, m, max(1, m // 64))[:64]
    got = qo.bf16_bits_to_f32(yb.download(np.uint16, (m, n)))[rows]
    ref = qo.matmul_ref_f64(qo.round_bf16(x32)[rows].astype(np.float16), w16)
    err = qo.normalized_error(got, ref)
    if not err <= 2e-3:
        _fail(f"bench: GEMM output failed parity (normalized error {err:.3e})")
    flops = 2.0 * m * n * k
    tf = flops / (us_per * 1e-6) / 1e12
    out = {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": m, "N": n, "K": k, "x": "bf16 (in the weight basis)", "y": "bf16"},
        "roofline": {"bound": "mfma", "achieved": round(tf, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / MFMA_PEAK_TFLOPS, 4), "traffic": None, "algorithmic_flops": flops,
                     "kernel_us": round(us_per, 3)},
        "normalized_error": err,
    }
    if not args.no_cpu:
        sample = min(m, 256)
        xs = qo.round_bf16(x32)[:sample].astype(np.float16)
        t0 = time.perf_counter()
        qo.cpu_oracle_gemv(blocks, xs, bits, group, is_m5)
        sec = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(2.0 * sample * n * k / sec / 1e12, 4), "unit": "TFLOP/s", "cores": os.cpu_count(),
                               "kind": "port", "sample": f"{sample} of {m} tokens, numpy dequant-to-fp32 + sgemm, {sec * 1e3:.0f} ms"}
    return out


WORKLOADS = {
    # label: (runner kind, fmt, n, k, m, outliers)
    "c1": ("gemv", "aq4_g32", 4096, 4096, 1, False),
    "c2": ("gemv", "hq4_g32_m5", 17408, 5120, 1, True),
    "c3": ("gemm", "hq4_g32_m5", 5120, 5120, 4096, False),
    "c5_qkv": ("gemv", "hq8_g32", 7168, 5120, None, False),
    "c5_down": ("gemv", "hq4_g64", 5120, 17408, None, False),
}
LABELS = {
    "c1": "C1 AQ4_G32 affine GEMV N=4096 K=4096",
    "c2": "C2 HQ4_G32 decode GEMV M=1 K=5120 N=17408 fused FWHT",
    "c3": "C3 HQ4_G32 prefill GEMM M=4096 K=5120 N=5120",
    "c5_qkv": "C5 verify GEMM HQ8_G32 K=5120 N=7168",
    "c5_down": "C5 verify GEMM HQ4_G64 K=17408 N=5120",
}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS) + ["headline"],
                    help="headline = c2 (the bench line) with the c3 prefill GEMM summarised under 'prefill_gemm'")
    ap.add_argument("--m", type=int, default=8, help="activation rows for the c5 workloads")
    ap.add_argument("--hot", action="store_true", help="single bank (Infinity-Cache resident) instead of the cold ring")
    ap.add_argument("--ring-mb", type=float, default=640.0)
    ap.add_argument("--variant", type=int, default=0, help="gemv kernel override (0 auto, 1 dot2, 2 mfma)")
    ap.add_argument("--rt", type=int, default=0, help="row tiles per wave for the mfma gemv (0 auto)")
    ap.add_argument("--cfg", type=int, default=0, help="gemm tile shape override (0 auto)")
    ap.add_argument("--prerot", action="store_true", help="hand the gemv activations already rotated")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=4096)
    args = ap.parse_args()
    if args.gpus != 1:
        _fail("bench.py: this build measures one GPU only (every box has one); run with --gpus 1")
    if args.workload == "headline":
        kind, fmt, n, k, m, outliers = WORKLOADS["c2"]
        out = run_gemv(args, fmt, n, k, m, LABELS["c2"], outliers)
        gargs = argparse.Namespace(**vars(args))
        gargs.steps, gargs.warmup, gargs.no_cpu = max(10, args.steps // 10), max(3, args.warmup // 4), True
        kind, fmt, n, k, m, outliers = WORKLOADS["c3"]
        g = run_gemm(gargs, fmt, n, k, m, LABELS["c3"])
        out["prefill_gemm"] = {"value": g["value"], "unit": g["unit"], "ms_per_step": g["ms_per_step"], "steps": g["steps"],
                               "config": g["config"], "roofline": g["roofline"], "normalized_error": g["normalized_error"]}
        print(json.dumps(out))
        return
    kind, fmt, n, k, m, outliers = WORKLOADS[args.workload]
    if m is None:
        m = args.m
    if kind == "gemm":
        out = run_gemm(args, fmt, n, k, m, LABELS[args.workload])
    else:
        out = run_gemv(args, fmt, n, k, m, LABELS[args.workload] + (f" M={m}" if args.workload.startswith("c5") else ""), outliers)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
