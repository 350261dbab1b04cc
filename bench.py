#!/usr/bin/env python3
"""Benchmark of the quantized matmul path on one MI355X.

Default workload (the configuration the headline metric is quoted on): HQ4_G32 decode GEMV,
M = 1, K = 5120, N = 17408, fused activation FWHT, cold-streamed over a ring of weight copies
larger than the 256 MB Infinity Cache.  One step = one GEMV launch over one bank of the ring.

Prints ONE JSON line: metric/value (GB/s over the algorithmic bytes), the HBM roofline of the
kernel measured with HIP events on the launch stream, and the CPU baseline (the reference's
oracle form - dequantize the bank to fp32, then one fp32 product - restated in numpy and timed
on this box's host cores over a bounded sample).

Other workloads: --workload c1|c2|c3|c4_decode|c4_prefill|c5_qkv|c5_down|mlp_gate_up|mlp_prefill|head|f32_decode|f32_verify4|f32_batched64|repack|norm_prefill|norm_decode (see WORKLOADS).
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

# HBM bytes per launch of the dominant kernel under its automatic configuration come from rocprofv3 --pmc passes
# (FETCH_SIZE KiB x 1024 x 2.000 + WRITE_SIZE KiB x 1024 x 1.000; the factors come from a streaming kernel of known
# size).  The passes are recorded as text under profiles/; the figure is read from the summary's line
# "traffic = <bytes> B per launch", so the bench line cannot drift from the committed profile.
TRAFFIC_PROFILES = {"c2": "gemv_col__c2_decode_n17408_k5120.txt", "c3": "gemm3_pingpong_256x320__c3_prefill_m4096_n5120_k5120.txt",
                    "c4_decode": "moe_decode_col__c4_decode_t1.txt", "c4_prefill": "moe_grouped_gemm__c4_prefill_t2048.txt"}


def measured_traffic(workload: str):
    """Bytes per launch from the committed rocprof summary of `workload`, or None when there is none."""
    import re
    name = TRAFFIC_PROFILES.get(workload)
    path = os.path.join(ROOT, "profiles", name) if name else None
    if not path or not os.path.exists(path):
        return None
    m = re.search(r"^\s*traffic\s*=\s*([0-9][0-9,]*)\s*B per launch", open(path).read(), re.M)
    return int(m.group(1).replace(",", "")) if m else None


def _fail(msg: str) -> None:
    print(msg, file=sys.stderr)
    sys.exit(2)


def _spin_up(dev, launch, ms: float = 150.0) -> None:
    """Untimed: repeats `launch(i)` for `ms` of wall clock before the warm-up steps. The card's clocks take tens of
    milliseconds of load to settle; a short run timed from idle reads 10-15 % slow."""
    t0, i = time.perf_counter(), 0
    while (time.perf_counter() - t0) * 1e3 < ms:
        for _ in range(16):
            launch(i)
            i += 1
        dev.stream.sync()


def _oracle_clib():
    """The oracle's C restatement (built by __graft_entry__.build(); compiled here with gcc when missing)."""
    from oracle import build_oracle
    if not build_oracle.LIB.exists():
        build_oracle.build()
    return C.CDLL(str(build_oracle.LIB))


def cpu_baseline_gemv(blocks, x_basis16, bits, group, is_m5, algo_bytes_full, rows_sample, budget_s=10.0):
    """Reference CPU oracle form (dequantize the bank to f16-rounded fp32, then one fp32 matrix-vector product:
    Scripts/oracle/gen_s1_q4_fixtures.py:28-31) in the oracle's C restatement, OpenMP over rows, on a row sample."""
    lib = _oracle_clib()
    sample = np.ascontiguousarray(blocks[:rows_sample])
    n_s, k = sample.shape[0], x_basis16.shape[-1]
    frac = n_s / blocks.shape[0]
    x = np.ascontiguousarray(x_basis16.reshape(-1, k)[0]).view(np.uint16)
    scratch, xf, y = np.empty((n_s, k), np.float32), np.empty(k, np.float32), np.empty(n_s, np.float32)
    vp = lambda a: a.ctypes.data_as(C.c_void_p)

    def once():
        if is_m5:
            lib.qwo_oracle_gemv_hq4(vp(sample), vp(x), C.c_int64(n_s), C.c_int64(k), vp(scratch), vp(xf), vp(y))
        else:
            lib.qwo_oracle_gemv_blocks(vp(sample), vp(x), C.c_int64(n_s), C.c_int64(k), bits, group, vp(scratch), vp(xf), vp(y))

    once()
    reps, t_total = 0, 0.0
    while t_total < budget_s and reps < 2000:
        t0 = time.perf_counter()
        once()
        t_total += time.perf_counter() - t0
        reps += 1
    sec = t_total / reps
    return {"value": round(algo_bytes_full * frac / sec / 1e9, 3), "unit": "GB/s", "cores": int(lib.qwo_threads()), "kind": "port",
            "sample": f"{n_s} of {blocks.shape[0]} rows, one activation row, C restatement of the oracle form (dequantize to fp32, "
                      f"then sgemv; OpenMP), {reps} reps, {sec * 1e3:.1f} ms each"}


def run_gemv(args, fmt, n, k, m, label, outliers, traffic=None, cpu_later=None):
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
    if getattr(args, "invariant", False):
        flags |= qwhip.GEMV_ROW_INVARIANT
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_gemv(st, C.byref(views[i % ring_n]), xb.ptr, qwhip.F16, m, flags, y16.ptr, None))

    _spin_up(dev, launch)
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
    # the yardstick: a launch that only reads the same banks (four 16-byte loads in flight per thread, one atomic per wave),
    # timed the same way over the same cold ring; its sum is checked against the host's
    sum_dev = dev.alloc(256 * 8)
    qwhip.check(lib.qwhip_fill_u32(st, sum_dev.ptr, 0, 512))
    qwhip.check(lib.qwhip_plane_checksum(st, banks[0].ptr, bank_bytes, sum_dev.ptr))
    dev.stream.sync()
    if int(sum_dev.download(np.uint64, (256,)).sum()) != int(blocks.ravel().view(np.uint32).astype(np.uint64).sum()):
        _fail("bench: plane checksum differs from the host's")
    for i in range(args.warmup):
        lib.qwhip_plane_checksum(st, banks[i % ring_n].ptr, bank_bytes, sum_dev.ptr)
    e0.record(dev.stream)
    for i in range(args.steps):
        lib.qwhip_plane_checksum(st, banks[i % ring_n].ptr, bank_bytes, sum_dev.ptr)
    e1.record(dev.stream)
    dev.stream.sync()
    read_us = e0.elapsed_ms(e1) * 1e3 / args.steps
    rows_us = None
    if fmt == "hq4_g32_m5" and m == 1:
        # the second yardstick: the decode GEMV's own launch (grid, 20-byte pieces per lane, rows in flight) with the
        # arithmetic taken out
        row_bytes = (k // 32) * 20
        qwhip.check(lib.qwhip_fill_u32(st, sum_dev.ptr, 0, 512))
        qwhip.check(lib.qwhip_plane_checksum_rows(st, banks[0].ptr, n, row_bytes, sum_dev.ptr))
        dev.stream.sync()
        if int(sum_dev.download(np.uint64, (256,)).sum()) != int(blocks.ravel().view(np.uint32).astype(np.uint64).sum()):
            _fail("bench: row checksum differs from the host's")
        for i in range(args.warmup):
            lib.qwhip_plane_checksum_rows(st, banks[i % ring_n].ptr, n, row_bytes, sum_dev.ptr)
        e0.record(dev.stream)
        for i in range(args.steps):
            lib.qwhip_plane_checksum_rows(st, banks[i % ring_n].ptr, n, row_bytes, sum_dev.ptr)
        e1.record(dev.stream)
        dev.stream.sync()
        rows_us = e0.elapsed_ms(e1) * 1e3 / args.steps
    out = {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": m, "N": n, "K": k, "fused_fwht": bool(rotate) and not prerot,
                   "cache": "hot" if args.hot else f"cold ring of {ring_n} banks ({ring_n * bank_bytes / 1e6:.0f} MB)"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": traffic if (args.variant == 0 and args.rt == 0 and not args.prerot and not getattr(args, "invariant", False)) else None,
                     "algorithmic_bytes": algo_bytes, "kernel_us": round(us_per, 3),
                     "read_only_launch_us": round(read_us, 3), "read_only_frac": round(bank_bytes / (read_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                     "read_only_rows_launch_us": None if rows_us is None else round(rows_us, 3),
                     "read_only_rows_frac": None if rows_us is None else round(bank_bytes / (rows_us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)},
        "normalized_error": err, "wall_ms_per_step": round(wall * 1e3 / args.steps, 6),
    }
    if not args.no_cpu:
        def baseline():
            return cpu_baseline_gemv(blocks, x_basis, bits, group, is_m5, algo_bytes, rows_sample=min(n, args.cpu_rows))
        if cpu_later is not None:
            cpu_later.append(baseline)     # the caller runs it after its GPU legs: ten seconds of host work idle the card
        else:
            out["cpu_baseline"] = baseline()
    return out


def cpu_baseline_c1(budget_s: float = 5.0):
    """The configuration the reference's CPU oracle path is named for (C1: AQ4_G32 affine GEMV, N = K = 4096): the oracle form
    in its C restatement on this box's host cores, over the whole bank."""
    from tests import helpers as H
    kind, fmt, n, k, m, outliers = WORKLOADS["c1"]
    _, bits, group, is_m5, _ = H.FORMATS[fmt]
    blocks, _ = H.make_bank(fmt, n, k, seed=0)
    x16 = H.make_x(1, k, 100).astype(np.float16)
    out = cpu_baseline_gemv(blocks, H.x_in_basis(x16, fmt), bits, group, is_m5, blocks.nbytes + k * 2 + n * 2, n, budget_s)
    out["config"] = LABELS["c1"]
    return out


def run_silu_pair(args, fmt, inter, k, m, label):
    """Dense MLP gate|up GEMV with the SwiGLU + rotation epilogue: act[m, inter] from a [2*inter, k] bank; one step = one launch."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip
    from tests import helpers as H

    dev = qwhip.Device(0)
    blocks, w16 = H.make_bank(fmt, 2 * inter, k, seed=0)
    x16 = H.make_x(m, k, 100).astype(np.float16)
    ring_n = max(2, int(np.ceil(args.ring_mb * 1e6 / blocks.nbytes))) if not args.hot else 1
    banks = [dev.put(blocks) for _ in range(ring_n)]
    views = [H.view_of(dev, b, fmt, 2 * inter, k) for b in banks]
    xb, act = dev.put(x16), dev.alloc(m * inter * 2)
    flags = args.variant << 8
    rot_out = 0 if getattr(args, "plain_out", False) else 1      # 0: act in the plain basis, the down projection rotates its input itself
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_gemv_silu_pair(st, C.byref(views[i % ring_n]), xb.ptr, qwhip.F16, m, flags, rot_out, act.ptr))

    _spin_up(dev, launch)
    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    got = act.download(np.float16, (m, inter)).astype(np.float32)
    gu = qo.matmul_ref_f64(H.x_in_basis(x16, fmt), w16)
    want = qo.swiglu_fwht_f16(gu[:, :inter].astype(np.float32), gu[:, inter:].astype(np.float32), rotate=bool(rot_out)).astype(np.float32)
    err = qo.normalized_error(got, want)
    if not err <= 2e-3:
        _fail(f"bench: SwiGLU pair output failed parity (normalized error {err:.3e})")
    algo_bytes = blocks.nbytes + m * k * 2 + m * inter * 2
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": m, "N": 2 * inter, "K": k, "fused_fwht": True, "output_rotation": bool(rot_out),
                   "cache": "hot" if args.hot else f"cold ring of {ring_n} banks ({ring_n * blocks.nbytes / 1e6:.0f} MB)"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "algorithmic_bytes": algo_bytes,
                     "kernel_us": round(us_per, 3)},
        "normalized_error": err,
    }


def run_mlp_decode(args, inter, hidden, label):
    """Dense MLP decode step on HQ4_G32_M5 banks, one token: gate|up GEMV with the gated activation, then the down GEMV;
    one step = the two launches.  Two forms of the same step: the reference's (the first launch also rotates act into the
    down bank's basis) and the one that suits this device (act stays plain, the down GEMV rotates its input in its prologue,
    which is free at one row, and the gate|up bank is read by the decode GEMV's own kernel).  Both are checked against the
    fp64 chain."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip
    from tests import helpers as H

    fmt = "hq4_g32_m5"
    dev = qwhip.Device(0)
    gu_blocks, gu16 = H.make_bank(fmt, 2 * inter, hidden, seed=0)
    dn_blocks, dn16 = H.make_bank(fmt, hidden, inter, seed=1)
    x16 = H.make_x(1, hidden, 100).astype(np.float16)
    step_bytes = gu_blocks.nbytes + dn_blocks.nbytes
    ring_n = max(2, int(np.ceil(args.ring_mb * 1e6 / step_bytes))) if not args.hot else 1
    gus, dns = [dev.put(gu_blocks) for _ in range(ring_n)], [dev.put(dn_blocks) for _ in range(ring_n)]
    vgu = [H.view_of(dev, b, fmt, 2 * inter, hidden) for b in gus]
    vdn = [H.view_of(dev, b, fmt, hidden, inter) for b in dns]
    xb, act, yb = dev.put(x16), dev.alloc(inter * 2), dev.alloc(hidden * 4)
    lib, st = dev.lib, dev.stream.handle

    def step(i, plain):
        qwhip.check(lib.qwhip_gemv_silu_pair(st, C.byref(vgu[i % ring_n]), xb.ptr, qwhip.F16, 1, 0, 0 if plain else 1, act.ptr))
        qwhip.check(lib.qwhip_gemv(st, C.byref(vdn[i % ring_n]), act.ptr, qwhip.F16, 1, 0 if plain else qwhip.X_PREROTATED, None, yb.ptr))

    gu = qo.matmul_ref_f64(H.x_in_basis(x16, fmt), gu16)
    act_ref = qo.swiglu_fwht_f16(gu[:, :inter].astype(np.float32), gu[:, inter:].astype(np.float32), rotate=True)
    want = qo.matmul_ref_f64(act_ref, dn16)
    res = {}
    for name, plain in (("reference_form", False), ("plain_act_form", True)):
        step(0, plain)
        dev.stream.sync()
        err = float(qo.normalized_error(yb.download(np.float32, (1, hidden)), want))
        if not err <= 2e-3:
            _fail(f"bench: dense MLP decode step ({name}) failed parity (normalized error {err:.3e})")
        _spin_up(dev, lambda i: step(i, plain))
        for i in range(args.warmup):
            step(i, plain)
        dev.stream.sync()
        e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
        e0.record(dev.stream)
        for i in range(args.steps):
            step(i, plain)
        e1.record(dev.stream)
        dev.stream.sync()
        res[name] = {"us_per_step": round(e0.elapsed_ms(e1) * 1e3 / args.steps, 3), "normalized_error": err}
    algo_bytes = step_bytes + hidden * 2 + 2 * inter * 2 + hidden * 4
    us_per = res["plain_act_form"]["us_per_step"]
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    for v in res.values():
        v["GB/s"] = round(algo_bytes / (v["us_per_step"] * 1e-6) / 1e9, 2)
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": 1, "hidden": hidden, "intermediate": inter,
                   "cache": "hot" if args.hot else f"cold ring of {ring_n} bank pairs ({ring_n * step_bytes / 1e6:.0f} MB)"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": algo_bytes, "kernel_us": us_per, "forms": res},
        "normalized_error": res["plain_act_form"]["normalized_error"],
    }


def run_head(args, fmt, n, k, label):
    """LM head for greedy decoding: GEMV over the vocabulary rows into f32 logits + per-row argmax fold; one step = both
    launches.  Algorithmic bytes: the bank, x, the logits written and read back once."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip
    from tests import helpers as H

    dev = qwhip.Device(0)
    blocks, w16 = H.make_bank(fmt, n, k, seed=0)
    x16 = H.make_x(1, k, 100).astype(np.float16)
    bank, xb = dev.put(blocks), dev.put(x16)
    logits, tok = dev.alloc(n * 4), dev.alloc(256)
    view = H.view_of(dev, bank, fmt, n, k)
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_head_argmax(st, C.byref(view), xb.ptr, qwhip.F16, 1, 0, logits.ptr, tok.ptr))

    launch(0)
    dev.stream.sync()
    got = logits.download(np.float32, (1, n))
    err = qo.normalized_error(got, qo.matmul_ref_f64(H.x_in_basis(x16, fmt), w16))
    if not (err <= 2e-3 and int(tok.download(np.int32, (1,))[0]) == int(qo.head_argmax(got)[0])):
        _fail(f"bench: head argmax failed parity (normalized error {err:.3e})")
    _spin_up(dev, launch)
    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    algo_bytes = blocks.nbytes + k * 2 + 2 * n * 4
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": 1, "N": n, "K": k, "cache": "one bank (larger than the Infinity Cache)"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": algo_bytes, "kernel_us": round(us_per, 3)},
        "normalized_error": err,
    }


def run_gemv_f32(args, fmt, n, k, m, label):
    """f32-activation GEMV (fp32 arithmetic, epilogue 0): one step = one pass over the bank for all m rows."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip
    from tests import helpers as H

    dev = qwhip.Device(0)
    _, bits, group, is_m5, _ = H.FORMATS[fmt]
    blocks, _ = H.make_bank(fmt, n, k, seed=0)
    x = H.make_x(m, k, 100)
    bank, xb, yb = dev.put(blocks), dev.put(x), dev.alloc(m * n * 4)
    view = H.view_of(dev, bank, fmt, n, k)
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_gemv_f32(st, C.byref(view), xb.ptr, m, 0, 1.0, yb.ptr))

    launch(0)
    dev.stream.sync()
    sample = min(n, 512)
    err = qo.normalized_error(yb.download(np.float32, (m, n))[:, :sample], qo.gemv_f32(blocks[:sample], x, bits, group, is_m5))
    if not err <= 2e-5:
        _fail(f"bench: f32 gemv failed parity (normalized error {err:.3e})")
    _spin_up(dev, launch)
    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    algo_bytes = blocks.nbytes + m * k * 4 + m * n * 4
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": m, "N": n, "K": k},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": algo_bytes, "kernel_us": round(us_per, 3)},
        "normalized_error": err,
    }


def run_mlp_prefill(args, inter, k, m, label):
    """Dense MLP prefill gate|up: X f16 [m, k] in the weight basis -> act f16 [m, inter] through the GEMM with the SwiGLU + FWHT-32
    epilogue fused; one step = one launch.  The bank is written by the device quantizer; parity on a sample of outputs."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip

    dev = qwhip.Device(0)
    lib, st = dev.lib, dev.stream.handle
    rng = np.random.default_rng(0)
    n = 2 * inter
    bank = dev.alloc(n * (k // 32) * 20)
    for r0 in range(0, n, 4096):           # weights N(0, 0.02), quantized on the device chunk by chunk
        rows_here = min(4096, n - r0)
        wsrc = dev.put((rng.standard_normal((rows_here, k), dtype=np.float32) * np.float32(0.02)))
        qwhip.check(lib.qwhip_quantize_hq4_g32(st, wsrc.ptr, qwhip.F32, rows_here, k, 0, bank.ptr + r0 * (k // 32) * 20))
        dev.stream.sync()
    view = dev.view(bank, n, k, qwhip.KIND_HQ4_G32_M5)
    x16 = rng.standard_normal((m, k), dtype=np.float32).astype(np.float16)
    xb, act = dev.put(x16), dev.alloc(m * inter * 2)

    def launch(i):
        qwhip.check(lib.qwhip_gemm_swiglu(st, C.byref(view), xb.ptr, qwhip.F16, m, 0, 1, act.ptr, 0, qwhip.X_PREROTATED, None, 0))

    launch(0)
    dev.stream.sync()
    # parity: the first 64 outputs (two rotation groups) of 64 sampled rows against the oracle on the downloaded blocks
    blocks = bank.download(np.uint8, (n, k // 32, 20))
    cols = np.arange(64)
    wg = qo.weights_f16_exact(blocks[cols], 4, 32, True)
    wu = qo.weights_f16_exact(blocks[inter + cols], 4, 32, True)
    rows = np.arange(0, m, max(1, m // 64))[:64]
    g = qo.matmul_ref_f64(x16[rows], wg).astype(np.float16).astype(np.float32)
    u = qo.matmul_ref_f64(x16[rows], wu).astype(np.float16).astype(np.float32)
    want = qo.swiglu_fwht_f16(g, u, rotate=True).astype(np.float32)
    got = act.download(np.float16, (m, inter))[rows][:, :64].astype(np.float32)
    err = qo.normalized_error(got, want)
    if not err <= 2e-3:
        _fail(f"bench: fused gate_up output failed parity (normalized error {err:.3e})")
    _spin_up(dev, launch, 300.0)
    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    flops = 2.0 * m * n * k
    tf = flops / (us_per * 1e-6) / 1e12
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": "hq4_g32_m5", "M": m, "N": n, "K": k, "x": "f16 (in the weight basis)", "act": "f16 [M, N/2]"},
        "roofline": {"bound": "mfma", "kernel": "gate|up GEMM with the SwiGLU + FWHT-32 epilogue", "achieved": round(tf, 2),
                     "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS, 4), "traffic": None,
                     "algorithmic_flops": flops, "kernel_us": round(us_per, 3)},
        "normalized_error": err,
    }


def run_repack(args, rows, cols, bits, group, label):
    """Load-time MLX affine -> AQ repack: one step = one launch.  Algorithmic bytes: codes and headers read, blocks written."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip

    dev = qwhip.Device(0)
    rng = np.random.default_rng(0)
    groups, payload = cols // group, group * bits // 8
    w = rng.integers(0, 256, size=(rows, groups * payload), dtype=np.uint8)
    sc = qo.f32_to_bf16_bits(rng.uniform(1e-3, 0.05, size=rows * groups).astype(np.float32))
    bi = qo.f32_to_bf16_bits((-rng.uniform(1e-2, 0.3, size=rows * groups)).astype(np.float32))
    wb, sb, bb_ = dev.put(w), dev.put(sc), dev.put(bi)
    out, cnt = dev.alloc(rows * groups * (4 + payload)), dev.put(np.zeros(1, np.uint32))
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_repack_mlx_affine(st, wb.ptr, sb.ptr, bb_.ptr, qwhip.BF16, rows, cols, bits, group, out.ptr, cnt.ptr))

    launch(0)
    dev.stream.sync()
    sample = min(rows, 64)
    want, refused = qo.repack_mlx_affine(w[:sample], sc[:sample * groups], bi[:sample * groups], sample, cols, bits, group, False)
    if not (np.array_equal(out.download(np.uint8, (rows, groups, 4 + payload))[:sample], want) and int(cnt.download(np.uint32, (1,))[0]) == 0):
        _fail("bench: repacked blocks differ from the oracle's")
    _spin_up(dev, launch)
    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    algo_bytes = rows * groups * (payload + 4) * 2
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8", "data": "synthetic",
        "config": {"workload": label, "rows": rows, "cols": cols, "bits": bits, "group": group},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": algo_bytes, "kernel_us": round(us_per, 3)},
    }


def run_norm(args, rows, hidden, label):
    """RMSNorm + rotation producer with the fused residual update: one step = one launch over [rows, hidden] f16.
    Algorithmic bytes: x read, residual read and written, y written, gamma read."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip

    dev = qwhip.Device(0)
    rng = np.random.default_rng(0)
    x16 = rng.standard_normal((rows, hidden)).astype(np.float16)
    gam = (rng.standard_normal(hidden) * 0.1).astype(np.float16)
    res0 = rng.standard_normal((rows, hidden)).astype(np.float16)
    xb, gb, rb, yb = dev.put(x16), dev.put(gam), dev.put(res0), dev.alloc(rows * hidden * 2)
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_rmsnorm(st, xb.ptr, gb.ptr, rb.ptr, rows, hidden, 1e-6, 1, yb.ptr))

    launch(0)
    dev.stream.sync()
    want, want_res = qo.rmsnorm_rot_f16(x16, gam, 1e-6, residual16=res0)
    got = yb.download(np.float16, (rows, hidden))
    err = float(np.max(np.abs(got.astype(np.float32) - want.astype(np.float32))))
    if not (err <= 1e-3 * max(1.0, float(np.max(np.abs(want)))) and np.array_equal(rb.download(np.float16, (rows, hidden)), want_res)):
        _fail(f"bench: norm output failed parity (max abs error {err:.3e})")
    _spin_up(dev, launch)
    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    algo_bytes = rows * hidden * 2 * 4 + hidden * 2
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": label, "rows": rows, "hidden": hidden, "residual": True, "rotate": True},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": algo_bytes, "kernel_us": round(us_per, 3)},
        "max_abs_error": err,
    }


def run_dense_f32(args, rows, n, k, label):
    """Dense fp32-weight GEMV door with no epilogue: one step = one launch, y[rows, n] = x[rows, k] W[n, k]^T.
    Algorithmic bytes: the weights once, the activation rows once, the outputs once."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip

    dev = qwhip.Device(0)
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((n, k)) / np.sqrt(k)).astype(np.float32)
    x = rng.standard_normal((rows, k)).astype(np.float32)
    wb, xb, yb = dev.put(w), dev.put(x), dev.alloc(rows * n * 4)
    lib, st = dev.lib, dev.stream.handle

    def launch(i):
        qwhip.check(lib.qwhip_f32_gemv(st, wb.ptr, xb.ptr, rows, n, k, 0, 1.0, yb.ptr))

    launch(0)
    dev.stream.sync()
    err = float(qo.normalized_error(yb.download(np.float32, (rows, n)), qo.f32_gemv(w, x, 0, 1.0)))
    if not err <= 2e-6:
        _fail(f"bench: dense f32 gemv failed parity (normalized error {err:.3e})")
    _spin_up(dev, launch)
    for i in range(args.warmup):
        launch(i)
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for i in range(args.steps):
        launch(i)
    e1.record(dev.stream)
    dev.stream.sync()
    us_per = e0.elapsed_ms(e1) * 1e3 / args.steps
    algo_bytes = (n * k + rows * k + rows * n) * 4
    gbs = algo_bytes / (us_per * 1e-6) / 1e9
    return {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": label, "rows": rows, "n": n, "k": k, "weights": "hot (one resident matrix)"},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(gbs / HBM_PEAK_GBS, 4),
                     "traffic": None, "algorithmic_bytes": algo_bytes, "kernel_us": round(us_per, 3)},
        "normalized_error": err,
    }


def vendor_plain_bmm(batch, m, n, k, steps=50):
    """The grouped counterpart of vendor_plain_gemm: `batch` independent products [m, k] x [n, k]^T on dense f16 / bf16
    operands (torch.bmm -> the vendor library's batched GEMM), i.e. an MoE layer's grouped GEMM if every expert got exactly
    m rows and its weights were ready-made f16 matrices."""
    import torch
    dev = torch.device("cuda:0")
    res = {}
    for name, dt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        a = torch.randn(batch, m, k, device=dev, dtype=dt)
        bt = (torch.randn(batch, n, k, device=dev, dtype=dt) * 0.02).transpose(1, 2)
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < 300.0:
            for _ in range(8):
                torch.bmm(a, bt)
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            torch.bmm(a, bt)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / steps
        tf = 2.0 * batch * m * n * k / (us * 1e-6) / 1e12
        res[name] = {"kernel_us": round(us, 3), "tflops": round(tf, 2), "frac": round(tf / MFMA_PEAK_TFLOPS, 4)}
    return res


def vendor_plain_gemm(m, n, k, steps=100):
    """A yardstick for the matrix pipe, as the read-only launches are for HBM: the vendor library's plain GEMM (PyTorch ->
    hipBLASLt) Y[m, n] = X[m, k] W[n, k]^T on dense f16 and bf16 operands of the same shape - no quantized bank, no
    dequantization - after the same spin-up, timed with events.  Nothing of the product is involved."""
    import torch
    dev = torch.device("cuda:0")
    res = {}
    for name, dt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        a = torch.randn(m, k, device=dev, dtype=dt)
        bt = (torch.randn(n, k, device=dev, dtype=dt) * 0.02).t()
        t0 = time.perf_counter()
        while (time.perf_counter() - t0) * 1e3 < 300.0:
            for _ in range(16):
                torch.matmul(a, bt)
            torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            torch.matmul(a, bt)
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / steps
        tf = 2.0 * m * n * k / (us * 1e-6) / 1e12
        res[name] = {"kernel_us": round(us, 3), "tflops": round(tf, 2), "frac": round(tf / MFMA_PEAK_TFLOPS, 4)}
    return res


def run_gemm(args, fmt, n, k, m, label, traffic=None):
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
    # f16 copy of the bf16 activations (only the kernels that do not convert in place use it), plus what --gemm-ws-mb asks for
    ws = dev.alloc(max(m * k * 2, getattr(args, "gemm_ws_mb", 0) << 20))
    view = H.view_of(dev, bank, fmt, n, k)
    flags = qwhip.X_PREROTATED | (args.cfg << 8)
    lib, st = dev.lib, dev.stream.handle

    def launch():
        qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, qwhip.BF16, m, 0, yb.ptr, qwhip.BF16, 0, flags, ws.ptr, ws.nbytes))

    _spin_up(dev, lambda i: launch())
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
    # parity of the step's output on a row sample (full-size parity is a test)
    rows = np.arange(0, m, max(1, m // 64))[:64]
    got = qo.bf16_bits_to_f32(yb.download(np.uint16, (m, n)))[rows]
    ref = qo.matmul_ref_f64(qo.round_bf16(x32)[rows].astype(np.float16), w16)
    err = qo.normalized_error(got, ref)
    if not err <= 2e-3:
        _fail(f"bench: GEMM output failed parity (normalized error {err:.3e})")
    # for comparison: the same kernel on f16 activations (no conversion in its staging phase); flags bit 16 makes one call
    # run the separate bf16 -> f16 pass into the workspace first
    qwhip.check(lib.qwhip_gemm(st, C.byref(view), xb.ptr, qwhip.BF16, m, 0, yb.ptr, qwhip.BF16, 0, flags | (1 << 16), ws.ptr, ws.nbytes))

    def launch_kernel_only():
        qwhip.check(lib.qwhip_gemm(st, C.byref(view), ws.ptr, qwhip.F16, m, 0, yb.ptr, qwhip.BF16, 0, flags, None, 0))

    _spin_up(dev, lambda i: launch_kernel_only())      # the parity check above left the card idle for seconds
    for _ in range(args.warmup):
        launch_kernel_only()
    dev.stream.sync()
    e0.record(dev.stream)
    for _ in range(args.steps):
        launch_kernel_only()
    e1.record(dev.stream)
    dev.stream.sync()
    us_kernel = e0.elapsed_ms(e1) * 1e3 / args.steps
    flops = 2.0 * m * n * k
    tf = flops / (us_per * 1e-6) / 1e12
    tf_k = flops / (us_kernel * 1e-6) / 1e12
    out = {
        "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)",
        "value": round(tf, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(us_per / 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": label, "format": fmt, "M": m, "N": n, "K": k, "x": "bf16 (in the weight basis)", "y": "bf16"},
        "roofline": {"bound": "mfma", "kernel": "the whole step: one launch of the quantized GEMM kernel, bf16 activations converted to f16 while the tile is staged",
                     "achieved": round(tf, 2), "peak": MFMA_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tf / MFMA_PEAK_TFLOPS, 4), "traffic": traffic if args.cfg == 0 else None,
                     "algorithmic_flops": flops, "kernel_us": round(us_per, 3),
                     "f16_activation_kernel_us": round(us_kernel, 3), "f16_activation_kernel_tflops": round(tf_k, 2)},
        "normalized_error": err,
    }
    if getattr(args, "vendor_gemm", False):
        # in a process of its own: PyTorch brings its own HIP runtime, which must not meet the one this library links
        import subprocess
        try:
            child = subprocess.run([sys.executable, os.path.abspath(__file__), "--workload", "vendor_gemm", "--gemm-rows", str(m)],
                                   capture_output=True, text=True, timeout=120)
            lines = [ln for ln in child.stdout.splitlines() if ln.startswith("{")]
            out["roofline"]["vendor_plain_gemm"] = json.loads(lines[-1])["vendor_plain_gemm"] if child.returncode == 0 and lines else None
        except (subprocess.TimeoutExpired, OSError, ValueError, KeyError):
            out["roofline"]["vendor_plain_gemm"] = None      # no PyTorch here, or it took too long: the yardstick is optional
    if not args.no_cpu:
        sample = min(m, 256)
        xs = qo.round_bf16(x32)[:sample].astype(np.float16)
        t0 = time.perf_counter()
        qo.cpu_oracle_gemv(blocks, xs, bits, group, is_m5)
        sec = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": round(2.0 * sample * n * k / sec / 1e12, 4), "unit": "TFLOP/s", "cores": os.cpu_count(),
                               "kind": "port", "sample": f"{sample} of {m} tokens, numpy dequant-to-fp32 + sgemm, {sec * 1e3:.0f} ms"}
    return out


class _LazyExpertBank:
    """Dequantizes one expert's exact f16 weights on demand from the host copy of a bank (oracle side of the parity check)."""

    def __init__(self, blocks, experts, rows, k, keep=True):
        self.blocks, self.shape, self._cache, self.keep = blocks.reshape(experts, rows, k // 32, 20), (experts, rows, k), {}, keep

    def __getitem__(self, e):
        from oracle import qworacle as qo
        if e in self._cache:
            return self._cache[e]
        w = qo.weights_f16_exact(self.blocks[e], 4, 32, True)
        if self.keep:
            self._cache[e] = w
        return w


def run_moe(args, t, label):
    """C4: 128 experts, top-8, hidden 2048, intermediate 768, HQ4_G32 banks.  One step = the whole routed-expert
    operator on t tokens from router logits to the combined output.  t <= 8: routed GEMVs (HBM bound, bf16 hidden
    un-rotated, rotation fused); t > 8: pair sort + grouped GEMMs (MFMA bound, bf16 hidden in the experts' basis, or f16
    with --moe-f16), every token checked against the fp64 oracle."""
    from oracle import qworacle as qo
    from qwegn_amd import qwhip

    E, K, Hd, I = 128, 8, 2048, 768
    dev = qwhip.Device(0)
    lib, st = dev.lib, dev.stream.handle
    rng = np.random.default_rng(0)
    gub, dnb = dev.alloc(E * 2 * I * (Hd // 32) * 20), dev.alloc(E * Hd * (I // 32) * 20)
    src = dev.alloc(2 * I * Hd * 4)
    check_e0 = None
    for e in range(E):                       # banks are written by the device quantizer (byte-identical to the packer)
        wg = rng.standard_normal((2 * I, Hd), dtype=np.float32) * np.float32(0.02)
        src.upload(wg)
        qwhip.check(lib.qwhip_quantize_hq4_g32(st, src.ptr, qwhip.F32, 2 * I, Hd, 1, gub.ptr + e * 2 * I * (Hd // 32) * 20))
        wd = rng.standard_normal((Hd, I), dtype=np.float32) * np.float32(0.02)
        src.upload(wd)
        qwhip.check(lib.qwhip_quantize_hq4_g32(st, src.ptr, qwhip.F32, Hd, I, 1, dnb.ptr + e * Hd * (I // 32) * 20))
        if e == 0:
            check_e0 = (wg, wd)
    dev.stream.sync()
    gu_blocks = gub.download(np.uint8, (E * 2 * I, Hd // 32, 20))
    dn_blocks = dnb.download(np.uint8, (E * Hd, I // 32, 20))
    if not (np.array_equal(gu_blocks[:2 * I], qo.quant_hq4_blocks(check_e0[0])) and np.array_equal(dn_blocks[:Hd], qo.quant_hq4_blocks(check_e0[1]))):
        _fail("bench: device quantizer bytes differ from the oracle's")
    vgu = dev.view(gub, E * 2 * I, Hd, qwhip.KIND_HQ4_G32_M5)
    vdn = dev.view(dnb, E * Hd, I, qwhip.KIND_HQ4_G32_M5)

    x32 = rng.standard_normal((t, Hd), dtype=np.float32)
    pairs = t * K
    decode = t <= 8
    # decode: a cycle of E / K steps whose tokens all route to different experts (a strong offset on a step's own K experts
    # of a random partition), so that consecutive steps read different experts and the cycle walks every expert of both
    # banks (377 MB, beyond the 256 MB Infinity Cache): cold figures.  Prefill: one batch of plain random logits.
    cycle = E // K if decode else 1
    logits_cycle = rng.standard_normal((cycle, t, E), dtype=np.float32)
    if decode:
        part = rng.permutation(E).reshape(cycle, K)
        shared = int(getattr(args, "moe_shared", 0) or 0)      # routes of a step's tokens 1.. that repeat token 0's experts
        for i in range(cycle):
            for j in range(t):
                own = part[(i * t + j) % cycle].copy()
                if j > 0 and shared:
                    own[:shared] = part[(i * t) % cycle][:shared]
                logits_cycle[i, j, own] += np.float32(12.0)
    logits = logits_cycle[0]
    lbs = [dev.put(np.ascontiguousarray(logits_cycle[i])) for i in range(cycle)]
    lb, ib, wb = lbs[0], dev.alloc(pairs * 4), dev.alloc(pairs * 4)
    act, out = dev.alloc(pairs * I * 2), dev.alloc(t * Hd * 4)
    if decode:
        xv = qo.round_bf16(x32)
        xb = dev.put(qo.f32_to_bf16_bits(x32))
        x_basis = qo.fwht32_ortho(xv).astype(np.float16)

        gu_flags = qwhip.MOE_REUSE_EXPERTS if getattr(args, "moe_reuse", False) else 0

        def gate_up(i=0):   # the dominant launch: routing + routed gate|up GEMVs + SwiGLU + rotation
            qwhip.check(lib.qwhip_moe_route_gateup_decode(st, C.byref(vgu), E, xb.ptr, qwhip.BF16, gu_flags, lbs[i % cycle].ptr, t, K, 1, 1.0,
                                                          ib.ptr, wb.ptr, act.ptr))

        def chain(i=0):
            gate_up(i)
            qwhip.check(lib.qwhip_moe_down_decode(st, C.byref(vdn), E, act.ptr, ib.ptr, wb.ptr, t, K, None, None, out.ptr, qwhip.F32))
    else:
        if getattr(args, "moe_f16", False):
            x_basis, xcode = qo.rotate_activation_f16(x32), qwhip.F16
            xb = dev.put(x_basis)
        else:       # bf16 rows in the experts' basis (the producer's rotation in fp32, one bf16 rounding)
            xbits, xcode = qo.f32_to_bf16_bits(qo.fwht32_ortho(x32)), qwhip.BF16
            x_basis, xb = qo.bf16_bits_to_f32(xbits), dev.put(xbits)
        mt = max(1, lib.qwhip_moe_max_tiles(E, pairs))
        off, sp, stok, inv = dev.alloc((E + 1) * 4), dev.alloc(pairs * 4), dev.alloc(pairs * 4), dev.alloc(pairs * 4)
        te, tr, tc = dev.alloc(mt * 4), dev.alloc(mt * 4), dev.alloc(16)
        dn_out = dev.alloc(pairs * Hd * 2)

        def gate_up(i=0):   # grouped gate|up GEMM with the SwiGLU + FWHT-32 epilogue fused
            qwhip.check(lib.qwhip_moe_grouped_gemm_swiglu(st, C.byref(vgu), E, xb.ptr, xcode, 0, stok.ptr, off.ptr, te.ptr, tr.ptr,
                                                          tc.ptr, mt, pairs, 1, act.ptr, 0))

        def chain(i=0):
            qwhip.check(lib.qwhip_moe_route(st, lb.ptr, t, E, K, 1, 1.0, ib.ptr, wb.ptr))
            qwhip.check(lib.qwhip_moe_group_pairs(st, ib.ptr, E, pairs, K, off.ptr, sp.ptr, stok.ptr, inv.ptr, te.ptr, tr.ptr, tc.ptr, 1))
            gate_up()
            qwhip.check(lib.qwhip_moe_grouped_gemm(st, C.byref(vdn), E, act.ptr, qwhip.F16, 0, None, off.ptr, te.ptr, tr.ptr, tc.ptr,
                                                   mt, pairs, dn_out.ptr, qwhip.F16, 0))
            qwhip.check(lib.qwhip_moe_combine(st, dn_out.ptr, qwhip.F16, inv.ptr, wb.ptr, t, K, Hd, None, None, out.ptr, qwhip.F32))

    def timed(fn, steps, warmup, hot=False):
        step = (lambda i: fn(0)) if hot else fn
        _spin_up(dev, step, 100.0)
        for i in range(warmup):
            step(i)
        dev.stream.sync()
        e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
        e0.record(dev.stream)
        for i in range(steps):
            step(i)
        e1.record(dev.stream)
        dev.stream.sync()
        return e0.elapsed_ms(e1) * 1e3 / steps

    us_chain = timed(chain, args.steps, args.warmup)
    us_gu = timed(gate_up, args.steps, max(2, args.warmup // 4))      # the dominant kernel alone, same inputs
    us_chain_hot = timed(chain, args.steps, max(2, args.warmup // 4), hot=True) if decode else None
    us_graph = None
    if decode:
        # the same cold cycle as one HIP graph (2 * cycle kernel nodes), replayed: what the step costs when the host's launch
        # calls are out of the way; the last replay's output must equal the eager step's, bit for bit
        graph = qwhip.Graph(dev.stream, lambda: [chain(i) for i in range(cycle)])
        reps = max(2, args.steps // cycle)
        for _ in range(3):
            graph.launch()
        dev.stream.sync()
        g0, g1 = qwhip.Event(dev), qwhip.Event(dev)
        g0.record(dev.stream)
        for _ in range(reps):
            graph.launch()
        g1.record(dev.stream)
        dev.stream.sync()
        us_graph = g0.elapsed_ms(g1) * 1e3 / (reps * cycle)
        replayed = out.download(np.uint32, (t, Hd))
        chain(cycle - 1)
        dev.stream.sync()
        if not np.array_equal(replayed, out.download(np.uint32, (t, Hd))):
            _fail("bench: the graph replay's output differs from the eager step's")
        graph.destroy()
    chain(0)                                                           # the step that is checked: the cycle's first
    dev.stream.sync()
    got = out.download(np.float32, (t, Hd))
    idx, wts = ib.download(np.int32, (t, K)), wb.download(np.float32, (t, K))
    ridx, rwts = qo.moe_route(logits, K, True, 1.0)
    if not (np.array_equal(idx, ridx) and np.allclose(wts, rwts, rtol=1e-5, atol=1e-7)):
        _fail("bench: routing differs from the oracle's")
    if decode:
        ref = qo.moe_forward_f64(x_basis, idx, wts, _LazyExpertBank(gu_blocks, E, 2 * I, Hd), _LazyExpertBank(dn_blocks, E, Hd, I),
                                 act_f16=True, rotate_act=True)
    else:           # every token: the oracle's expert-ordered form, two fp64 matrix products per expert
        ref = qo.moe_forward_grouped_f64(x_basis, idx, wts, _LazyExpertBank(gu_blocks, E, 2 * I, Hd, keep=False),
                                         _LazyExpertBank(dn_blocks, E, Hd, I, keep=False), act_f16=True, rotate_act=True)
    err = qo.normalized_error(got, ref)
    row_err = np.sqrt(((got - ref) ** 2).sum(axis=1) / np.maximum((ref ** 2).sum(axis=1), 1e-300))
    if not (err <= 2e-3 and float(row_err.max()) <= 2e-3):
        _fail(f"bench: MoE output failed parity (normalized error {err:.3e}, worst token {float(row_err.max()):.3e})")

    base = {"n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us_chain / 1e3, 6), "higher_is_better": True,
            "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
            "metric": "HQ4 GEMV GB/s (% HBM peak) at M=1; prefill GEMM TFLOP/s (% MFMA peak)", "normalized_error": err,
            "worst_token_error": float(row_err.max()), "tokens_checked": int(t)}
    cfg = {"workload": label, "format": "hq4_g32_m5", "tokens": t, "experts": E, "top_k": K, "hidden": Hd, "intermediate": I,
           "activations": "bf16" if decode or not getattr(args, "moe_f16", False) else "f16"}
    if decode:
        used = len({int(e) for e in idx.ravel() if e >= 0})      # bytes are counted once per distinct expert of the step
        w_bytes = used * (2 * I * (Hd // 32) * 20 + Hd * (I // 32) * 20)
        algo = w_bytes + t * Hd * 2 + t * Hd * 4 + t * E * 4
        gu_bytes = used * 2 * I * (Hd // 32) * 20 + t * Hd * 2 + pairs * I * 2
        gbs, gu_gbs = algo / (us_chain * 1e-6) / 1e9, gu_bytes / (us_gu * 1e-6) / 1e9
        cfg["distinct_experts_per_step"] = used
        cfg["cache"] = (f"cold: a cycle of {cycle} steps whose tokens route to different experts walks all {E} experts "
                        f"({E * (2 * I * (Hd // 32) * 20 + Hd * (I // 32) * 20) / 1e6:.0f} MB of banks)")
        base["graph_replay"] = {"ms_per_step": round(us_graph / 1e3, 6), "value": round(algo / (us_graph * 1e-6) / 1e9, 2), "unit": "GB/s",
                                "note": f"the cold cycle of {cycle} steps captured as one HIP graph and replayed"}
        base["hot_cache"] = {"ms_per_step": round(us_chain_hot / 1e3, 6), "value": round(algo / (us_chain_hot * 1e-6) / 1e9, 2), "unit": "GB/s",
                             "note": "the same step repeated: its experts (23.6 MB per token) stay in the Infinity Cache"}
        base.update({"value": round(gbs, 2), "unit": "GB/s", "config": cfg,
                     "roofline": {"bound": "hbm", "kernel": "routed gate_up GEMV", "achieved": round(gu_gbs, 2), "peak": HBM_PEAK_GBS,
                                  "unit": "GB/s", "frac": round(gu_gbs / HBM_PEAK_GBS, 4),
                                  "traffic": measured_traffic("c4_decode") if (t == 1 and not getattr(args, "moe_tokens", 0) and not getattr(args, "hot", False)) else None,
                                  "algorithmic_bytes": gu_bytes, "kernel_us": round(us_gu, 3)}})
    else:
        valid = int((idx >= 0).sum())
        flops = valid * (2.0 * 2 * I * Hd + 2.0 * Hd * I)
        gu_flops = valid * 2.0 * 2 * I * Hd
        tf, gu_tf = flops / (us_chain * 1e-6) / 1e12, gu_flops / (us_gu * 1e-6) / 1e12
        base.update({"value": round(tf, 2), "unit": "TFLOP/s", "config": cfg,
                     "roofline": {"bound": "mfma", "kernel": "grouped gate_up GEMM", "achieved": round(gu_tf, 2), "peak": MFMA_PEAK_TFLOPS,
                                  "unit": "TFLOP/s", "frac": round(gu_tf / MFMA_PEAK_TFLOPS, 4),
                                  "traffic": measured_traffic("c4_prefill") if (t == 2048 and not getattr(args, "moe_f16", False)) else None,
                                  "algorithmic_flops": gu_flops, "kernel_us": round(us_gu, 3)}})
    if not args.no_cpu:
        rows_c = np.arange(min(t, 2))
        t0 = time.perf_counter()
        qo.moe_forward_f64(x_basis[rows_c], idx[rows_c], wts[rows_c], _LazyExpertBank(gu_blocks, E, 2 * I, Hd),
                           _LazyExpertBank(dn_blocks, E, Hd, I), act_f16=True, rotate_act=True)
        sec = time.perf_counter() - t0
        per_tok = sec / len(rows_c)
        if decode:
            v, u = (K * (2 * I * (Hd // 32) * 20 + Hd * (I // 32) * 20)) / per_tok / 1e9, "GB/s"
        else:
            v, u = K * (2.0 * 2 * I * Hd + 2.0 * Hd * I) / per_tok / 1e12, "TFLOP/s"
        base["cpu_baseline"] = {"value": round(v, 5), "unit": u, "cores": 1, "kind": "port",
                                "sample": f"{len(rows_c)} token(s): numpy oracle (dequantize the routed experts, fp64 products), {sec:.1f} s"}
    return base


def run_calibration(args):
    """A plain streaming kernel of known size (f32 -> f16 cast of 2^26 elements: reads 256 MiB, writes 128 MiB), the
    reference point the FETCH_SIZE / WRITE_SIZE counter readings of the other workloads are scaled by."""
    from qwegn_amd import qwhip
    dev = qwhip.Device(0)
    n = 1 << 26
    src, dst = dev.alloc(n * 4), dev.alloc(n * 2)
    qwhip.check(dev.lib.qwhip_fill_u32(dev.stream.handle, src.ptr, 0x3F800000, n))
    for _ in range(args.warmup):
        qwhip.check(dev.lib.qwhip_cast_f32_to_f16(dev.stream.handle, src.ptr, dst.ptr, n))
    dev.stream.sync()
    e0, e1 = qwhip.Event(dev), qwhip.Event(dev)
    e0.record(dev.stream)
    for _ in range(args.steps):
        qwhip.check(dev.lib.qwhip_cast_f32_to_f16(dev.stream.handle, src.ptr, dst.ptr, n))
    e1.record(dev.stream)
    dev.stream.sync()
    us = e0.elapsed_ms(e1) * 1e3 / args.steps
    if not np.all(dst.download(np.float16, (1024,)) == np.float16(1.0)):
        _fail("bench: calibration kernel wrote wrong values")
    return {"workload": "calibration cast f32->f16", "read_bytes": n * 4, "write_bytes": n * 2, "kernel_us": round(us, 3),
            "GB/s": round(n * 6 / (us * 1e-6) / 1e9, 1)}


WORKLOADS = {
    # label: (runner kind, fmt, n, k, m, outliers)
    "c1": ("gemv", "aq4_g32", 4096, 4096, 1, False),
    "c2": ("gemv", "hq4_g32_m5", 17408, 5120, 1, True),
    "c3": ("gemm", "hq4_g32_m5", 5120, 5120, 4096, False),
    "c4_decode": ("moe", None, None, None, 1, False),
    "c4_prefill": ("moe", None, None, None, 2048, False),
    "c5_qkv": ("gemv", "hq8_g32", 7168, 5120, None, False),
    "c5_down": ("gemv", "hq4_g64", 5120, 17408, None, False),
    "mlp_gate_up": ("pair", "hq4_g32_m5", 17408, 5120, 1, False),      # n = intermediate size: the bank has 2n rows
    "mlp_prefill": ("mlp_prefill", "hq4_g32_m5", 17408, 5120, 4096, False),   # n = intermediate size
    "mlp_decode": ("mlp_decode", "hq4_g32_m5", 17408, 5120, 1, False),         # n = intermediate size, k = hidden
    "head": ("head", "hq4_g32_m5", 151936, 5120, 1, False),
    "f32_decode": ("gemv_f32", "hq4_g32_m5", 17408, 5120, 1, False),
    "f32_verify4": ("gemv_f32", "hq4_g32_m5", 17408, 5120, 4, False),
    "f32_batched64": ("gemv_f32", "hq4_g32_m5", 17408, 5120, 64, False),      # 32 rows and more: the matrix-core form
    "repack": ("repack", None, 34816, 5120, None, False),              # MLX 4-bit group 64, gate|up sized
    "norm_prefill": ("norm", None, 5120, None, 4096, False),           # n = hidden, m = rows
    "norm_decode": ("norm", None, 5120, None, 1, False),
    "dense_f32_ba": ("dense_f32", None, 64, 2048, 1, False),           # the gated-delta b|a projection of one token
    "dense_f32_square": ("dense_f32", None, 5120, 5120, 1, False),
}
LABELS = {
    "c1": "C1 AQ4_G32 affine GEMV N=4096 K=4096",
    "c2": "C2 HQ4_G32 decode GEMV M=1 K=5120 N=17408 fused FWHT",
    "c3": "C3 HQ4_G32 prefill GEMM M=4096 K=5120 N=5120",
    "c4_decode": "C4 MoE decode T=1 E=128 top-8 H=2048 I=768",
    "c4_prefill": "C4 MoE prefill T=2048 E=128 top-8 H=2048 I=768",
    "c5_qkv": "C5 verify GEMM HQ8_G32 K=5120 N=7168",
    "c5_down": "C5 verify GEMM HQ4_G64 K=17408 N=5120",
    "mlp_gate_up": "dense MLP gate|up GEMV + SwiGLU + FWHT, HQ4_G32 M=1 K=5120 I=17408",
    "mlp_prefill": "dense MLP prefill gate|up GEMM + SwiGLU + FWHT fused, HQ4_G32 M=4096 K=5120 I=17408",
    "mlp_decode": "dense MLP decode step: gate|up GEMV + SwiGLU, down GEMV, HQ4_G32 M=1 H=5120 I=17408",
    "head": "LM head GEMV + argmax, HQ4_G32 M=1 K=5120 N=151936",
    "f32_decode": "f32-activation GEMV, HQ4_G32 M=1 K=5120 N=17408",
    "f32_verify4": "f32-activation GEMV, HQ4_G32 M=4 K=5120 N=17408",
    "f32_batched64": "f32-activation batched GEMM, HQ4_G32 M=64 K=5120 N=17408",
    "repack": "MLX affine -> AQ4_G64 repack, 34816 x 5120",
    "norm_prefill": "RMSNorm + residual + FWHT producer, 4096 rows x 5120",
    "norm_decode": "RMSNorm + residual + FWHT producer, 1 row x 5120",
    "dense_f32_ba": "dense f32 GEMV (qwg_f32_gemv), 1 row, N=64 K=2048",
    "dense_f32_square": "dense f32 GEMV (qwg_f32_gemv), 1 row, N=5120 K=5120",
}


def main() -> None:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS) + ["headline", "calib", "vendor_gemm"],
                    help="headline = c2 (the bench line) with the c3 prefill GEMM summarised under 'prefill_gemm'")
    ap.add_argument("--m", type=int, default=8, help="activation rows for the c5 workloads")
    ap.add_argument("--hot", action="store_true", help="single bank (Infinity-Cache resident) instead of the cold ring")
    ap.add_argument("--ring-mb", type=float, default=640.0)
    ap.add_argument("--variant", type=int, default=0, help="gemv kernel override (0 auto; 1..7 as the flags of qwhip_gemv)")
    ap.add_argument("--rt", type=int, default=0, help="row tiles per wave for the mfma gemv (0 auto)")
    ap.add_argument("--cfg", type=int, default=0, help="gemm tile shape override (0 auto)")
    ap.add_argument("--moe-tokens", type=int, default=0, help="tokens of a c4 workload when run by itself (0 = the benchmark's 1 / 2048)")
    ap.add_argument("--moe-shared", type=int, default=0, help="c4_decode with several tokens: how many of a token's routes repeat token 0's experts (0..8)")
    ap.add_argument("--moe-reuse", action="store_true",
                    help="c4_decode with 2..4 tokens: QWHIP_MOE_REUSE_EXPERTS (one workgroup reads a shared expert for all of its tokens)")
    ap.add_argument("--moe-f16", action="store_true", help="c4_prefill on f16 hidden rows (the reference's own type) instead of bf16")
    ap.add_argument("--gemm-rows", type=int, default=0, help="activation rows of the c3 or mlp_prefill workload when run by itself (0 = the benchmark's 4096)")
    ap.add_argument("--gemm-ws-mb", type=int, default=0,
                    help="workspace handed to qwhip_gemm in MiB (0 = the activation copy only; more lets small row counts split K)")
    ap.add_argument("--plain-out", action="store_true",
                    help="mlp_gate_up: no output rotation (act in the plain basis; the down projection then rotates its input itself)")
    ap.add_argument("--no-vendor", action="store_true", help="headline: leave out the vendor library's plain GEMM beside the C3 figure")
    ap.add_argument("--vendor-gemm", action="store_true",
                    help="c3: also time the vendor library's plain f16 / bf16 GEMM of the same shape (needs PyTorch; a yardstick, not the product)")
    ap.add_argument("--prerot", action="store_true", help="hand the gemv activations already rotated")
    ap.add_argument("--invariant", action="store_true", help="gemv workloads with QWHIP_GEMV_ROW_INVARIANT (every row as in a call of its own)")
    ap.add_argument("--format", default=None,
                    help="container override for the gemv / gemm / pair workloads, e.g. hq3_g32, aq6_g128 (the workload's shape is kept)")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--cpu-rows", type=int, default=1 << 30, help="rows of the bank the CPU baseline runs over (default: all)")
    args = ap.parse_args()
    if args.gpus != 1:
        _fail("bench.py: this build measures one GPU only (every box has one); run with --gpus 1")
    if args.workload == "calib":
        print(json.dumps(run_calibration(args)))
        return
    if args.workload == "vendor_gemm":      # PyTorch only: this process never loads the library
        _, _, n, k, m, _ = WORKLOADS["c3"]
        m = args.gemm_rows or m
        out = {"workload": f"vendor library plain GEMM M={m} K={k} N={n} (f16, bf16)", "vendor_plain_gemm": vendor_plain_gemm(m, n, k)}
        if args.moe_tokens:                 # the C4 layer's two grouped products with every expert at tokens * 8 / 128 rows
            rows = args.moe_tokens * 8 // 128
            out["vendor_plain_bmm"] = {"rows_per_expert": rows, "gate_up_128x[rows,2048]x[1536,2048]^T": vendor_plain_bmm(128, rows, 1536, 2048),
                                       "down_128x[rows,768]x[2048,768]^T": vendor_plain_bmm(128, rows, 2048, 768)}
        print(json.dumps(out))
        return
    if args.workload == "headline":
        kind, fmt, n, k, m, outliers = WORKLOADS["c2"]
        later = []
        out = run_gemv(args, fmt, n, k, m, LABELS["c2"], outliers, measured_traffic("c2"), cpu_later=later)
        gargs = argparse.Namespace(**vars(args))
        gargs.steps, gargs.warmup, gargs.no_cpu = max(50, args.steps // 4), max(5, args.warmup // 2), True
        gargs.vendor_gemm = not args.no_vendor      # the matrix-pipe yardstick beside the C3 figure (a child process, PyTorch only)
        kind, fmt, n, k, m, outliers = WORKLOADS["c3"]
        g = run_gemm(gargs, fmt, n, k, m, LABELS["c3"], measured_traffic("c3"))
        out["prefill_gemm"] = {"value": g["value"], "unit": g["unit"], "ms_per_step": g["ms_per_step"], "steps": g["steps"],
                               "config": g["config"], "roofline": g["roofline"], "normalized_error": g["normalized_error"]}
        for fn in later:
            out["cpu_baseline"] = fn()
        if not args.no_cpu:
            out["cpu_baseline_c1"] = cpu_baseline_c1()
        print(json.dumps(out))
        return
    kind, fmt, n, k, m, outliers = WORKLOADS[args.workload]
    if m is None:
        m = args.m
    label, traffic = LABELS[args.workload], measured_traffic(args.workload)
    if args.format and args.format != fmt:
        from tests import helpers as H
        if kind not in ("gemv", "gemm", "pair", "head") or args.format not in H.FORMATS:
            ap.error(f"--format takes one of {sorted(H.FORMATS)} on a gemv, gemm, pair or head workload")
        fmt, traffic = args.format, None
        label += f" [container {fmt}]"
    if kind == "moe":
        tokens = args.moe_tokens or m
        out = run_moe(args, tokens, LABELS[args.workload] + (f" [tokens {tokens}]" if args.moe_tokens else ""))
    elif kind == "gemv_f32":
        out = run_gemv_f32(args, fmt, n, k, m, LABELS[args.workload])
    elif kind == "mlp_prefill":
        rows_label = f" [rows {args.gemm_rows}]" if args.gemm_rows else ""
        out = run_mlp_prefill(args, n, k, args.gemm_rows or m, LABELS[args.workload] + rows_label)
    elif kind == "mlp_decode":
        out = run_mlp_decode(args, n, k, LABELS[args.workload])
    elif kind == "head":
        out = run_head(args, fmt, n, k, label)
    elif kind == "repack":
        out = run_repack(args, n, k, 4, 64, LABELS[args.workload])
    elif kind == "norm":
        out = run_norm(args, m, n, LABELS[args.workload])
    elif kind == "dense_f32":
        out = run_dense_f32(args, m, n, k, LABELS[args.workload])
    elif kind == "pair":
        rows = args.gemm_rows or m
        out = run_silu_pair(args, fmt, n, k, rows, label + (f" [rows {rows}]" if args.gemm_rows else ""))
    elif kind == "gemm":
        if args.gemm_rows:
            m, traffic = args.gemm_rows, None
            label += f" [rows {m}, workspace {max(m * k * 2, args.gemm_ws_mb << 20) >> 20} MiB]"
        out = run_gemm(args, fmt, n, k, m, label, traffic)
    else:
        out = run_gemv(args, fmt, n, k, m, label + (f" M={m}" if args.workload.startswith("c5") else ""), outliers, traffic)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
