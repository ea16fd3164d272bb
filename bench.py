#!/usr/bin/env python3
"""Benchmark of the blkq4 hot path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--configs C4,C2,...] [--no-cpu]

One "step" is one call of ``blkq4_fp16_gemm_sm80`` on the headline workload (C4: the M=2048 prefill
GEMM); the GEMV (C2) and the other configurations are measured the same way and reported inside the
same JSON line.  Inputs are resident in HBM before the timed region.  HBM-bound configurations rotate
over distinct weight sets whose total size is at least twice the 256 MB Infinity Cache, and the timed
graph visits every set equally often whatever ``--steps`` is.  Every configuration is replayed untimed
until the clocks have settled.  Kernel time comes from HIP events on the launch stream around a captured
graph of back-to-back launches (median of a few such regions); wall time around the same region gives
``value``.  After timing, the output buffer the timed launches wrote and the packed buffers they read are
compared with the oracle (``parity`` in the JSON line; a mismatch makes the exit code 1).  The CPU baseline
is the oracle (quantize, dequantize + fp32-accumulate GEMM, OpenMP) on a bounded sample of the same
workload, reported next to every GPU figure, and is only a baseline.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

METRIC = "blkq4 GEMM TFLOP/s (M=2048) + GEMV HBM GB/s (M=1), as % of MI355X roofline"
PEAK_MFMA_TFLOPS = 2500.0   # fp16 dense MFMA, MI355X published
PEAK_HBM_GBPS = 8000.0      # HBM3E, MI355X published
INFINITY_CACHE_BYTES = 256 << 20

# name: (M, K, N, block_size, has_offsets, bound); blocks run along K except where COLUMN_WISE says otherwise
CONFIGS = {
    "C1": (64, 1024, 1024, 32, True, "mfma"),
    "C2": (1, 4096, 4096, 64, False, "hbm"),
    "C3": (16, 4096, 11008, 32, True, "hbm"),
    "C4": (2048, 4096, 4096, 64, True, "mfma"),
    "C5": (4096, 8192, 28672, 16, True, "mfma"),
    "C4r": (2048, 4096, 4096, 64, True, "mfma"),
    "C2r": (1, 4096, 4096, 64, False, "hbm"),
    "M128": (128, 4096, 4096, 64, True, "hbm"),
    "V128K": (1, 4096, 128256, 64, False, "hbm"),
    "B16": (16, 8192, 28672, 64, True, "hbm"),
    "C4b": (2048, 4096, 4096, 64, True, "mfma"),
    "C2b": (1, 4096, 4096, 64, False, "hbm"),
    "M256": (256, 4096, 4096, 64, True, "mfma"),
    "M512": (512, 4096, 4096, 64, True, "mfma"),
    "M768N11K": (768, 4096, 11008, 64, True, "mfma"),
    "M256K11K": (256, 11008, 4096, 64, True, "mfma"),
}
BF16 = {"C4b", "C2b"}  # through blkq4_bf16_quant_sm80 / blkq4_bf16_gemm_sm80
# every workload is replayed untimed for this long before the timed replays (a few milliseconds after an
# idle gap run at ramping clocks: the figure wanted is the steady state, whatever --steps is)
SETTLE_SECONDS = 0.4
TIMED_REGIONS = 5       # the reported time is the median over this many timed regions of the same graph
TOLERANCE = 1e-2        # max |got - ref| / max(|ref|, 1e-3 max|ref|) against the oracle
COLUMN_WISE = {"C4r": False, "C2r": False}
DESCRIPTION = {
    "C1": "C1 CPU-runnable case M=64 K=1024 N=1024 bs32 asym",
    "C2": "C2 decode GEMV M=1 K=4096 N=4096 bs64 sym",
    "C3": "C3 skinny GEMM M=16 K=4096 N=11008 bs32 asym",
    "C4": "C4 prefill GEMM M=2048 K=4096 N=4096 bs64 asym",
    "C5": "C5 large-layer GEMM M=4096 K=8192 N=28672 bs16 asym",
    "C4r": "C4 shape with blocks along N (column_wise_blocking=false) M=2048 K=4096 N=4096 bs64 asym",
    "C2r": "C2 shape with blocks along N (column_wise_blocking=false) M=1 K=4096 N=4096 bs64 sym",
    "M128": "mid-size batch M=128 K=4096 N=4096 bs64 asym (streaming kernel in four row groups)",
    "V128K": "vocabulary projection GEMV M=1 K=4096 N=128256 bs64 sym (waves with a column tile of their own)",
    "B16": "batch-16 decode on a wide layer M=16 K=8192 N=28672 bs64 asym (rows staged per slice)",
    "C4b": "C4 shape in bf16 (blkq4_bf16_gemm_sm80) M=2048 K=4096 N=4096 bs64 asym",
    "C2b": "C2 shape in bf16 (blkq4_bf16_gemm_sm80) M=1 K=4096 N=4096 bs64 sym",
    "M256": "mid-size batch M=256 K=4096 N=4096 bs64 asym",
    "M512": "mid-size batch M=512 K=4096 N=4096 bs64 asym",
    "M768N11K": "ragged tile grid M=768 K=4096 N=11008 bs64 asym",
    "M256K11K": "mid-size batch on a down projection M=256 K=11008 N=4096 bs64 asym (split tiles)",
}


# HBM-side traffic per launch, measured with `rocprofv3 --pmc FETCH_SIZE` and `--pmc WRITE_SIZE` (two runs of
# this script, KiB per dispatch, mean over the dispatches of the kernel) and scaled by what the same counter
# reads for the runtime's device-to-device copy of a 128 MiB buffer in the same run (FETCH_SIZE reads
# 65 552 KiB for 131 072 KiB fetched: factor 2.0; WRITE_SIZE reads 131 072 KiB: factor 1.0).  The counters
# sit between L2 and the memory fabric, so reads served by the Infinity Cache are included.  A script cannot
# read these counters for itself; the figures are refreshed when a kernel changes, and `traffic_kernel` in the
# figure of a workload is reported only while the library still picks the kernel it was taken from (TRAFFIC_KERNEL).
COUNTER_SCALE = {"FETCH_SIZE": 131072.0 / 65552.0, "WRITE_SIZE": 1.0}
COUNTER_KIB = {  # name: (FETCH_SIZE, WRITE_SIZE)
    "C4": (34411.6, 16388.8),
    "C2": (4406.1, 8.0),
    "C3": (13653.7, 344.0),
    "C5": (860380.2, 229382.3),
    "C5_prepack": (229410.8, 157706.9),
    "C4r": (34415.1, 16386.6),
    "C2r": (4428.1, 8.0),
    "C1": (869.0, 128.0),
    "M128": (8649.1, 1024.0),
    "M256": (14387.1, 2048.0),
    "M512": (17233.5, 4183.2),
    "M768N11K": (60863.0, 16513.7),
    "M256K11K": (43374.1, 19434.3),
    "V128K": (136348.8, 250.8),
    "B16": (64097.7, 896.0),
    "C4b": (34440.5, 16387.2),
    "C2b": (4418.6, 8.0),
}


TRAFFIC_KERNEL = {  # what blkq4_gemm_plan_sm80 said the workload runs when its counters were taken
    "C1": "streaming: 8 waves splitting K, 1 column tile(s) x 32 rows, 2 slices in flight, rows whole in LDS, 2 row group(s), 128 workgroups",
    "C2": "decode: 8 waves splitting K, 4 slices requested by each, 1 column tile(s) x 1 row(s), 256 workgroups",
    "C3": "decode: 8 waves splitting K, 4 slices requested by each, 3 column tile(s) x 16 row(s), 230 workgroups",
    "C4": "tile: 128 x 256, 4 + 4 waves, 256 tiles, blocks of 4 x 8 tiles per XCD",
    "C5": "tile: 256 x 256, 4 + 0 waves, 1792 tiles",
    "C4r": "tile: 128 x 256, 4 + 4 waves, 256 tiles, blocks of 4 x 8 tiles per XCD",
    "C2r": "decode (blocks along N): 4 waves splitting K, 8 slices requested by each, 1 column tile(s) x 1 row(s), 256 workgroups",
    "M128": "streaming: 8 waves splitting K, 4 column tile(s) x 32 rows, 2 slices in flight, rows staged per slice, 4 row group(s), 256 workgroups",
    "V128K": "decode: 8 waves splitting K, 4 slices requested by each, 2 column tile(s) x 1 row(s), 4008 workgroups",
    "B16": "streaming: 8 waves splitting K, 7 column tile(s) x 16 rows, 2 slices in flight, rows staged per slice, 1 row group(s), 256 workgroups",
    "C4b": "tile: 128 x 256, 4 + 4 waves, 256 tiles, blocks of 4 x 8 tiles per XCD",
    "C2b": "decode: 8 waves splitting K, 4 slices requested by each, 1 column tile(s) x 1 row(s), 256 workgroups",
    "M256": "tile: 128 x 32, 4 + 4 waves (the computing waves split the k tile), 256 tiles",
    "M512": "tile: 64 x 128, 4 + 4 waves, 256 tiles, blocks of 4 x 8 tiles per XCD",
    "M768N11K": "tile: 256 x 256, 4 + 0 waves, 129 tiles",
    "M256K11K": "tile: 128 x 128, 4 + 4 waves, 64 tiles, the last 64 in 4 parts (workspace 16793600 bytes)",
}


def traffic_bytes(name, kernel=None):
    """HBM-side bytes per launch, or None when there is no figure or it was taken from another kernel."""
    if name not in COUNTER_KIB or (name in TRAFFIC_KERNEL and kernel is not None and TRAFFIC_KERNEL[name] != kernel):
        return None
    f, w = COUNTER_KIB[name]
    return int(round((f * COUNTER_SCALE["FETCH_SIZE"] + w * COUNTER_SCALE["WRITE_SIZE"]) * 1024))


def algorithmic(m, k, n, bs, has_offsets):
    """FLOPs and bytes of one GEMM call: A + packed W + scales + zero-points (uint8) + C."""
    flops = 2 * m * n * k
    nbytes = 2 * m * k + k * n // 2 + 2 * k * n // bs + (k * n // bs if has_offsets else 0) + 2 * m * n
    return flops, nbytes


def prepack_bytes(k, n, bs, has_offsets):
    return 2 * k * n + k * n // 2 + 2 * k * n // bs + (k * n // bs if has_offsets else 0)


def timed_region(torch, launches, steps, warmup, settle_seconds=SETTLE_SECONDS, regions=TIMED_REGIONS):
    """launches: list of zero-argument callables that each enqueue ONE kernel on the current stream;
    call i uses launches[i % len].  A region is `steps` back-to-back launches (one graph replay), bracketed by
    synchronize on both sides; the median over `regions` regions is returned as
    (wall seconds, event seconds, 'graph'|'eager')."""
    nl = len(launches)
    for i in range(warmup):
        launches[i % nl]()
    torch.cuda.synchronize()
    mode = "graph"
    graph = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=side):
                for i in range(steps):
                    launches[i % nl]()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph.replay()  # untimed: first replay uploads the graph
        torch.cuda.synchronize()
    except Exception as e:  # pragma: no cover - depends on the runtime
        sys.stderr.write(f"[bench] graph capture unavailable ({type(e).__name__}: {e}); timing eager launches\n")
        graph = None
        mode = "eager"
        torch.cuda.synchronize()

    def region():
        if graph is not None:
            graph.replay()
        else:
            for i in range(steps):
                launches[i % nl]()

    t_settle = time.perf_counter()
    while time.perf_counter() - t_settle < settle_seconds:
        for _ in range(4):
            region()
        torch.cuda.synchronize()
    walls, evts = [], []
    for _ in range(regions):
        ev0 = torch.cuda.Event(enable_timing=True)
        ev1 = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record()
        region()
        ev1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        walls.append(t1 - t0)
        evts.append(ev0.elapsed_time(ev1) * 1e-3)
    walls.sort()
    evts.sort()
    return walls[len(walls) // 2], evts[len(evts) // 2], mode


def np_view(t):
    """device or host tensor (fp16 / bf16 / uint8) -> numpy array of the same bits (fp16 as float16, bf16 as uint16)."""
    import numpy as np
    import torch
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float16:
        return t.view(torch.int16).numpy().view(np.float16)
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def make_problem(torch, capi, name, device, copies):
    """Inputs of one workload, resident on the device.  The LAST weight set comes from the seeded CPU generator
    (its fp16 source is kept on the host for the oracle); the sets before it are drawn on the device."""
    m, k, n, bs, has_offsets, _ = CONFIGS[name]
    col = COLUMN_WISE.get(name, True)
    bf = name in BF16
    dtype = torch.bfloat16 if bf else torch.float16
    g = torch.Generator(device="cpu").manual_seed(1234 + list(CONFIGS).index(name))
    a = torch.randn(m, k, generator=g, dtype=torch.float32).to(dtype).to(device)
    w_host = (torch.randn(n, k, generator=g, dtype=torch.float32) * 0.02).to(dtype)
    gd = torch.Generator(device=device).manual_seed(99 + list(CONFIGS).index(name))
    w_elems, meta_elems = capi.quant_size(bs, col, k, n)
    sets = []
    for c in range(copies):
        if c == copies - 1:
            w = w_host.to(device)
        else:
            w = (torch.randn(n, k, generator=gd, dtype=torch.float32, device=device) * 0.02).to(dtype)
        q_w = torch.empty(w_elems, dtype=torch.uint8, device=device)
        q_s = torch.empty(meta_elems, dtype=dtype, device=device)
        q_zp = torch.empty(meta_elems, dtype=torch.uint8, device=device) if has_offsets else None
        capi.quant(bs, col, w, q_w, q_s, q_zp, bf16=bf)
        sets.append((q_w, q_s, q_zp))
        del w
    torch.cuda.synchronize()
    out = torch.full((m, n), float("nan"), dtype=dtype, device=device)
    return a, sets, out, w_host


def check_and_baseline(name, a_dev, last_set, out_dev, w_host, with_cpu=True):
    """Parity gate and CPU baseline of one workload, both from the oracle on the host.

    Parity: the packed weights, scales and zero-points the timed launches read (the last weight set) against the
    oracle's quantizer, byte for byte; the output buffer the last timed launch wrote against the oracle's
    dequantize + GEMM (every row up to 64 rows, else a spread sample of rows).
    CPU baseline: the same oracle calls, timed: dequantize (whole B) + GEMM over a bounded number of rows."""
    import numpy as np
    from oracle import blkq4_oracle as O
    m, k, n, bs, has_offsets, bound = CONFIGS[name]
    col = COLUMN_WISE.get(name, True)
    bf = name in BF16
    w = np_view(w_host)
    a = np_view(a_dev)
    t0 = time.perf_counter()
    canon, s, z = O.quantize(bs, col, w, has_offsets, bf16=bf)
    t_quant = time.perf_counter() - t0
    ps, pz = O.prepack_meta_sm80(bs, col, k, n, s.view(np.float16) if bf else s, z)
    q_w, q_s, q_zp = last_set
    prepack_ok = bool(np.array_equal(np_view(q_w), O.native_from_canonical(canon).reshape(-1))
                      and np.array_equal(np_view(q_s).view(np.uint16).reshape(-1), ps.view(np.uint16).reshape(-1))
                      and (q_zp is None or np.array_equal(np_view(q_zp).reshape(-1), pz.reshape(-1))))
    t0 = time.perf_counter()
    b = O.dequantize(bs, col, canon, s, z, bf16=bf)
    t_deq = time.perf_counter() - t0
    if m <= 64:
        rows = np.arange(m)
    else:
        want = m if m * n * k <= (1 << 35) else 64 if m * n * k <= (1 << 37) else 12
        rows = np.unique(np.concatenate([np.linspace(0, m - 1, want).astype(np.int64), [0, m - 1]]))
    a_rows = np.ascontiguousarray(a[rows])
    t0 = time.perf_counter()
    ref = O.gemm(a_rows, b, bf16=bf)
    t_gemm = time.perf_counter() - t0
    got = np_view(out_dev)[rows]
    if bf:
        got, ref = O.bf16_to_f32(got), O.bf16_to_f32(ref)
    g64, r64 = got.astype(np.float64), ref.astype(np.float64)
    floor = 1e-3 * float(np.max(np.abs(r64))) + 1e-30
    err = float(np.max(np.abs(g64 - r64) / np.maximum(np.abs(r64), floor))) if np.all(np.isfinite(g64)) else float("inf")
    parity = {"prepack_bit_exact": prepack_ok, "gemm_max_rel_err": float(f"{err:.3e}"), "rows_checked": int(len(rows)),
              "of_rows": m, "ok": bool(prepack_ok and err <= TOLERANCE)}
    base = None
    if with_cpu:
        flops, nbytes = algorithmic(m, k, n, bs, has_offsets)
        # GEMM time for the whole workload, from the rows just computed (a second, larger sample for the big ones
        # would add minutes; the oracle's GEMM time is linear in the rows)
        t_whole = t_deq + t_gemm * m / len(rows)
        if bound == "mfma":
            value, unit = flops / t_whole / 1e12, "TFLOP/s"
        else:
            value, unit = nbytes / t_whole / 1e9, "GB/s"
        base = {"value": float(f"{value:.4g}"), "unit": unit, "cores": O.num_threads(), "kind": "port",
                "sample": f"oracle dequantize of the whole B {t_deq:.3f}s + GEMM of {len(rows)} of {m} rows {t_gemm:.3f}s "
                          f"(scaled to {m} rows); oracle quantize of B {t_quant:.3f}s = "
                          f"{prepack_bytes(k, n, bs, has_offsets) / t_quant / 1e9:.2f} GB/s"}
    return parity, base, t_quant


def bench_gemm(torch, capi, name, device, steps, warmup, with_cpu=True):
    m, k, n, bs, has_offsets, bound = CONFIGS[name]
    flops, nbytes = algorithmic(m, k, n, bs, has_offsets)
    copies = 1
    per_set = nbytes - 2 * m * k - 2 * m * n
    if bound == "hbm":
        copies = 2 * INFINITY_CACHE_BYTES // per_set + 1
    a, sets, out, w_host = make_problem(torch, capi, name, device, copies)
    col = COLUMN_WISE.get(name, True)

    def mk(s):
        q_w, q_s, q_zp = s
        return lambda: capi.gemm(bs, col, m, n, k, a, q_w, q_s, q_zp, out, bf16=name in BF16)

    launches = [mk(s) for s in sets]
    kernel = capi.gemm_plan(bs, col, m, n, k, has_offsets, name in BF16)[2]
    # every weight set is visited equally often, and the last launch reads the last (seeded) set
    n_launch = copies * ((max(steps, copies) + copies - 1) // copies)
    wall, evt, mode = timed_region(torch, launches, n_launch, warmup)
    per_call_wall = wall / n_launch
    per_call_evt = evt / n_launch
    if bound == "mfma":
        achieved, peak, unit = flops / per_call_evt / 1e12, PEAK_MFMA_TFLOPS, "TFLOP/s"
        value = flops / per_call_wall / 1e12
    else:
        achieved, peak, unit = nbytes / per_call_evt / 1e9, PEAK_HBM_GBPS, "GB/s"
        value = nbytes / per_call_wall / 1e9
    res = {
        "workload": DESCRIPTION[name], "value": round(value, 3), "unit": unit,
        "ms_per_step": round(per_call_wall * 1e3, 6), "kernel_us": round(per_call_evt * 1e6, 3),
        "kernel": kernel,
        "timing": mode, "launches_per_region": n_launch, "weight_sets": copies,
        "weight_footprint_bytes": copies * per_set, "flops": flops, "bytes": nbytes,
        "tflops": round(flops / per_call_evt / 1e12, 3), "gbps": round(nbytes / per_call_evt / 1e9, 3),
        "roofline": {"bound": bound, "achieved": round(achieved, 3), "peak": peak, "unit": unit,
                     "frac": round(achieved / peak, 4), "traffic": traffic_bytes(name, kernel)},
    }
    torch.cuda.synchronize()
    parity, base, _ = check_and_baseline(name, a, sets[-1], out, w_host, with_cpu)
    res["parity"] = parity
    if base is not None:
        res["cpu_baseline"] = base
    return res, (a, sets, out, w_host)


def bench_prepack(torch, capi, device, steps, warmup, with_cpu=True):
    import numpy as np
    _, k, n, bs, has_offsets, _ = CONFIGS["C5"]
    nbytes = prepack_bytes(k, n, bs, has_offsets)
    g = torch.Generator(device="cpu").manual_seed(4321)
    w_host = (torch.randn(n, k, generator=g, dtype=torch.float32) * 0.02).to(torch.float16)
    w = w_host.to(device)
    w_elems, meta_elems = capi.quant_size(bs, True, k, n)
    q_w = torch.full((w_elems,), 0xA5, dtype=torch.uint8, device=device)
    q_s = torch.full((meta_elems,), float("nan"), dtype=torch.float16, device=device)
    q_zp = torch.full((meta_elems,), 0xEE, dtype=torch.uint8, device=device)
    launches = [lambda: capi.quant(bs, True, w, q_w, q_s, q_zp)]
    steps = max(10, steps // 10)
    wall, evt, mode = timed_region(torch, launches, steps, max(2, warmup // 10))
    per = evt / steps
    ach = nbytes / per / 1e9
    # the same bytes moved the same way with no arithmetic (the probe library's twin of the kernel), same run
    import ctypes
    import bench_probe
    probe = ctypes.CDLL(bench_probe.build())
    vp = ctypes.c_void_p
    probe.blkq4_probe_prepack_traffic.argtypes = [vp, ctypes.c_int, ctypes.c_int, ctypes.c_int, vp, vp, vp, vp]
    t_w, t_s, t_z = torch.empty_like(q_w), torch.empty_like(q_s), torch.empty_like(q_zp)
    twin = [lambda: probe.blkq4_probe_prepack_traffic(w.data_ptr(), k, n, k, t_w.data_ptr(), t_s.data_ptr(), t_z.data_ptr(),
                                                     vp(torch.cuda.current_stream().cuda_stream))]
    _, twin_evt, _ = timed_region(torch, twin, steps, max(2, warmup // 10))
    del t_w, t_s, t_z
    res = {
        "workload": "C5 quantize+prepack K=8192 N=28672 bs16 asym", "value": round(nbytes / (wall / steps) / 1e9, 3),
        "unit": "GB/s", "ms_per_step": round(wall / steps * 1e3, 6), "kernel_us": round(per * 1e6, 3), "timing": mode,
        "launches_per_region": steps, "bytes": nbytes, "gbps": round(ach, 3),
        "traffic_only_twin_us": round(twin_evt / steps * 1e6, 3),
        "roofline": {"bound": "hbm", "achieved": round(ach, 3), "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                     "frac": round(ach / PEAK_HBM_GBPS, 4), "traffic": traffic_bytes("C5_prepack")},
    }
    # parity: every byte the timed launches wrote, against the oracle's quantizer (timed: the CPU baseline)
    from oracle import blkq4_oracle as O
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    canon, s, z = O.quantize(bs, True, np_view(w_host), has_offsets)
    t_quant = time.perf_counter() - t0
    ps, pz = O.prepack_meta_sm80(bs, True, k, n, s, z)
    ok = bool(np.array_equal(np_view(q_w), O.native_from_canonical(canon).reshape(-1))
              and np.array_equal(np_view(q_s).view(np.uint16), ps.view(np.uint16).reshape(-1))
              and np.array_equal(np_view(q_zp), pz.reshape(-1)))
    res["parity"] = {"prepack_bit_exact": ok, "bytes_checked": int(q_w.numel() + 2 * q_s.numel() + q_zp.numel()), "ok": ok}
    if with_cpu:
        res["cpu_baseline"] = {"value": float(f"{nbytes / t_quant / 1e9:.4g}"), "unit": "GB/s", "cores": O.num_threads(),
                               "kind": "port", "sample": f"oracle quantize of the whole B (one run) {t_quant:.3f}s"}
    return res


def bench_copy(torch, capi, device, steps, warmup):
    """A plain copy of known size (the library's layout conversion of a packed weight buffer reads
    every byte once and writes every byte once): the reference that hardware traffic counters are
    scaled by.  Not part of the default run."""
    rows, cols = 16384, 16384
    nbytes = rows * cols // 2
    src = torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=device)
    dst = torch.empty_like(src)
    launches = [lambda: capi.repack(True, rows, cols, src, dst)]
    steps = max(10, steps // 10)
    for _ in range(steps):  # the runtime's own device-to-device copy of the same buffer, as a second reference
        dst.copy_(src)
    wall, evt, mode = timed_region(torch, launches, steps, max(2, warmup // 10))
    per = evt / steps
    ach = 2 * nbytes / per / 1e9
    return {
        "workload": "copy reference: repack of a 16384x16384 packed buffer (128 MiB read + 128 MiB written)",
        "value": round(ach, 3), "unit": "GB/s", "ms_per_step": round(wall / steps * 1e3, 6),
        "kernel_us": round(per * 1e6, 3), "timing": mode, "bytes": 2 * nbytes, "read_bytes": nbytes,
        "write_bytes": nbytes,
    }


GEMV_FORM_SHAPES = [(1, 4096, 4096, 64, False), (1, 4096, 4096, 64, True), (2, 4096, 4096, 64, False), (4, 4096, 4096, 64, False),
                    (1, 2048, 2048, 64, False), (1, 2048, 8192, 64, False), (1, 4096, 11008, 32, True), (1, 8192, 4096, 64, False),
                    (1, 11008, 4096, 64, False), (1, 14336, 4096, 64, False), (1, 8192, 8192, 64, False), (1, 8192, 28672, 64, False),
                    (1, 4096, 128256, 64, False), (4, 4096, 14336, 64, True)]


def bench_gemv_forms(torch, capi, device, shapes, steps):
    """The two forms of the GEMV on the same data in the same process: the one blkq4_fp16_gemm_sm80 picks (MFMA:
    every wave converts its weights and feeds v_mfma_f32_16x16x32_f16) and blkq4_fp16_gemv_valu_sm80 (no MFMA:
    per-lane fp32 partial sums with v_dot2_f32_f16, lane exchanges across K).  shapes: (M, K, N, block size,
    zero-points).  Weight sets rotate over twice the Infinity Cache."""
    rows = []
    for m, k, n, bs, zp in shapes:
        per_set = k * n // 2 + 2 * k * n // bs + (k * n // bs if zp else 0)
        copies = min(64, 2 * INFINITY_CACHE_BYTES // per_set + 1)
        g = torch.Generator(device=device).manual_seed(7)
        a = torch.randn(m, k, generator=g, device=device).to(torch.float16)
        w_elems, meta = capi.quant_size(bs, True, k, n)
        sets = []
        for _ in range(copies):
            w = (torch.randn(n, k, generator=g, device=device) * 0.02).to(torch.float16)
            q_w = torch.empty(w_elems, dtype=torch.uint8, device=device)
            q_s = torch.empty(meta, dtype=torch.float16, device=device)
            q_z = torch.empty(meta, dtype=torch.uint8, device=device) if zp else None
            capi.quant(bs, True, w, q_w, q_s, q_z)
            sets.append((q_w, q_s, q_z))
            del w
        out = torch.empty(m, n, dtype=torch.float16, device=device)
        n_launch = copies * ((max(steps, copies) + copies - 1) // copies)
        row = {"shape": f"M={m} K={k} N={n} bs{bs} {'asym' if zp else 'sym'}", "weight_sets": copies}
        for key, valu in (("mfma_us", False), ("valu_us", True)):
            launches = [(lambda s=s: capi.gemm(bs, True, m, n, k, a, s[0], s[1], s[2], out, valu=valu)) for s in sets]
            _, evt, _ = timed_region(torch, launches, n_launch, 5, settle_seconds=0.2)
            row[key] = round(evt / n_launch * 1e6, 3)
        rows.append(row)
        del sets
        torch.cuda.empty_cache()
    return rows


def bench_context(torch, capi, device, head_problem, steps, warmup):
    """Figures the headline numbers are read against, measured in the same run:
    * what a graph node costs when its kernel does nothing, and what a kernel costs that issues the GEMV's
      memory requests and nothing else (the probe library built next to the product library);
    * the vendor library's plain fp16 GEMM (torch.matmul on an fp16 copy of the dequantized-size weight
      matrix, no 4-bit weights involved) on the headline shape;
    * the headline GEMM on all-zero activations and weights: same instruction stream, idle data paths --
      the difference to the real run is what the clock loses under load;
    * a kernel that does nothing but back-to-back fp16 MFMAs (one wave per SIMD, all 256 compute units) on
      random and on all-zero operands: the rate the chip sustains, which is the ceiling of any fp16 GEMM."""
    import ctypes
    import bench_probe
    out = {}
    probe = ctypes.CDLL(bench_probe.build())
    probe.blkq4_probe_empty.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    probe.blkq4_probe_stream.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_void_p, ctypes.c_void_p]
    scratch = torch.zeros(1 << 16, dtype=torch.int32, device=device)
    steps = max(steps, 100)  # the floors are small numbers: at least 100 launches per region
    probe.blkq4_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]

    def stream_ptr():
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    wall, evt, _ = timed_region(torch, [lambda: probe.blkq4_probe_empty(scratch.data_ptr(), stream_ptr())], steps, warmup)
    out["empty_kernel_us"] = round(evt / steps * 1e6, 3)
    mfma_iters = 4000  # about 2 ms of MFMAs per launch, long enough for the clock to settle
    for random_operands, key in ((1, "mfma_only_random_operands_tflops"), (0, "mfma_only_zero_operands_tflops")):
        n_launch = 20
        wall, evt, _ = timed_region(
            torch, [lambda: probe.blkq4_probe_mfma(random_operands, mfma_iters, scratch.data_ptr(), stream_ptr())],
            n_launch, 3, settle_seconds=0.2, regions=3)
        out[key] = round(256 * 4 * mfma_iters * 8 * 32768.0 / (evt / n_launch) / 1e12, 1)
    m, k, n, bs, has_offsets, _ = CONFIGS["C2"]
    per_set = k * n // 2 + 2 * k * n // bs
    copies = 2 * INFINITY_CACHE_BYTES // per_set + 1
    floor_launches = copies * ((max(steps, copies) + copies - 1) // copies)
    ws = [torch.randint(0, 256, (k * n // 2,), dtype=torch.uint8, device=device) for _ in range(copies)]
    ss = [torch.ones(k // bs * n, dtype=torch.float16, device=device) for _ in range(copies)]
    for with_scales in (False, True):
        launches = [(lambda w=w, sc=sc: probe.blkq4_probe_stream(w.data_ptr(), sc.data_ptr() if with_scales else None,
                                                                 n, k, scratch.data_ptr(), stream_ptr()))
                    for w, sc in zip(ws, ss)]
        wall, evt, _ = timed_region(torch, launches, floor_launches, warmup)
        out["c2_requests_only_us" if with_scales else "c2_weight_requests_only_us"] = round(evt / floor_launches * 1e6, 3)
    # the same bytes requested the way the decode kernel requests them (eight waves, four slices each, at once)
    probe.blkq4_probe_decode_requests.argtypes = probe.blkq4_probe_stream.argtypes
    launches = [(lambda w=w, sc=sc: probe.blkq4_probe_decode_requests(w.data_ptr(), sc.data_ptr(), n, k, scratch.data_ptr(), stream_ptr()))
                for w, sc in zip(ws, ss)]
    wall, evt, _ = timed_region(torch, launches, floor_launches, warmup)
    out["c2_decode_requests_only_us"] = round(evt / floor_launches * 1e6, 3)
    del ws, ss
    out["gemv_forms_c2_shape"] = bench_gemv_forms(torch, capi, device, [(1, 4096, 4096, 64, False)], steps)[0]
    if head_problem is not None:
        a, sets, c, w_host = head_problem
        m, k, n, bs, has_offsets, _ = CONFIGS["C4"]
        b = (torch.randn(n, k, device=device, dtype=torch.float32) * 0.02).to(torch.float16).t()
        wall, evt, _ = timed_region(torch, [lambda: torch.matmul(a, b)], steps, warmup)
        out["library_fp16_gemm_c4_shape"] = {"us": round(evt / steps * 1e6, 3),
                                             "tflops": round(2.0 * m * n * k / (evt / steps) / 1e12, 3)}
        del b
        m5, k5, n5 = CONFIGS["C5"][:3]
        a5 = torch.randn(m5, k5, device=device, dtype=torch.float32).to(torch.float16)
        b5 = (torch.randn(n5, k5, device=device, dtype=torch.float16) * 0.02).t()
        wall, evt, _ = timed_region(torch, [lambda: torch.matmul(a5, b5)], max(10, steps // 10), max(2, warmup // 10))
        per = evt / max(10, steps // 10)
        out["library_fp16_gemm_c5_shape"] = {"us": round(per * 1e6, 3), "tflops": round(2.0 * m5 * n5 * k5 / per / 1e12, 3)}
        del a5, b5
        q_w, q_s, q_zp = sets[0]
        za, zw, zs, zz = torch.zeros_like(a), torch.zeros_like(q_w), torch.zeros_like(q_s), torch.zeros_like(q_zp)
        wall, evt, _ = timed_region(torch, [lambda: capi.gemm(bs, True, m, n, k, za, zw, zs, zz, c)], steps, warmup)
        out["c4_all_zero_data_us"] = round(evt / steps * 1e6, 3)
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--configs", default="C4,C2,C1,C3,C5,prepack,C4r,C2r,M128,M256,M512,M768N11K,M256K11K,V128K,B16,C4b,C2b")
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--no-context", action="store_true", help="skip the floors and the library comparison")
    ap.add_argument("--settle", type=float, default=None,
                    help="seconds of untimed replay before the timed regions (default 0.4; profiling runs use less)")
    ap.add_argument("--gemv-forms", action="store_true",
                    help="only the A/B of the two forms of the GEMV (MFMA / no MFMA) over a list of shapes")
    args = ap.parse_args(argv)
    if args.settle is not None:
        global SETTLE_SECONDS
        SETTLE_SECONDS = args.settle
        timed_region.__defaults__ = (SETTLE_SECONDS, TIMED_REGIONS)
    if args.gpus != 1:
        print("bench.py measures one GPU: this path has no multi-GPU part (run with --gpus 1)", file=sys.stderr)
        return 2

    import torch
    from gemmlib_amd import capi
    capi.load()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    if args.gemv_forms:
        print(json.dumps({"gemv_forms": bench_gemv_forms(torch, capi, device, GEMV_FORM_SHAPES, max(args.steps, 100))}))
        return 0
    wanted = [c.strip() for c in args.configs.split(",") if c.strip()]
    with_cpu = not args.no_cpu
    results = {}
    head = None
    head_problem = None
    for name in wanted:
        sys.stderr.write(f"[bench] {name}\n")
        sys.stderr.flush()
        if name == "prepack":
            results["C5_prepack"] = bench_prepack(torch, capi, device, args.steps, args.warmup, with_cpu)
        elif name == "copy":
            results["copy"] = bench_copy(torch, capi, device, args.steps, args.warmup)
        else:
            res, problem = bench_gemm(torch, capi, name, device, args.steps, args.warmup, with_cpu)
            results[name] = res
            if name == "C4":
                head, head_problem = res, problem
            else:
                del problem
        torch.cuda.empty_cache()
    if head is None:  # headline not requested: report the first one measured
        head = next(iter(results.values()))

    checked = {k: v["parity"] for k, v in results.items() if "parity" in v}
    parity_ok = all(v["ok"] for v in checked.values())
    line = {
        "metric": METRIC, "value": head["value"], "unit": head["unit"], "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": head["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": head["workload"], "timing": head.get("timing"),
                   "launches_per_timed_region": head.get("launches_per_region"), "timed_regions": TIMED_REGIONS,
                   "settle_seconds": SETTLE_SECONDS},
        "roofline": head["roofline"],
        "parity": {"ok": parity_ok, "tolerance": TOLERANCE,
                   "metric": "max |got - ref| / max(|ref|, 1e-3 max|ref|) against the oracle; prepack byte for byte",
                   "checked": checked},
    }
    if "cpu_baseline" in head:
        line["cpu_baseline"] = dict(head["cpu_baseline"])
    # The metric has two halves (the M=2048 GEMM and the M=1 GEMV) and the configurations beside them: the
    # objects a reader of this line is sure to keep whole carry all of them, compactly.
    line["roofline"] = dict(head["roofline"])
    line["roofline"]["kernel_us"] = head.get("kernel_us")
    by_workload = {}
    for key, res in results.items():
        r = res.get("roofline")
        if r is not None and key != "copy":
            by_workload[key] = {"bound": r["bound"], "frac": r["frac"], "kernel_us": res["kernel_us"]}
            if "traffic_only_twin_us" in res:
                by_workload[key]["traffic_only_twin_us"] = res["traffic_only_twin_us"]
    line["roofline"]["by_workload"] = by_workload
    if "C2" in results:
        c2 = results["C2"]
        line["gemv"] = {"workload": c2["workload"], "value": c2["value"], "unit": "GB/s",
                        "kernel_us": c2["kernel_us"], "roofline": c2["roofline"], "weight_sets": c2["weight_sets"],
                        "weight_footprint_bytes": c2["weight_footprint_bytes"],
                        "launches_per_timed_region": c2["launches_per_region"]}
        if "cpu_baseline" in c2:
            line["gemv"]["cpu_baseline"] = c2["cpu_baseline"]
        line["roofline"]["gemv"] = {"workload": c2["workload"], "bound": "hbm", "achieved": c2["roofline"]["achieved"],
                                    "peak": PEAK_HBM_GBPS, "unit": "GB/s", "frac": c2["roofline"]["frac"],
                                    "kernel_us": c2["kernel_us"], "traffic": c2["roofline"]["traffic"],
                                    "weight_sets": c2["weight_sets"]}
        if "cpu_baseline" in c2 and "cpu_baseline" in line:
            line["cpu_baseline"]["gemv"] = {k: c2["cpu_baseline"][k] for k in ("value", "unit", "cores", "kind")}
    if not args.no_context:
        sys.stderr.write("[bench] context\n")
        line["context"] = bench_context(torch, capi, device, head_problem, args.steps, args.warmup)
        for key, ctx in (("C4", "library_fp16_gemm_c4_shape"), ("C5", "library_fp16_gemm_c5_shape")):
            if key in by_workload and ctx in line["context"]:
                by_workload[key]["library_fp16_gemm_us"] = line["context"][ctx]["us"]
    # the configurations the metric is defined on go last, so that they are what the end of the output shows
    last = [k for k in ("C1", "C3", "C5_prepack", "C5", "C2", "C4") if k in results]
    line["all"] = {k: results[k] for k in [k for k in results if k not in last] + last}
    print(json.dumps(line))
    if not parity_ok:
        sys.stderr.write("[bench] PARITY FAILED: " + json.dumps({k: v for k, v in checked.items() if not v["ok"]}) + "\n")
        return 1
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
