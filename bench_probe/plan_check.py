"""The cost model's choice against the alternatives, measured: for every shape of a list, the GEMM is timed with the
plan ``blkq4_gemm_plan_sm80`` names ("auto") and with every other plan that exists for it, forced through
``blkq4_gemm_with_plan_sm80``; one JSON line per shape says what was chosen, what was fastest and by how much.

    python -m bench_probe.plan_check [--part i/n] [--quick] [--shapes variant:m:n:k,...] [--every-plan]

The shapes cover what the constants of the model were NOT fitted on: bf16, blocks of 16 and 32, blocks along N, next to
M = 1 ... 512, N = 4096 ... 28672, K = 4096 ... 11008.  Weight sets rotate over more than the Infinity Cache for the
shapes that stream their weights.  Every forced plan's result is compared with the chosen plan's (they differ in the
order of summation only)."""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

INFINITY_CACHE_BYTES = 256 << 20

# (bf16, block size, blocks along K, zero-points)
VARIANTS = {
    "bf16/bs64": (True, 64, True, True),
    "fp16/bs16": (False, 16, True, True),
    "fp16/bs32/sym": (False, 32, True, False),
    "fp16/bs64/along-N": (False, 64, False, True),
}
# the variant the constants were fitted on, for --shapes
FITTED_VARIANTS = {"fp16/bs64": (False, 64, True, True), "fp16/bs64/sym": (False, 64, True, False),
                   # combinations, for --shapes
                   "bf16/bs16": (True, 16, True, True), "bf16/bs64/along-N": (True, 64, False, True),
                   "fp16/bs16/along-N": (False, 16, False, True), "fp16/bs32": (False, 32, True, True)}
LAYERS = [(4096, 4096), (11008, 4096), (4096, 11008), (28672, 8192), (14336, 4096)]   # (N, K)
ROWS = [1, 4, 8, 16, 32, 64, 128, 256, 512]


def shapes():
    """About forty (variant, M, N, K): the variants dealt round robin over rows x layers."""
    out = []
    names = list(VARIANTS)
    i = 0
    for n, k in LAYERS:
        for m in ROWS:
            if (n, k) == (14336, 4096) and m not in (1, 16, 128, 512):
                continue
            out.append((names[i % len(names)], m, n, k))
            i += 1
    return out


def candidate_plans(column_wise, m, n, k):
    plans = ["auto"]
    kt = k // 64
    tile_shapes = [(2, 1, 1, 4, 4, 1), (4, 1, 1, 4, 4, 1), (4, 2, 1, 4, 4, 1), (8, 2, 1, 4, 0, 1)]
    if column_wise:
        tile_shapes.append((4, 1, 1, 1, 4, 4))
        if m <= 64:
            rt = 1 if m <= 32 else 2
            tile_shapes += [(rt, 1, 1, 4, 4, 1), (rt, 1, 1, 8, 0, 1)]
    if m > 16:
        for rt, nt, wm, wn, pw, kw in tile_shapes:
            tiles = -(-m // (32 * rt * wm)) * -(-n // (32 * nt * wn))
            rem = tiles % 256 or tiles
            for parts in (1, 2, 3, 4):
                if parts > 1 and (kw > 1 or rt == 1 or (rt == 2 and wn == 8) or rem * parts > 256 or kt // parts < 4):
                    continue
                plans.append(f"tile {rt} {nt} {wm} {wn} {pw} {kw} {parts}")
                # the tile order of whole rounds dealt to the XCDs in blocks (1, 2, 4 or 8 row bands)
                m_tiles = -(-m // (32 * rt * wm))
                if parts == 1 and tiles >= 256 and m_tiles & (m_tiles - 1) == 0:
                    plans += [f"tile {rt} {nt} {wm} {wn} {pw} {kw} 1 {bands}" for bands in (1, 2, 4, 8)
                              if bands <= m_tiles <= 32 * bands]
    if m <= 16:
        plans += ["streaming 2 1 1 16 1 16", "streaming 2 2 1 16 1 16", "streaming 4 1 1 8 1 8", "streaming 4 2 1 8 1 8",
                  "streaming 4 1 1 4 1 1", "streaming 2 4 1 8 2 8", "streaming 2 4 1 4 2 4", "streaming 2 7 1 8 2 8",
                  "streaming 4 1 1 8 2 8", "streaming 4 3 1 8 2 8"]
        rows = 1 if m == 1 else 4 if m <= 4 else 8 if m <= 8 else 16
        slices = k // 128
        for waves in (4, 8, 16):
            depth = -(-slices // waves)
            for nt in (1, 2, 3, 4):
                plans.append(f"decode {rows} {nt} {waves} {depth}")
    elif m <= 1024:
        for nt in (1, 2, 4, 6, 8):
            for rows_in in (1, 2):
                plans.append(f"streaming 2 {nt} 2 8 {rows_in} 8")
    return plans


def time_plan(torch, launch_on_set, sets, settle, regions=3):
    copies = len(sets)
    n_launch = copies * max(1, 48 // copies)
    idx = [0]

    def fn():
        launch_on_set(sets[idx[0] % copies])
        idx[0] += 1

    fn()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            for _ in range(n_launch):
                fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < settle:
        graph.replay()
        torch.cuda.synchronize()
    times = []
    for _ in range(regions):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        graph.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1) * 1e3 / n_launch)
    times.sort()
    del graph
    return times[len(times) // 2]


def check_shape(torch, capi, device, variant, m, n, k, settle, every_plan=False):
    bf16, bs, column_wise, has_zp = {**VARIANTS, **FITTED_VARIANTS}[variant]
    dtype = torch.bfloat16 if bf16 else torch.float16
    per_set = k * n // 2 + 2 * k * n // bs + (k * n // bs if has_zp else 0)
    streams_weights = m <= 128
    copies = min(24, 2 * INFINITY_CACHE_BYTES // per_set + 1) if streams_weights else 1
    g = torch.Generator(device=device).manual_seed(m + n + k)
    a = torch.randn(m, k, generator=g, device=device).to(dtype)
    w_elems, meta = capi.quant_size(bs, column_wise, k, n)
    sets = []
    for _ in range(copies):
        w = (torch.randn(n, k, generator=g, device=device) * 0.02).to(dtype)
        q_w = torch.empty(w_elems, dtype=torch.uint8, device=device)
        q_s = torch.empty(meta, dtype=dtype, device=device)
        q_z = torch.empty(meta, dtype=torch.uint8, device=device) if has_zp else None
        capi.quant(bs, column_wise, w, q_w, q_s, q_z, bf16=bf16)
        sets.append((q_w, q_s, q_z))
        del w
    out = torch.empty(m, n, dtype=dtype, device=device)
    want = torch.empty(m, n, dtype=dtype, device=device)
    capi.gemm_with_plan("auto", bs, column_wise, m, n, k, a, *sets[0], want, bf16=bf16)
    torch.cuda.synchronize()
    scale = want.float().abs().max().item()
    chosen_text = capi.gemm_plan(bs, column_wise, m, n, k, has_zp, bf16)[2]
    results = {}
    for plan in candidate_plans(column_wise, m, n, k):
        def launch(s, plan=plan):
            capi.gemm_with_plan(plan, bs, column_wise, m, n, k, a, s[0], s[1], s[2], out, bf16=bf16)
        out.fill_(float("nan"))
        try:
            launch(sets[0])
        except capi.Blkq4Error:
            continue  # no such kernel for this problem
        torch.cuda.synchronize()
        diff = (out.float() - want.float()).abs().max().item()
        if not diff <= (2e-2 if bf16 else 4e-3) * scale:
            results[plan] = {"error": diff / scale}
            continue
        results[plan] = {"us": round(time_plan(torch, launch, sets, settle), 2)}
        # every recording of a split plan got a workspace of its own: the recording is gone, hand them back
        torch.cuda.synchronize()
        capi.workspace_release()
    timed = {p: r["us"] for p, r in results.items() if "us" in r}
    chosen_us = timed["auto"]
    forced = {p: t for p, t in timed.items() if p != "auto"}
    best_plan = min(forced, key=forced.get)
    row = {"variant": variant, "m": m, "n": n, "k": k, "weight_sets": copies, "chosen": chosen_text, "chosen_us": chosen_us,
           "best_forced": best_plan, "best_forced_us": forced[best_plan],
           "chosen_over_best": round(chosen_us / min(chosen_us, forced[best_plan]), 3),
           "wrong_results": [p for p, r in results.items() if "error" in r], "plans_timed": len(timed)}
    if every_plan:
        row["us_by_plan"] = forced
    return row


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--part", default="1/1", help="i/n: the i-th of n slices of the shape list")
    ap.add_argument("--quick", action="store_true", help="shorter settle phase")
    ap.add_argument("--shapes", default="", help="variant:m:n:k,... instead of the built-in list")
    ap.add_argument("--every-plan", action="store_true", help="print every forced plan's time, not only the best one's")
    args = ap.parse_args(argv)
    import torch
    from gemmlib_amd import capi
    capi.load()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    i, n_parts = (int(x) for x in args.part.split("/"))
    todo = shapes()[i - 1::n_parts]
    if args.shapes:
        todo = [(v, int(m), int(n), int(k)) for v, m, n, k in (item.split(":") for item in args.shapes.split(","))]
    rows = []
    for variant, m, n, k in todo:
        row = check_shape(torch, capi, device, variant, m, n, k, 0.05 if args.quick else 0.15, args.every_plan)
        rows.append(row)
        print(json.dumps(row), flush=True)
        torch.cuda.empty_cache()
    within = sum(r["chosen_over_best"] <= 1.05 for r in rows)
    print(json.dumps({"shapes": len(rows), "chosen_within_5_percent_of_best": within,
                      "worst": max(rows, key=lambda r: r["chosen_over_best"])}), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
