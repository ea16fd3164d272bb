"""What instructions cost a wave next to its MFMAs, measured: ``python -m bench_probe.issue_probe``.

One workgroup of 4, 8 or 16 waves (one, two, four per SIMD) runs rounds of four independent 32 x 32 x 16 fp16 MFMAs, each
followed by N independent packed vector instructions; every wave reports its cycles per MFMA (``s_memtime``).  The
same launch over the whole chip gives the rate in TFLOP/s.  The tile kernel's shapes are read against these figures:
a shape with n instructions per MFMA in its computing wave cannot run that wave faster than the single-wave column."""

from __future__ import annotations

import ctypes
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def main() -> int:
    import torch
    import bench_probe
    lib = ctypes.CDLL(bench_probe.build())
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    cycles = torch.zeros(64, dtype=torch.int64, device=device)
    iters = 2000
    for threads in (256, 512, 1024):
        for n in (0, 2, 4, 6, 8, 12, 16):
            row = {"waves_per_simd": threads // 256, "vector_instructions_per_mfma": n}
            for _ in range(2):
                rc = lib.blkq4_probe_issue(n, 1, threads, iters, ctypes.c_void_p(cycles.data_ptr()), None)
                assert rc == 0, rc
                torch.cuda.synchronize()
            per_wave = cycles.cpu()[: threads // 64].tolist()
            row["cycles_per_mfma_first_wave_of_a_simd"] = per_wave[0]
            row["cycles_per_mfma_last_wave_of_a_simd"] = per_wave[-1]
            workgroups = 256 * (1024 // threads)
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            lib.blkq4_probe_issue(n, workgroups, threads, iters, ctypes.c_void_p(cycles.data_ptr()), None)
            e0.record()
            lib.blkq4_probe_issue(n, workgroups, threads, iters, ctypes.c_void_p(cycles.data_ptr()), None)
            e1.record()
            torch.cuda.synchronize()
            flop = workgroups * (threads // 64) * iters * 4 * 32768
            row["whole_chip_tflops"] = round(flop / (e0.elapsed_time(e1) * 1e-3) / 1e12, 1)
            print(json.dumps(row), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
