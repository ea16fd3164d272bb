"""Measurement aids for ``bench.py``: a small library of its own (an empty kernel, a kernel that only issues the
GEMV's memory requests, a kernel that only issues MFMAs).  Not part of the product: ``bench.py`` builds it when it
is missing, ``__graft_entry__.build()`` builds it together with everything else."""

from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCE = os.path.join(HERE, "blkq4_probe.hip")
LIB_PATH = os.path.join(HERE, "libblkq4_probe.so")
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function",
]


def build(force: bool = False) -> str:
    if not force and os.path.exists(LIB_PATH) and os.path.getmtime(LIB_PATH) >= os.path.getmtime(SOURCE):
        return LIB_PATH
    proc = subprocess.run([HIPCC, *FLAGS, "-shared", "-o", LIB_PATH, SOURCE], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True)
    if proc.returncode != 0:
        sys.stderr.write(proc.stdout + proc.stderr)
        raise RuntimeError("building the bench probe failed")
    return LIB_PATH
