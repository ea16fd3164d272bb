"""Builds the native parts in-tree:

* ``gemmlib_amd/lib/libms_blkq4gemm.so`` -- the C-ABI library (host code + gfx950 HIP kernels);
* ``ms_blkq4linear_ext*.so`` at the top of the tree, next to ``ms_blkq4linear.py`` -- the PyTorch-ROCm
  extension on top of it, importable as the reference's is: ``import ms_blkq4linear_ext``
  (reference: python/ms_blkq4linear.py:7, python/setup.py:17-26).

Run as ``python -m gemmlib_amd.build [--no-ext]``.  hipcc cross-compiles for gfx950, so no GPU is
needed to build.
"""

from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import sysconfig
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_DIR = os.path.join(PKG_DIR, "lib")
OBJ_DIR = os.path.join(PKG_DIR, "build")
INCLUDE = os.path.join(ROOT, "include")
LIB_PATH = os.path.join(LIB_DIR, "libms_blkq4gemm.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# Sources and flags come from csrc/build_manifest.json, which CMakeLists.txt reads too.
#   -ffp-contract=off: every fused multiply-add the quantizer needs is written as an explicit fmaf.
#   The division stays IEEE correctly rounded; no fast-math anywhere.
#   packed-fp32-ops is switched off for the device code (the host pass prints a harmless warning).
#   Kernel arguments of the decode kernels arrive in registers with the wave (the code object keeps a prologue that
#   loads them for firmware that does not preload).
with open(os.path.join(CSRC, "build_manifest.json")) as _f:
    MANIFEST = json.load(_f)
HIP_SOURCES = list(MANIFEST["hip_sources"])
HOST_SOURCES = list(MANIFEST["host_sources"])
EXTRA_HIP_FLAGS = {k: list(v) for k, v in MANIFEST["extra_hip_flags"].items()}
HIP_FLAGS = ["--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fvisibility=hidden", *MANIFEST["hip_flags"]]
for _feature in MANIFEST["hip_target_features_off"]:
    HIP_FLAGS += ["-Xclang", "-target-feature", "-Xclang", "-" + _feature]
HOST_FLAGS = ["-std=c++17", "-fPIC", "-fvisibility=hidden", *MANIFEST["host_flags"]]


def _run(cmd, quiet_stderr_filter=None):
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    err = proc.stderr
    if quiet_stderr_filter:
        err = "\n".join(l for l in err.splitlines() if quiet_stderr_filter not in l)
    if proc.returncode != 0:
        sys.stderr.write(" ".join(cmd) + "\n" + proc.stdout + err + "\n")
        raise RuntimeError(f"command failed ({proc.returncode}): {cmd[0]} ... {cmd[-1]}")
    if err.strip():
        sys.stderr.write(err + "\n")


def build_library(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = []
    objs = []
    for src in HIP_SOURCES:
        obj = os.path.join(OBJ_DIR, src + ".o")
        objs.append(obj)
        jobs.append(([HIPCC, *HIP_FLAGS, *EXTRA_HIP_FLAGS.get(src, []), "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj],
                     "packed-fp32-ops"))
    for src in HOST_SOURCES:
        obj = os.path.join(OBJ_DIR, src + ".o")
        objs.append(obj)
        jobs.append((["g++", *HOST_FLAGS, "-I", INCLUDE, "-I", CSRC, "-c", os.path.join(CSRC, src), "-o", obj], None))
    with ThreadPoolExecutor(max_workers=min(8, len(jobs))) as pool:
        list(pool.map(lambda j: _run(*j), jobs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs], "packed-fp32-ops")
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


def ext_path() -> str:
    suffix = sysconfig.get_config_var("EXT_SUFFIX") or ".so"
    return os.path.join(ROOT, "ms_blkq4linear_ext" + suffix)


def build_extension(verbose: bool = True, out: str | None = None) -> str:
    """The pybind11/torch extension, compiled as plain C++ against PyTorch-ROCm and linked to the
    C-ABI library (no hipify pass, no CUDA headers).  It finds the library at ``gemmlib_amd/lib`` next to
    itself, in the source tree and in an installed one alike."""
    import torch
    from torch.utils import cpp_extension

    out = out or ext_path()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    inc = []
    for p in cpp_extension.include_paths():
        inc += ["-isystem", p]
    inc += ["-isystem", sysconfig.get_paths()["include"], "-isystem", "/opt/rocm/include"]
    cmd = [
        "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
        "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=ms_blkq4linear_ext",
        "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        "-Wno-deprecated-declarations",
        *inc, "-I", INCLUDE,
        os.path.join(CSRC, "ms_blkq4linear_ext.cpp"), "-o", out,
        "-L", LIB_DIR, "-lms_blkq4gemm", "-Wl,-rpath,$ORIGIN/gemmlib_amd/lib",
        "-L", torch_lib, "-ltorch", "-ltorch_cpu", "-ltorch_hip", "-lc10", "-lc10_hip", "-ltorch_python",
        "-Wl,-rpath," + torch_lib,
    ]
    _run(cmd)
    if verbose:
        print(f"built {out}")
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--no-ext", action="store_true", help="build only the C-ABI library")
    args = ap.parse_args(argv)
    build_library()
    if not args.no_ext:
        build_extension()
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
