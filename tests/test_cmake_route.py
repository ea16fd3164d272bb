"""The CMake route (CMakeLists.txt), which a project that linked the reference's `ms_blkq4gemm` target uses
(reference: CMakeLists.txt:48-53 builds a static position-independent archive, python/setup.py:17-22 links it):
both flavours configure, every source gets the flags of gemmlib_amd/csrc/build_manifest.json -- the list the Python
build uses too -- and the static archive builds and links into a C++ program.  The archive of this test is made
from the host code and the smallest kernel file only, so that the test takes seconds; BLKQ4_CMAKE_FULL=1 in the
environment builds all of it (minutes) and runs the size query through it."""

import json
import os
import shutil
import subprocess
import textwrap

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIP_CXX = "/opt/rocm/llvm/bin/clang++"
pytestmark = pytest.mark.skipif(shutil.which("cmake") is None or not os.path.exists(HIP_CXX),
                                reason="needs cmake and the ROCm compiler")


def _configure(build_dir, shared, only=None):
    cmd = ["cmake", "-S", ROOT, "-B", str(build_dir), f"-DCMAKE_HIP_COMPILER={HIP_CXX}", "-DCMAKE_EXPORT_COMPILE_COMMANDS=ON",
           f"-DBUILD_SHARED_LIBS={'ON' if shared else 'OFF'}"]
    if only:
        cmd.append("-DBLKQ4_ONLY_SOURCES=" + ";".join(only))
    subprocess.run(cmd, check=True, capture_output=True, text=True)
    with open(os.path.join(build_dir, "compile_commands.json")) as f:
        return {os.path.basename(c["file"]): c["command"] for c in json.load(f)}


def test_both_flavours_configure_with_the_manifests_sources_and_flags(tmp_path):
    with open(os.path.join(ROOT, "gemmlib_amd", "csrc", "build_manifest.json")) as f:
        manifest = json.load(f)
    for shared in (True, False):
        commands = _configure(tmp_path / ("shared" if shared else "static"), shared)
        assert set(commands) == set(manifest["hip_sources"]) | set(manifest["host_sources"])
        for src in manifest["hip_sources"]:
            cmd = commands[src]
            for flag in manifest["hip_flags"] + ["--offload-arch=gfx950", "-fPIC", "-fvisibility=hidden"]:
                assert f" {flag} " in cmd, (src, flag)
            for feature in manifest["hip_target_features_off"]:
                assert f"-Xclang -target-feature -Xclang -{feature}" in cmd, src
            for flag in manifest["extra_hip_flags"].get(src, []):
                assert f" {flag} " in cmd + " ", (src, flag)
            if src not in manifest["extra_hip_flags"]:
                assert "kernarg-preload" not in cmd
        for src in manifest["host_sources"]:
            for flag in manifest["host_flags"] + ["-fPIC", "-fvisibility=hidden"]:
                assert f" {flag} " in commands[src], (src, flag)
    # the Python build compiles with the same lists
    from gemmlib_amd import build as native
    assert native.HIP_SOURCES == manifest["hip_sources"] and native.HOST_SOURCES == manifest["host_sources"]
    assert all(f in native.HIP_FLAGS for f in manifest["hip_flags"]) and all(f in native.HOST_FLAGS for f in manifest["host_flags"])


CONSUMER = textwrap.dedent(r"""
    #include <cstdio>
    #include <string>
    #include "ms_blkq4gemm.h"
    int main() {
      std::string err;
      int64_t w = -1, meta = -1;
      if (blkq4_fp16_quant_size_sm80(32, true, 4096, 11008, w, meta, &err) != 0) return 1;
      std::printf("%lld %lld\n", static_cast<long long>(w), static_cast<long long>(meta));
      return 0;
    }
""")


def test_static_archive_builds_and_links(tmp_path):
    full = os.environ.get("BLKQ4_CMAKE_FULL") == "1"
    build_dir = tmp_path / "static"
    _configure(build_dir, shared=False, only=None if full else ["blkq4_api.cpp", "blkq4_workspace.hip"])
    subprocess.run(["cmake", "--build", str(build_dir), "-j8"], check=True, capture_output=True, text=True)
    archive = build_dir / "libms_blkq4gemm.a"
    assert archive.exists()
    members = subprocess.run(["ar", "t", str(archive)], check=True, capture_output=True, text=True).stdout.split()
    assert "blkq4_api.cpp.o" in members and "blkq4_workspace.hip.o" in members
    symbols = subprocess.run(["nm", "-g", "--defined-only", str(archive)], check=True, capture_output=True, text=True).stdout
    for name in ("blkq4_fp16_gemm_sm80", "blkq4_fp16_quant_sm80", "blkq4_fp16_quant_size_sm80", "blkq4_dev_workspace"):
        assert f" T {name}\n" in symbols, name
    if not full:
        return  # the archive lacks the kernels' launchers: nothing to link a program against
    src = tmp_path / "consumer.cpp"
    exe = tmp_path / "consumer"
    src.write_text(CONSUMER)
    subprocess.run([HIP_CXX, "-std=c++17", "-D_GLIBCXX_USE_CXX11_ABI=1", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
                    str(archive), "-L/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert out.strip() == "22544384 1409024"
