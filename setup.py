"""Installable build: ``pip install --no-build-isolation .`` or ``python setup.py build_ext --inplace``.

Takes the place of the reference's ``python/setup.py:17-26`` (a ``CUDAExtension`` linked against a CMake-built
``libms_blkq4gemm``) and of its ``CMakeLists.txt:48-53``: here one command compiles the gfx950 C-ABI library
with hipcc and the PyTorch-ROCm extension with g++ (no hipify pass), and installs

* ``ms_blkq4linear_ext`` (top-level extension module) and ``ms_blkq4linear`` (top-level module),
* the ``gemmlib_amd`` package with ``gemmlib_amd/lib/libms_blkq4gemm.so`` and ``gemmlib_amd/include/ms_blkq4gemm.h``
  (what a C or C++ consumer links and includes).
"""

import os
import shutil
import sys

from setuptools import Extension, setup
from setuptools.command.build_ext import build_ext
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)


class BuildNative(build_ext):
    """Builds the library and the extension with the package's own build module (hipcc + g++)."""

    def run(self):
        from gemmlib_amd import build as native
        native.build_library(verbose=False)
        ext_out = native.build_extension(verbose=False)
        if not self.inplace:
            target = self.get_ext_fullpath("ms_blkq4linear_ext")
            os.makedirs(os.path.dirname(target), exist_ok=True)
            shutil.copy2(ext_out, target)
            lib_dir = os.path.join(self.build_lib, "gemmlib_amd", "lib")
            os.makedirs(lib_dir, exist_ok=True)
            shutil.copy2(native.LIB_PATH, lib_dir)


class BuildPy(build_py):
    """Also ships the C header inside the package."""

    def run(self):
        super().run()
        inc = os.path.join(self.build_lib, "gemmlib_amd", "include")
        os.makedirs(inc, exist_ok=True)
        shutil.copy2(os.path.join(ROOT, "include", "ms_blkq4gemm.h"), inc)


setup(
    name="ms_blkq4linear_ext",
    version="0.2.0",
    description="blkq4 (blockwise int4 weights x fp16/bf16) GEMM, GEMV and quantizer for MI355X (gfx950)",
    packages=["gemmlib_amd"],
    py_modules=["ms_blkq4linear"],
    # the sources listed here are only what setuptools wants to see; BuildNative compiles everything itself
    ext_modules=[Extension("ms_blkq4linear_ext", sources=["gemmlib_amd/csrc/ms_blkq4linear_ext.cpp"])],
    cmdclass={"build_ext": BuildNative, "build_py": BuildPy},
    python_requires=">=3.9",
    zip_safe=False,
)
