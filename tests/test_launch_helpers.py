"""Host-side launch helpers (gemmlib_amd/csrc/blkq4_launch.h), compiled with g++ and run on the CPU.

Every instantiation of a kernel template has the same function TYPE, so the once-per-device flags of the
dynamic-LDS limit must be keyed by the function VALUE: two instantiations get two sets of flags."""

import os
import subprocess
import textwrap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SOURCE = textwrap.dedent(r"""
    #include <cstdio>
    #include "blkq4_launch.h"

    template <int A, int B>
    void kernel_like(const int*, int) {}

    int main() {
      auto& f1 = blkq4::lds_limit_flags<kernel_like<1, 2>>();
      auto& f2 = blkq4::lds_limit_flags<kernel_like<2, 1>>();
      auto& f1_again = blkq4::lds_limit_flags<kernel_like<1, 2>>();
      if (&f1 == &f2) return 1;          // same type, different kernels: flags of their own
      if (&f1 != &f1_again) return 2;    // one kernel: one set of flags
      f1.fetch_or(1);
      if (f2.load() != 0 || f1_again.load() != 1) return 3;
      std::puts("distinct");
      return 0;
    }
""")


def test_two_kernel_instantiations_get_distinct_lds_limit_flags(tmp_path):
    src = tmp_path / "flags.cpp"
    exe = tmp_path / "flags"
    src.write_text(SOURCE)
    subprocess.run(["g++", "-std=c++17", "-D__HIP_PLATFORM_AMD__=1", "-I", "/opt/rocm/include", "-I",
                    os.path.join(ROOT, "gemmlib_amd", "csrc"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert out.strip() == "distinct"
