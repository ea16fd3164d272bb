"""A C++ caller of the C ABI, compiled with g++ against include/ms_blkq4gemm.h and linked to the library the way
the reference's own callers are (reference: python/ms_blkq4linear_ext/ms_blkq4linear.cpp:33,56,105 pass a
std::string* for the error message and int64_t references for the sizes).  Host-only calls: the size query and
validation failures, which return before anything touches a GPU."""

import os
import subprocess
import textwrap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SOURCE = textwrap.dedent(r"""
    #include <cstdio>
    #include <string>
    #include "ms_blkq4gemm.h"

    int main() {
      std::string err;
      int64_t w = -1, meta = -1;
      if (blkq4_fp16_quant_size_sm80(32, true, 4096, 11008, w, meta, &err) != 0) return 1;
      std::printf("%lld %lld\n", static_cast<long long>(w), static_cast<long long>(meta));
      if (blkq4_fp16_quant_size_sm80(32, true, 96, 32, w, meta, &err) != -1) return 2;
      std::printf("%s\n", err.c_str());
      char dummy[16];
      err.clear();
      if (blkq4_fp16_gemm_sm80(64, true, 4, 64, 64, nullptr, dummy, 10, dummy, 2048, dummy, 128, nullptr, 0, dummy, 512,
                               &err) != -1) return 3;
      std::printf("%s\n", err.c_str());
      err.clear();
      if (blkq4_fp16_gemm_bias_sm80(64, true, 4, 64, 64, nullptr, dummy, 512, dummy, 2048, dummy, 128, nullptr, 0, dummy,
                                    100, dummy, 512, &err) != -1) return 4;
      std::printf("%s\n", err.c_str());
      // a null error message is allowed
      if (blkq4_fp16_quant_sm80(8, true, 64, 32, 64, nullptr, dummy, 0, dummy, 0, dummy, 0, nullptr, 0, nullptr) != -1) return 5;
      return 0;
    }
""")


def test_cxx_program_links_and_gets_the_reference_messages(capi, tmp_path):
    capi.load()
    lib = capi.LIB_PATH
    src = tmp_path / "consumer.cpp"
    exe = tmp_path / "consumer"
    src.write_text(SOURCE)
    subprocess.run(["g++", "-std=c++17", "-D_GLIBCXX_USE_CXX11_ABI=1", "-I", os.path.join(ROOT, "include"), str(src),
                    "-o", str(exe), lib, "-Wl,-rpath," + os.path.dirname(lib)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines()
    assert out == [
        "22544384 1409024",
        "Cannot block quantize matrix with rows: 96",
        "Unexpected activation tensor size: 10 expected: 512",
        "Unexpected bias tensor size: 100 expected: 128",
    ]
