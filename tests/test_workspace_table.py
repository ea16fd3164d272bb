"""Who owns which workspace of the split tile kernels (gemmlib_amd/csrc/blkq4_workspace_table.h): host-only
bookkeeping, compiled with g++ and run on the CPU.  The reference's GEMM has no workspace
(src/blkq4_f16_gemm_sm80.cu:38-153), so there is nothing of the reference's to compare with: the properties checked
are the ones the public header promises about which calls share a buffer and how many buffers there can be."""

import os
import subprocess
import textwrap

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SOURCE = textwrap.dedent(r"""
    #include <cstdio>
    #include "blkq4_workspace_table.h"

    #define CHECK(x) do { if (!(x)) { std::printf("line %d: %s\n", __LINE__, #x); return 1; } } while (0)

    int main() {
      using blkq4::WorkspaceKey;
      blkq4::WorkspaceTable t;
      char buffers[64];
      const void* s1 = buffers + 40, *s2 = buffers + 41;
      // eager calls on one stream share a buffer; another stream, another device, a recording do not
      CHECK(t.find(WorkspaceKey{0, s1, 0}) == nullptr);
      CHECK(t.add(WorkspaceKey{0, s1, 0}, &buffers[0]));
      CHECK(t.find(WorkspaceKey{0, s1, 0}) == &buffers[0]);
      CHECK(t.find(WorkspaceKey{0, s2, 0}) == nullptr);
      CHECK(t.find(WorkspaceKey{1, s1, 0}) == nullptr);
      CHECK(t.find(WorkspaceKey{0, s1, 7}) == nullptr);       // a graph being recorded on s1
      CHECK(!t.add(WorkspaceKey{0, s1, 0}, &buffers[1]));      // one buffer per key
      CHECK(!t.add(WorkspaceKey{0, s2, 0}, nullptr));
      CHECK(t.add(WorkspaceKey{0, s1, 7}, &buffers[1]));
      CHECK(t.add(WorkspaceKey{0, s1, 8}, &buffers[2]));       // a second recording on the same stream
      CHECK(t.find(WorkspaceKey{0, s1, 7}) == &buffers[1] && t.find(WorkspaceKey{0, s1, 8}) == &buffers[2]);
      CHECK(t.in_use() == 3 && t.in_use_by_recordings() == 2);
      // the bounds: 16 streams and 16 recordings, counted separately
      for (int i = 1; i < blkq4::kMaxEagerWorkspaces; ++i) CHECK(t.add(WorkspaceKey{0, buffers + i, 0}, &buffers[3]));
      CHECK(!t.has_room(false) && t.has_room(true));
      CHECK(!t.add(WorkspaceKey{0, buffers + 50, 0}, &buffers[3]));
      CHECK(t.find(WorkspaceKey{0, buffers + 50, 0}) == nullptr);
      for (int i = 2; i < blkq4::kMaxCapturedWorkspaces; ++i) CHECK(t.add(WorkspaceKey{0, s2, 100ull + i}, &buffers[4]));
      CHECK(!t.has_room(true));
      CHECK(!t.add(WorkspaceKey{0, s2, 99}, &buffers[4]));
      CHECK(t.in_use() == blkq4::WorkspaceTable::capacity());
      CHECK(t.find(WorkspaceKey{0, s1, 0}) == &buffers[0]);    // full, and still finds what it has
      // release: every buffer handed back exactly once, then room again
      int freed = 0, on_device_0 = 0;
      t.release_all([&](int device, void* p) { ++freed; on_device_0 += device == 0; CHECK(p != nullptr); return 0; });
      CHECK(freed == blkq4::WorkspaceTable::capacity() && on_device_0 == freed);
      CHECK(t.in_use() == 0 && t.has_room(false) && t.has_room(true));
      CHECK(t.find(WorkspaceKey{0, s1, 0}) == nullptr);
      std::puts("ok");
      return 0;
    }
""")


def test_workspace_table_keys_bounds_and_release(tmp_path):
    src = tmp_path / "table.cpp"
    exe = tmp_path / "table"
    src.write_text(SOURCE)
    subprocess.run(["g++", "-std=c++17", "-Wall", "-Werror", "-I", os.path.join(ROOT, "gemmlib_amd", "csrc"), str(src),
                    "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout


def test_workspace_queries_fail_cleanly_without_a_gpu(capi):
    """No GPU here: the bookkeeping queries must come back with -1 and a message, not crash."""
    import torch
    if torch.cuda.is_available():
        state, in_use, most, nbytes = capi.workspace_info(0)
        assert state in (0, 1) and most == 32 and nbytes == (32 << 20) + (16 << 10) and 0 <= in_use <= most
        return
    for call in (lambda: capi.workspace_info(0), capi.workspace_release, capi.noalloc_init):
        try:
            call()
        except capi.Blkq4Error as e:
            assert "Kernel execution failed" in str(e) or str(e), str(e)
        else:
            raise AssertionError("expected a failure without a GPU")
