"""The library's scratch-buffer bookkeeping is host code written against an allocator interface
(clblas_amd/csrc/workspace.hpp); this compiles it with a counting allocator and checks that
buffers are reused, that create/use/destroy cycles of streams do not accumulate memory with or
without an explicit release, and that nothing is allocated for a stream under graph capture."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_workspace_cache_is_bounded(tmp_path):
    exe = str(tmp_path / "ws_check")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-g", "-Wall", "-Werror", "-fsanitize=address,undefined",
                           "-static-libasan", "-static-libubsan",
                           "-I", os.path.join(ROOT, "clblas_amd", "csrc"),
                           os.path.join(ROOT, "tests", "cpp", "workspace_cache_check.cpp"), "-o", exe, "-pthread"])
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip() == "ok", out.stdout + out.stderr
