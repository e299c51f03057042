"""The host side of the library (argument validation, folding, status mapping, scratch bookkeeping)
built for the CPU with AddressSanitizer and UBSan and driven through every validation path: no
kernel is launched (every call fails validation before it reaches a launch), so no GPU is needed.

Recipe: hipcc compiles clblas_amd/csrc/api.cpp for the host only, with -fsanitize=address,undefined
(each directly after -Xarch_host); the kernel launchers it would link against are replaced by stubs
that abort if they are ever reached (tests/cpp/host_api_sanitize.cpp, which also holds the driver)."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HIPCC = "/opt/rocm/bin/hipcc"


@pytest.mark.skipif(not os.path.exists(HIPCC), reason="needs hipcc for the HIP host headers")
def test_validation_paths_under_asan_ubsan(tmp_path):
    exe = str(tmp_path / "host_api_sanitize")
    cmd = [HIPCC, "-std=c++17", "-O1", "-g", "-Wall", "-Wno-unused-function",
           "-Xarch_host", "-fsanitize=address", "-Xarch_host", "-fsanitize=undefined",
           "-Xarch_host", "-fno-sanitize-recover=undefined", "--offload-arch=gfx950",
           os.path.join(ROOT, "clblas_amd", "csrc", "api.cpp"),
           os.path.join(ROOT, "tests", "cpp", "host_api_sanitize.cpp"), "-o", exe]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-3000:]
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0 and out.stdout.strip().endswith("ok"), out.stdout[-2000:] + out.stderr[-3000:]
