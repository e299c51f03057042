"""Builds libclblas_amd.so (HIP kernels + C ABI) for gfx950, in-tree.

Usage:  python -m clblas_amd.build        (or  clblas_amd.build.build_library())
hipcc cross-compiles without a GPU present.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libclblas_amd.so")
CLIENT_PATH = os.path.join(HERE, "client", "clblas_amd-client")

SOURCES = ["api.cpp", "gemm_f32.hip", "gemm_f64.hip", "gemm_c32.hip", "gemm_c64.hip", "level3.hip", "trsm.hip", "noalloc.hip"]

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar float code.
DEVICE_FLAGS = ["--offload-arch=gfx950", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# -Wno-align-mismatch: C is accessed through element-aligned vector types on purpose (offsets and odd ld).
COMMON_FLAGS = ["-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
                "-Wno-align-mismatch"]


def _hipcc():
    return os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc()] + COMMON_FLAGS
    if src.endswith(".hip"):
        cmd += DEVICE_FLAGS
        cmd += ["-Rpass-analysis=kernel-resource-usage"]
    cmd += ["-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # The host pass warns that it does not know the packed-fp32 feature; that is harmless.
    lines = [l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l]
    # Resource-usage remarks: a kernel whose accumulators end up in scratch memory still gives
    # right answers, fifty times slower - refuse to build it.
    spilled, name = [], "?"
    for l in lines:
        if "Function Name:" in l:
            name = l.split("Function Name:")[1].split("[-Rpass")[0].strip()
        elif "ScratchSize [bytes/lane]:" in l:
            if int(l.split("ScratchSize [bytes/lane]:")[1].split()[0]) > 0:
                spilled.append(name)
    kept, in_remark = [], False
    for l in lines:  # drop the remarks together with the source excerpt that follows each of them
        if "-Rpass-analysis=kernel-resource-usage" in l:
            in_remark = True
        elif in_remark and (l.lstrip().startswith("|") or l.lstrip().split(" ", 1)[0].isdigit()):
            pass
        else:
            in_remark = False
            kept.append(l)
    if not any("warning" in l or "error" in l for l in kept):
        kept = []  # only include-stack lines of the dropped remarks are left
    err = "\n".join(kept)
    if res.returncode != 0:
        raise RuntimeError("compile failed: %s\n%s" % (" ".join(cmd), err))
    if spilled:
        raise RuntimeError("%s: kernels use scratch memory (register spills): %s" % (src, ", ".join(spilled)))
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build_library(verbose=True):
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as ex:
        objs = list(ex.map(_compile, SOURCES))
    cmd = [_hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950"] + objs + ["-o", LIB_PATH]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed: %s\n%s" % (" ".join(cmd), res.stderr))
    if verbose:
        print("built", LIB_PATH)
    build_client(verbose)
    return LIB_PATH


def build_client(verbose=True):
    """Benchmark command line (CSV in the schema of the reference's published results)."""
    cmd = [_hipcc()] + COMMON_FLAGS + [os.path.join(HERE, "client", "client.cpp"), "-o", CLIENT_PATH,
                                      "-L" + HERE, "-lclblas_amd", "-Wl,-rpath,$ORIGIN/.."]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("client build failed: %s\n%s" % (" ".join(cmd), res.stderr))
    if verbose:
        print("built", CLIENT_PATH)
    return CLIENT_PATH


if __name__ == "__main__":
    build_library()
