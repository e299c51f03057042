"""The benchmark command line: option parsing (CPU) and one small run per function (GPU).
Its CSV columns are those of the reference's published results
(doc/performance/clBLAS_2.7.1/S9150/sgemmNT_S9150_14.50.2_2.7.1_8.csv:1)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLIENT = os.path.join(ROOT, "clblas_amd", "client", "clblas_amd-client")
HEADER = ("m,n,k,lda,ldb,ldc,offa,offb,offc,alpha,beta,order,transa,transb,side,uplo,diag,function,device,library,"
          "numQueues,label,GFLOPS")


def test_help_and_bad_options():
    assert os.path.exists(CLIENT), "build with python -m clblas_amd.build"
    r = subprocess.run([CLIENT, "--help"], capture_output=True, text=True)
    assert r.returncode == 2 and "--transposeA" in r.stdout and "--apiCallCount" in r.stdout
    r = subprocess.run([CLIENT, "-f", "gemv"], capture_output=True, text=True)
    assert r.returncode == 2
    r = subprocess.run([CLIENT, "--nonsense"], capture_output=True, text=True)
    assert r.returncode == 2


@pytest.mark.gpu
def test_csv_rows():
    r = subprocess.run([CLIENT, "-f", "gemm", "-r", "s", "--sizes", "256:512:256", "--transposeB", "1", "-p", "2",
                        "--apiCallCount", "2", "--label", "t"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    lines = r.stdout.strip().splitlines()
    assert lines[0] == HEADER and len(lines) == 3
    row = dict(zip(HEADER.split(","), lines[2].split(",")))
    assert row["m"] == "512" and row["transb"] == "transpose" and row["function"] == "sgemm"
    assert row["library"] == "clblas_amd" and float(row["GFLOPS"]) > 0
    r = subprocess.run([CLIENT, "-f", "trsm", "-r", "d", "-m", "300", "-n", "200", "--uplo", "1", "--diag", "1", "-p",
                        "2", "--apiCallCount", "1", "--noheader"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    row = dict(zip(HEADER.split(","), r.stdout.strip().split(",")))
    assert row["function"] == "dtrsm" and row["uplo"] == "lower" and float(row["GFLOPS"]) > 0
    for fn, prec, extra in (("gemm", "z", ["--transposeA", "2"]), ("trmm", "c", ["--side", "1"]),
                            ("trsm", "z", ["--transposeA", "2", "--uplo", "1"]),
                            ("syr2k", "s", ["--transposeA", "1"]), ("herk", "c", ["--transposeA", "2"]),
                            ("her2k", "z", ["--uplo", "1"]), ("hemm", "c", ["--side", "1", "--uplo", "1"]),
                            ("syrk", "d", ["--uplo", "1", "--transposeA", "1"]), ("symm", "s", ["--side", "1"])):
        r = subprocess.run([CLIENT, "-f", fn, "-r", prec, "-m", "300", "-n", "200", "-k", "100", "-p", "2",
                            "--apiCallCount", "1", "--noheader"] + extra, capture_output=True, text=True, timeout=120)
        assert r.returncode == 0, r.stderr
        row = dict(zip(HEADER.split(","), r.stdout.strip().split(",")))
        assert row["function"] == prec + fn and float(row["GFLOPS"]) > 0
    for fn, prec in (("trsv", "z"), ("herk", "d")):
        r = subprocess.run([CLIENT, "-f", fn, "-r", prec], capture_output=True, text=True, timeout=120)
        assert r.returncode == 2
