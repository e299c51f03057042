"""bench.py's own pieces that can be checked without a GPU: its input generator (evaluated with torch,
on the device in a real run) against the CPU generator the parity tests draw from, the OpenCL probe,
and the reader of the tracked traffic profile."""
import numpy as np
import pytest
import torch

import bench
import oracle


@pytest.mark.parametrize("seed", [1, 2, 3, 11, 21, 12345678901234567, 2 ** 63 + 5])
@pytest.mark.parametrize("n", [1, 5, 4099])
def test_uniform_streams_equal_the_test_generator(n, seed):
    for tdt, ndt in ((torch.float32, np.float32), (torch.float64, np.float64)):
        got = bench.gen_uniform(torch, n, seed, tdt, device="cpu").numpy()
        np.testing.assert_array_equal(got, oracle.uniform(n, seed, ndt))


def test_uniform_is_cut_into_chunks_consistently():
    whole = bench._in_chunks(torch, 1000, "cpu", torch.float64, lambda f, c: torch.arange(f, f + c, dtype=torch.float64), chunk=64)
    np.testing.assert_array_equal(whole.numpy(), np.arange(1000.0))
    a = bench.gen_uniform(torch, (1 << 24) + 3, 7, torch.float32, device="cpu").numpy()
    b = oracle.uniform((1 << 24) + 3, 7, np.float32)
    np.testing.assert_array_equal(a[-5:], b[-5:])
    np.testing.assert_array_equal(a[(1 << 24) - 2:(1 << 24) + 2], b[(1 << 24) - 2:(1 << 24) + 2])


@pytest.mark.parametrize("seed", [11, 12, 22])
def test_normal_streams_equal_the_test_generator_to_rounding(seed):
    # Box-Muller through torch's log / cos instead of libm's: the same stream up to a few units in the last place.
    n = 5000
    got = bench.gen_normal(torch, n, seed, torch.float64, device="cpu").numpy()
    want = oracle.normal(n, seed, np.float64)
    assert np.abs(got - want).max() <= 8 * np.finfo(np.float64).eps * np.abs(want).max()
    assert abs(got.mean()) < 0.1 and abs(got.std() - 1) < 0.1


@pytest.mark.parametrize("n", [1, 2, 37])
def test_triangle_equals_the_test_generator(n):
    got = bench.gen_triangular(torch, n, 21, torch.float64, device="cpu").numpy()
    want = oracle.triangular(n, n, True, 21, np.float64)
    np.testing.assert_array_equal(got, want)   # NaN above the diagonal in both
    m = got.reshape(n, n).T                     # m[r, c]
    assert np.isnan(m[np.triu_indices(n, 1)]).all()
    d = np.diag(m)
    assert ((d >= 1) & (d < 2)).all()
    low = m[np.tril_indices(n, -1)]
    assert (np.abs(low) <= 1.0 / n).all()


def test_opencl_probe_reports_what_it_saw():
    usable, text = bench.opencl_cpu_probe()
    assert isinstance(usable, bool) and isinstance(text, str) and text
    # whatever the box offers, the sentence names the loader or says that there is none
    assert "OpenCL" in text


def test_traffic_reader_guards_on_the_kernel(tmp_path, monkeypatch):
    prof = tmp_path / "p.md"
    prof.write_text(
        "| workload | kernel | counter | per-dispatch mean | scaled bytes per dispatch |\n"
        "|---|---|---|---|---|\n"
        "| sgemm | `gemm_mfma_kernel<float, 256, 128, 16, 128, 64, false>` | FETCH_SIZE | 1 KiB (n=4) | 4.5 GB |\n"
        "| sgemm | `gemm_mfma_kernel<float, 256, 128, 16, 128, 64, false>` | WRITE_SIZE | 1 KiB (n=4) | 0.5 GB |\n"
        "| dtrsm | `gemm_mfma_kernel<double, 128, 128, 16, 64, 64, false>` | FETCH_SIZE | 1 KiB (n=4) | 0.8 GB |\n"
        "* dtrsm: 32 kernels per call\n"
        "* dtrsm: 8.966 GB per call = 1.11 TB/s\n")
    monkeypatch.setattr(bench, "TRAFFIC_PROFILE", str(prof))
    same = "gemm_mfma_kernel<s,256x128x16,256 threads> NN M=8192 N=8192 K=8192 grid=(2048,1) splits=1 tail_slices=1"
    other = same.replace("256x128x16", "128x128x16")
    assert bench.profiled_traffic("sgemm", same)[0] == pytest.approx(5.0e9)
    assert bench.profiled_traffic("sgemm", other)[0] is None
    assert bench.profiled_traffic("sgemm", same.replace("splits=1", "splits=4"))[0] is None
    assert bench.profiled_traffic("dgemm", same.replace("<s,", "<d,"))[0] is None          # no dgemm rows
    d = "gemm_mfma_kernel<d,128x128x16,256 threads> NN M=4096 N=8192 K=4096 grid=(2048,1) splits=1 tail_slices=1"
    assert bench.profiled_traffic("dtrsm", d, 32)[0] == pytest.approx(8.966e9)
    assert bench.profiled_traffic("dtrsm", d, 30)[0] is None
    assert bench.profiled_traffic("dtrsm", d.replace("128x128x16", "64x64x16"), 32)[0] is None
