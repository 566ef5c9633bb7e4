"""The command-line driver keeps the reference drivers' arguments and output format
(kernel/ft_sgemm/sgemm.cu:14-27,186-196,419-422; kernel/sgemm/sgemm.cu:17-30,367-377; kernel/saxpy/saxpy.cu:57-66)."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "hpcdeepneuralnetworks_amd", "lib", "hpcdnn_bench")


def _run(*args):
    assert os.path.exists(BIN), "build the driver first (make -C hpcdeepneuralnetworks_amd/csrc)"
    p = subprocess.run([BIN, *map(str, args)], capture_output=True, text=True, timeout=110)
    assert p.returncode == 0, p.stderr
    return p.stdout


def _floats(text):
    return [float(v) for v in re.findall(r"[-+]?\d+\.\d+", text)]


def test_ft_sgemm_series_lines():
    out = _run("ft_sgemm", 256, 768, 256, 0, 23)
    assert out.startswith("     256|     512|     768|")
    assert "finish verified!" in out
    series = dict(re.findall(r"^(\w+) = th\.as_tensor\(\[(.*)\]\)(?:  #.*)?$", out, flags=re.M))
    assert list(series) == ["hpcdnn_sgemm", "kernel_sgemm_small", "kernel_sgemm_medium", "kernel_sgemm_large",
                            "kernel_sgemm_tall", "kernel_sgemm_wide", "kernel_sgemm_huge", "abft_baseline",
                            "abft_kernel_medium", "abft_kernel_large", "abft_kernel_tall", "abft_kernel_wide",
                            "abft_kernel_huge", "thread_abft_kernel", "warp_abft_kernel", "abft_kernel_huge_workspace",
                            "abft_kernel_large_workspace", "abft_kernel_wide_workspace",
                            "hpcdnn_sgemm_column_major", "abft_kernel_huge_column_major"]
    # the thread-level series keeps its name and is empty: matrix cores have no per-thread accumulator tile
    assert series.pop("thread_abft_kernel") == ""
    for name, body in series.items():
        vals = _floats(body)
        assert len(vals) == 3 and all(v > 0 for v in vals), (name, body)
    # a sub-range of series, as the reference's <st_kernel> <end_kernel> arguments select
    out = _run("ft_sgemm", 256, 256, 256, 10, 16)
    assert re.findall(r"^(\w+) = th", out, flags=re.M) == ["abft_baseline", "abft_kernel_medium", "abft_kernel_large",
                                                                "abft_kernel_tall", "abft_kernel_wide", "abft_kernel_huge"]


def test_sgemm_rows():
    lines = _run("sgemm", 512, 1024, 512).splitlines()
    assert lines[0] == "     512|    1024|"
    assert _floats(lines[1]) == [157300.0, 157300.0]
    vals = _floats(lines[2])
    assert len(vals) == 2 and all(0 < v < 157300.0 for v in vals)


@pytest.mark.parametrize("which", ["saxpy", "sdot"])
def test_vector_rows(which):
    lines = _run(which, 14).splitlines()
    assert lines[0] == "".join(f"{e:8d}|" for e in range(10, 15))
    vals = _floats(lines[1])
    assert len(vals) == 5 and all(v > 0 for v in vals)


def test_usage_on_bad_arguments():
    p = subprocess.run([BIN, "sgemm", "0", "10"], capture_output=True, text=True, timeout=30)
    assert p.returncode == 2 and "usage" in p.stderr
