"""The reference's C++ call sites re-targeted at libflashMoe.so (tests/cpp):
the API test runs anywhere; the end-to-end test and the benchmark need the GPU."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "bin")


def _run(name, timeout):
    exe = os.path.join(BIN, name)
    if not os.path.exists(exe):
        pytest.fail("%s is not built: run `make -C tests/cpp` (or __graft_entry__.build())" % exe)
    p = subprocess.run([exe], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True,
                       timeout=timeout)
    print(p.stdout)
    assert p.returncode == 0, p.stdout[-2000:]
    return p.stdout


def test_moe_api_test():
    out = _run("moeApiTest", 60)
    assert "0 failed" in out


@pytest.mark.gpu
def test_moe_test():
    out = _run("moeTest", 300)
    assert "2 tests, 0 failed" in out


@pytest.mark.gpu
def test_moe_kernel_benchmark():
    out = _run("moeKernelBenchmark", 300)
    assert out.count("Moe kernel avg time for num of tokens") == 9
