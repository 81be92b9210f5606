"""The C++ face of the library (engine/ shim headers, libabq_engine.a, ABQGEMMWrapper) and the
autotune harness, run as the prebuilt binaries under abq-llm_amd/build/."""
import os
import re
import subprocess

import pytest

from conftest import PKG

API_TEST = os.path.join(PKG, "build", "test_engine_api")
HARNESS = os.path.join(PKG, "build", "test_any_mma")


def _need(path):
    if not os.path.exists(path):
        pytest.fail("%s is not built: run `make -C abq-llm_amd` (or __graft_entry__.build())" % path)


def test_engine_api_host_error_paths():
    _need(API_TEST)
    out = subprocess.run([API_TEST, "--no-gpu"], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "PASSED" in out.stdout
    assert "[ABQ][Error] unsupport K = 100" in out.stdout  # message of abq_gemm_wrapper.cu:101


def test_harness_usage_and_k_check():
    _need(HARNESS)
    out = subprocess.run([HARNESS], capture_output=True, text=True, timeout=60)
    assert out.returncode != 0 and "Usage: ./test_any_mma M N K X_BITS W_BITS SIGNED" in out.stdout
    out = subprocess.run([HARNESS, "1", "64", "100", "8", "2", "1"], capture_output=True, text=True, timeout=60)
    assert out.returncode != 0 and "k must >= 128" in out.stdout


@pytest.mark.gpu
def test_engine_api_on_gpu():
    _need(API_TEST)
    out = subprocess.run([API_TEST], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "PASSED (0 failed checks)" in out.stdout


@pytest.mark.gpu
@pytest.mark.parametrize("args", [["4", "512", "1024", "8", "2", "1"], ["64", "384", "512", "4", "4", "0"]])
def test_autotune_harness_checks_every_config(args):
    _need(HARNESS)
    out = subprocess.run([HARNESS] + args + ["--repeat", "20", "--rotate-mib", "8"], capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    lines = [l for l in out.stdout.splitlines() if l.startswith("gfx950 ")]
    assert len(lines) >= 20
    assert all(l.split("|")[2].strip() == "PASSED" for l in lines), out.stdout
    m = re.search(r"The best kernel config is ([\d, ]+) with ([\d.]+) TOPS", out.stdout)
    assert m and float(m.group(2)) > 0
