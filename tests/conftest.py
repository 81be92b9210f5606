import importlib.util
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "abq-llm_amd")
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def load_abq_gemm():
    """The package directory name is not a Python identifier, so load the binding by path."""
    if "abq_gemm" in sys.modules:
        return sys.modules["abq_gemm"]
    spec = importlib.util.spec_from_file_location("abq_gemm", os.path.join(PKG, "abq_gemm.py"))
    mod = importlib.util.module_from_spec(spec)
    sys.modules["abq_gemm"] = mod
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="session")
def abq():
    return load_abq_gemm()


@pytest.fixture(scope="session")
def oracle():
    from oracle import abq_oracle
    abq_oracle.build()
    return abq_oracle
