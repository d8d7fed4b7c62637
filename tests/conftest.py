"""Shared fixtures.  `-m "not gpu"` runs on CPU only; `-m gpu` needs an MI355X."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))
sys.path.insert(0, os.path.join(ROOT, "cuda-cnn-gan-vae_amd"))
sys.path.insert(0, ROOT)

import oracle_api  # noqa: E402  (test infrastructure: the CPU checker)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    if not oracle_api.available("oracle"):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    return oracle_api.Oracle("oracle")


@pytest.fixture(scope="session")
def ref():
    """The reference's own CPU headers, compiled in the authoring container (absent elsewhere -> skip)."""
    if not oracle_api.available("ref"):
        pytest.skip("oracle/_ref/libtensor_ref.so not built (needs /root/reference)")
    return oracle_api.Oracle("ref")


@pytest.fixture(scope="session")
def kat():
    return json.load(open(os.path.join(ROOT, "tests", "golden", "ctensortest_kat.json")))


@pytest.fixture(scope="session")
def golden():
    return np.load(os.path.join(ROOT, "tests", "golden", "ref_vectors.npz"))


def rel_err(got, want):
    """max|got-want| / max|want| per tensor -- the parity metric for fp32 results."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    scale = np.max(np.abs(want))
    return float(np.max(np.abs(got - want)) / (scale if scale > 0 else 1.0))
