"""Shared fixtures. GPU tests are marked `gpu`; everything else runs on the CPU."""
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """Without a GPU, skip gpu-marked tests instead of failing them."""
    try:
        import torch
        have = torch.cuda.is_available()
    except Exception:
        have = False
    if have:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for it in items:
        if "gpu" in it.keywords:
            it.add_marker(skip)


@pytest.fixture(scope="session")
def orc():
    from oracle import binding
    if not os.path.exists(binding.ORACLE_SO):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "libqlm_oracle.so"])
    return binding.Oracle()


@pytest.fixture(scope="session")
def ref():
    """The reference's own CPU backend; only present where it was built from the reference."""
    from oracle import binding
    if not binding.have_ref():
        pytest.skip("oracle/_ref not built (reference sources not mounted)")
    return binding.Ref()


def load_golden(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False)


@pytest.fixture(scope="session")
def golden():
    return load_golden
