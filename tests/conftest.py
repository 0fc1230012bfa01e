"""Shared pytest set-up: import paths, the ``gpu`` marker, oracle fixtures."""

import os
import sys
from pathlib import Path

import pytest

# PyTorch-ROCm bundles its own copy of the HIP runtime.  Two copies in one
# process cannot both initialise the device, so torch (used by the GPU tests
# for device memory) is loaded before anything pulls in libkge_hip.so, which
# then binds to the copy already present.
import torch  # noqa: F401,E402

ROOT = Path(__file__).resolve().parent.parent
PKG = ROOT / "distributed-kge-poplar_amd"
for p in (ROOT, PKG, ROOT / "tests"):
    if os.fspath(p) not in sys.path:
        sys.path.insert(0, os.fspath(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle64():
    from oracle.kge_oracle import Oracle

    return Oracle("f64")


@pytest.fixture(scope="session")
def oracle32():
    from oracle.kge_oracle import Oracle

    return Oracle("f32")
