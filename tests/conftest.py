import ctypes
import os
import subprocess
import sys

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(REPO, "sparse-quant_amd")
for p in (PKG, os.path.join(REPO, "oracle"), REPO):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _gpu_available():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle_c():
    """The C restatement of the oracle, built on first use (gcc, < 1 s)."""
    so = os.path.join(REPO, "oracle", "build", "libw4a16_oracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", os.path.join(REPO, "oracle")])
    lib = ctypes.CDLL(so)
    lib.sq_oracle_h2f.restype = ctypes.c_float
    lib.sq_oracle_h2f.argtypes = [ctypes.c_uint16]
    lib.sq_oracle_f2h.restype = ctypes.c_uint16
    lib.sq_oracle_f2h.argtypes = [ctypes.c_float]
    return lib


@pytest.fixture(scope="session")
def built_lib():
    """Path of libsq_w4a16.so; the tests never build it themselves on the GPU box."""
    so = os.path.join(PKG, "libsq_w4a16.so")
    if not os.path.exists(so):
        if _gpu_available():
            pytest.fail("libsq_w4a16.so is not built; run __graft_entry__.build() first")
        sys.path.insert(0, PKG)
        from sqamd import build
        build.build_lib(verbose=False)
    return so
