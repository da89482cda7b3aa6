import os
import sys

import zlib

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as ge  # noqa: E402

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (test infrastructure)."""
    return ge.load_oracle()


@pytest.fixture(scope="session")
def pkg():
    """ctypes bindings of the product libraries; builds them if absent."""
    p = ge.load_package()
    if not p.is_built():
        p.build(force=False)
    return p


@pytest.fixture(scope="session")
def gpu(pkg):
    """torch device + initialised kernel library; the product path has no CPU
    fallback, so a GPU test on a box without a GPU is an error, not a skip."""
    import torch
    assert torch.cuda.is_available(), "gpu-marked test started without a GPU"
    pkg.ops()  # mgpuOpsInit
    return torch.device("cuda:0")


@pytest.fixture
def rng(request):
    # one independent, reproducible stream per test
    seed = zlib.crc32(request.node.nodeid.encode())  # str hashes change from run to run
    return np.random.Generator(np.random.PCG64(20240 + (seed % 1000)))


def to_dev(a, dev):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).to(dev)
