import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "oracle")):
    if p not in sys.path:
        sys.path.insert(0, p)


# every segment reduction that goes through pytorch_scatter_amd.capi also checks its status word
os.environ.setdefault("TS_CHECK_STATUS", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import ts_oracle
    ts_oracle.lib()
    return ts_oracle


@pytest.fixture(scope="session")
def ref_ops():
    """The reference's own CPU kernels (oracle/_ref), or skip when not built."""
    import torch
    path = os.path.join(ROOT, "oracle", "_ref", "libts_ref_cpu.so")
    if not os.path.exists(path):
        pytest.skip("oracle/_ref not built (reference tree absent)")
    torch.ops.load_library(path)
    return torch.ops.ts_ref
