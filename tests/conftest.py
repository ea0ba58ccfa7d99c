import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

entry.load_package()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    """The CPU oracle (checker only)."""
    return entry.load_oracle()


@pytest.fixture(scope="session")
def hip():
    from ttmlir_amd import hip as h
    h.lib()  # raises if the native library is missing: no fallback
    # a kernel that runs past a buffer faults the whole device: every pointer a test hands over is checked against the
    # extent the kernels touch before the call goes out
    h.check_buffers(True)
    return h


@pytest.fixture(scope="session")
def dev():
    import torch
    if os.environ.get("TTMLIR_AMD_NULL_DEVICE") == "1":
        # the host runtime over tests/cpp/null_device.cpp (tests/test_null_device.py): programs run on the CPU, every launch
        # is held against the extents of its buffers, results are meaningless
        return torch.device("cpu")
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")
