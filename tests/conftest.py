import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "mlu-ops_amd", "python"), os.path.join(ROOT, "oracle"),
          os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gpu_handle():
    import torch
    import mluop_hip
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    torch.cuda.set_device(0)
    # every output tensor and workspace the wrappers allocate sits between 4 KiB guard bands,
    # checked after each operator call (the reference's test runner: pb_gtest/src/runtime.cpp:99-145)
    mluop_hip.GUARD_BYTES = 4096
    h = mluop_hip.make_handle_on_current_stream()
    yield h
    torch.cuda.synchronize()
    h.close()
