import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionfinish(session, exitstatus):
    import parity
    parity.write_report(ROOT)


@pytest.fixture(scope="session")
def rt():
    """Stream + handles shared by the GPU tests (one set per process)."""
    from tinyflow_amd import gpu_op, ndarray

    class RT:
        pass

    r = RT()
    r.ctx = ndarray.gpu(0)
    r.stream = gpu_op.create_cudaStream()
    r.cudnn = gpu_op.create_cudnnHandle(r.stream)
    r.cublas = gpu_op.create_cublasHandle(r.stream)
    return r
