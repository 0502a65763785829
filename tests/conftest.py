import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for extra in (os.path.join(ROOT, "fasttree-artifact_amd"), os.path.join(ROOT, "tests", "golden"),
              os.path.join(ROOT, "oracle"), os.path.join(ROOT, "tests"), ROOT):
    if extra not in sys.path:
        sys.path.insert(0, extra)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    if os.environ.get("PYTEST_XDIST_WORKER"):
        # several workers, each with a thread per core for torch's CPU kernels, spend their time waiting on
        # one another (the oracle's small matrix products then take minutes instead of seconds)
        import torch

        torch.set_num_threads(max(1, (os.cpu_count() or 2) // max(1, int(os.environ.get("PYTEST_XDIST_WORKER_COUNT", "4")))))


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")
