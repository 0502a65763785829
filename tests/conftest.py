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


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")
