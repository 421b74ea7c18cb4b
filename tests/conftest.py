import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


# A chain compiled at run time that needs scratch memory (a per-thread array the optimiser could not keep in registers: an
# order of magnitude slower, silently) is refused during the tests, like the ahead-of-time build refuses it; the reference's
# programs that tests/test_gpu_reference_programs.py starts inherit the setting.
os.environ.setdefault("FKLHIP_JIT_STRICT", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("GPU test collected on a machine without a GPU; run with -m 'not gpu'")
    return torch.device("cuda:0")
