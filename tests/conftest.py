import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests", "golden")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


def pytest_collection_modifyitems(config, items):
    """Operator parity first, whole-model tests last: the runs that stop at the first failure (`-x`) then report on
    the kernels before a failure of the much larger model tests (several GB of weights, Hugging Face's own eager
    modules beside ours) can hide them.  The order inside a file is kept."""
    rank = {"test_capi_cpu.py": 0, "test_oracle.py": 0, "test_deal_cpu.py": 0, "test_index_gpu.py": 1,
            "test_ops_gpu.py": 2, "test_full_size_gpu.py": 3, "test_model.py": 4}
    items.sort(key=lambda it: rank.get(os.path.basename(str(it.fspath)), 3))
