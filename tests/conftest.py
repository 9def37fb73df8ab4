import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# Order of the GPU run.  `pytest -x` stops at the first failure, so the parity tests of the five
# configurations come first, then the other bit-exactness / oracle tests, then everything that
# launches whole benchmark runs or times kernels (those only report what they measure), and the
# entry point that allocates nothing last.  Files not listed keep their alphabetical place in the
# middle group.
FIRST = ("test_gpu_pairs.py", "test_gpu_small.py", "test_gpu_models.py", "test_gpu_general.py", "test_gpu_batch.py", "test_gpu_layout.py",
         "test_gpu_multi.py", "test_gpu_frontend.py", "test_gpu_sync_giveup.py", "test_gpu_built_pairs.py", "test_gpu_built_operators.py")
LATE = ("test_gpu_driver.py", "test_gpu_suite.py", "test_gpu_rt_plan.py", "test_bench_contract.py")
LAST = ("test_zz_no_alloc.py",)


def _rank(item):
    name = os.path.basename(str(item.fspath))
    if name in FIRST:
        return (0, FIRST.index(name))
    if name in LATE:
        return (2, LATE.index(name))
    if name in LAST:
        return (3, LAST.index(name))
    return (1, 0)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(session, config, items):
    items.sort(key=_rank)          # stable: the order inside a file and inside a group is kept


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")
