import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


# Oracle parity of the core path first; the cases that depend most on the box
# (worker processes, concurrency, native programs) last, and the entry point that
# allocates nothing after everything else.  Files not named here keep their
# alphabetical place between the two groups.
_FIRST = ["test_oracle", "test_golden", "test_transfer_gpu", "test_ce_analysis", "test_ce_gpu",
          "test_staging_gpu", "test_groups_gpu", "test_multi_group_gpu", "test_layout_transform",
          "test_full_size_gpu"]
_LAST = ["test_worker_gpu", "test_concurrency_gpu", "test_native_abi_gpu", "test_zz_no_alloc"]


def pytest_collection_modifyitems(session, config, items):
    def rank(item):
        name = os.path.splitext(os.path.basename(str(item.fspath)))[0]
        if name in _FIRST:
            return (0, _FIRST.index(name))
        if name in _LAST:
            return (2, _LAST.index(name))
        return (1, 0)
    items.sort(key=rank)  # stable: the order inside a file stays


@pytest.fixture(scope="session", autouse=True)
def _oracle_built():
    from oracle import fkv_oracle
    fkv_oracle.build()
    yield


@pytest.fixture(scope="session")
def gpu_device():
    import torch
    if not torch.cuda.is_available():
        pytest.fail("a test marked gpu ran without a GPU")
    return "cuda:0"
