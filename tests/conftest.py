import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_present() -> bool:
    return os.path.exists("/dev/kfd")


def pytest_collection_modifyitems(config, items):
    # A GPU test on a box without a GPU is skipped rather than failed; on a GPU box a
    # missing library is a hard error (see h100_gemm_amd._lib.load).
    if _gpu_present():
        return
    skip = pytest.mark.skip(reason="no GPU device (/dev/kfd) in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.lib()
    return oracle


@pytest.fixture(scope="session")
def mi():
    import __graft_entry__
    __graft_entry__.ensure_built()      # uses what is built; compiles only if nothing is
    import h100_gemm_amd
    h100_gemm_amd._lib.load()
    return h100_gemm_amd
