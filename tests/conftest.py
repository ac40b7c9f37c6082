import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _have_gpu() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _have_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def native_libs():
    """The in-tree HIP libraries; built on first use only if nothing is built yet."""
    from raf_amd import _lib, build

    if not _lib.OPTIM_LIB.exists() or not _lib.DIALECT_LIB.exists() or not _lib.GLUE_LIB.exists():
        build.build_all()
    return _lib


@pytest.fixture(scope="session")
def c_oracle():
    from oracle import c_oracle as co

    co.build()
    return co
