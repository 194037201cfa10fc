import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (MI355X); run with -m gpu")


def pytest_collection_modifyitems(config, items):
    import torch

    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session", autouse=True)
def _library_is_built():
    """The tests load the library that is built; only when none is there (a fresh checkout) they build
    it first.  The product itself never builds or falls back: kfold_amd._lib raises if the file is
    missing."""
    from kfold_amd import _lib

    if not _lib.LIB_PATH.exists():
        import shutil

        from kfold_amd import build

        if shutil.which(build.HIPCC) is None and not os.path.exists(build.HIPCC):
            pytest.exit(f"{_lib.LIB_PATH} is not built and {build.HIPCC} is not available", returncode=2)
        build.build()
    yield
