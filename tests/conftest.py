import pathlib
import sys

import pytest
import torch

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X; run with `-m gpu` on the GPU box")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def library():
    """The built kernel library; built once here only if nothing is built yet."""
    from fast_llm_amd import _lib

    if not _lib.LIBRARY_PATH.is_file():
        from fast_llm_amd.build import build_library

        build_library()
    return _lib.lib()


@pytest.fixture(scope="session")
def device(library):
    return torch.device("cuda:0")
