import importlib
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    """The product package (its directory name is not a Python identifier).  The tests load what is built;
    only when nothing is built do they run the build first."""
    import __graft_entry__
    __graft_entry__.ensure_built()
    return importlib.import_module("torch-hipress-extension_amd")


@pytest.fixture(scope="session")
def capi(pkg):
    pkg._capi.load()
    return pkg._capi


@pytest.fixture(scope="session")
def hp_cuda_compiled(pkg):
    """The compiled torch extension `hp_cuda` (csrc/hp_cuda_module.cpp), imported by its top-level name as
    a caller of the reference's extension would; it must have been built (make -C csrc)."""
    import torch  # noqa: F401  (the extension links libtorch)
    ext_dir = os.path.join(os.path.dirname(pkg.__file__), "ext")
    if ext_dir not in sys.path:
        sys.path.insert(0, ext_dir)
    return importlib.import_module("hp_cuda")


@pytest.fixture(scope="session")
def oracle_cpu():
    from oracle import cpu
    cpu.lib()
    return cpu
