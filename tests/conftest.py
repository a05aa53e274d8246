import os
import sys

import pytest

REPO_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if REPO_ROOT not in sys.path:
    sys.path.insert(0, REPO_ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # load what is built; compile only if the library is missing altogether
    from lmserve_amd.build import ensure_built
    ensure_built()


@pytest.fixture(scope="session")
def gpu():
    """The CUDA/HIP device the GPU tests run on; they fail (not skip) without one,
    and without the built HIP library."""
    import torch
    from lmserve_amd import _lib

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    _lib.lib()  # raises if libkvcache.so is not built
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def default_tuning(request):
    """Every test starts and ends with the library's launch-shape knobs at their
    defaults, whatever an earlier test set. Tests that never load the library
    (oracle pinning, host logic) run without it."""
    from lmserve_amd import _lib

    try:
        L = _lib.lib()
    except _lib.KVCacheLibraryError:
        if request.node.get_closest_marker("gpu") is not None:
            raise
        yield
        return
    assert L.kvc_tuning_modified() == 0, "a tuning knob was left modified by an earlier test"
    yield
    _lib.reset_tuning()
