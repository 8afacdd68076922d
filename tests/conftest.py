import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu():
    """The CUDA/HIP device, or skip.  GPU tests also require the built kernel library: a missing
    library is a failure on a GPU box, never a silent fallback."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    from triton_amd import _lib

    _lib.load()  # raises ImportError if the HIP library has not been built
    assert _lib.load().mi355_query(_lib.Q_IS_GFX950) == 1, "these kernels are gfx950-only"
    return torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def _library_rereads_environment():
    """Autouse fixtures are set up first and torn down last: after monkeypatch has restored the MI355_*
    variables a test changed (util.set_knob), the library (if built and loaded) reads them again."""
    yield
    from triton_amd import _lib

    if _lib._lib is not None:
        _lib._lib.mi355_refresh_env()
