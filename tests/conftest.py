import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc
    orc.build()
    return orc


@pytest.fixture(scope="session")
def gpu():
    """torch + the C-ABI library, all launches on one non-default torch stream."""
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from weed_amd import capi
    lib = capi.load()  # raises if libweed_hip.so has not been built: no CPU fallback
    capi.check(lib.weed_hip_init(0))
    stream = torch.cuda.Stream()
    capi.use_torch_stream(stream)
    ctx = torch.cuda.stream(stream)
    ctx.__enter__()
    yield capi
    capi.sync()
    ctx.__exit__(None, None, None)
