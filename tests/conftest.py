import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "triton-distributed_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    from triton_dist import _lib
    _lib.check(_lib.load().tdist_init())  # fails loudly if the HIP library is missing or the GPU is not gfx950
    return torch.device("cuda", 0)


def announce(msg):
    """Print and flush the case about to touch the GPU, so that a fault names its test."""
    print("[gpu-case] " + msg, flush=True)


@pytest.fixture
def switches():
    """``switches(key, value)`` sets one of the library's test and measurement switches (tdist_debug_set; None = the
    library decides again); all of them are put back when the test ends, after the GPU has drained."""
    from triton_dist import _lib
    lib = _lib.load()
    saved = {}

    def set_switch(key, value):
        saved.setdefault(key, lib.tdist_debug_get(key))
        _lib.check(lib.tdist_debug_set(key, -1 if value is None else int(value)))

    yield set_switch
    try:
        import torch
        if torch.cuda.is_available():
            torch.cuda.synchronize()
    finally:
        for key, old in saved.items():
            lib.tdist_debug_set(key, old)
