import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def rt():
    """One runtime context on cuda:0 for the GPU tests; fails loudly if the HIP library is missing."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    from sofie_amd import Runtime
    r = Runtime(0)
    yield r
    r.close()


@pytest.fixture
def opt(rt):
    """opt(name, value) sets a kernel-choice override on the shared context (sofie_hip_ctx_set_option); the defaults are put
    back when the test ends."""
    defaults = {"swizzle": 4, "i8_tile": 0, "f8_tile": 0, "gemm_variant": 0, "conv_explicit": 0, "f32_skinny": -1, "f32_chain": -1}
    touched = []

    def set_option(name, value):
        rt.set_option(name, value)
        touched.append(name)
    yield set_option
    for name in touched:
        rt.set_option(name, defaults[name])


@pytest.fixture(scope="session", autouse=True)
def _torch_initialises_the_gpu_first(request):
    """torch brings its own copy of the HIP runtime: whichever of torch and libsofie_hip.so touches the GPU first decides which copy the process uses.
    The GPU tests share device memory between the two, so torch goes first whatever test file happens to run first."""
    if any(item.get_closest_marker("gpu") for item in request.session.items):
        import torch
        if torch.cuda.is_available():
            torch.cuda.init()
    yield
