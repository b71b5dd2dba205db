import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def gpu_ctx():
    """One device context for the whole GPU session; fails loudly if the HIP library or the
    GPU is missing (there is no CPU fallback to hide behind)."""
    from accelerate_amd import hip
    ctx = hip.Context(0)
    yield ctx
    ctx.close()


@pytest.fixture(scope="session")
def cc_ctx():
    """Compile-only context: code generation + hipRTC for gfx950, no GPU needed."""
    from accelerate_amd import hip
    ctx = hip.Context(-1)
    yield ctx
    ctx.close()


@pytest.fixture
def knobs(gpu_ctx):
    """knobs(name, value) overrides one launch-time choice of the session's context for the
    duration of the test."""
    before = {}

    def put(name, value):
        old = gpu_ctx.set_knob(name, value)
        before.setdefault(name, old)

    yield put
    for name, old in before.items():
        gpu_ctx.set_knob(name, old)
