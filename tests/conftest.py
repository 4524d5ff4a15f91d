import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


COMPILE_ONLY = os.environ.get("FT_TESTS_COMPILE_ONLY") == "1"


@pytest.fixture(autouse=True)
def _compile_only(monkeypatch):
    """FT_TESTS_COMPILE_ONLY=1: run the GPU tests on a machine without a GPU
    up to the point where a plan would be loaded, compile the plan's kernels
    into the on-disk cache instead, and skip the rest of the test. This is how
    the kernels the GPU tests use are built ahead of time."""
    if not COMPILE_ONLY:
        yield
        return
    from flextensor_amd import plan as plan_mod

    def compile_and_skip(self, plan, **kwargs):
        plan.compile()
        pytest.skip("kernels compiled")

    monkeypatch.setattr(plan_mod.BuiltPlan, "__init__", compile_and_skip)
    yield


@pytest.hookimpl(hookwrapper=True)
def pytest_runtest_call(item):
    outcome = yield
    if COMPILE_ONLY and outcome.excinfo is not None \
            and not issubclass(outcome.excinfo[0], pytest.skip.Exception):
        # without a device a test that touches it before building a plan cannot go on;
        # any other error (a config the templates reject, a compile error) stays an error
        text = repr(outcome.excinfo[1])
        if any(k in text for k in ("No HIP GPUs", "no GPU", "hipErrorNoDevice", "no ROCm-capable", "Found no NVIDIA")):
            outcome.force_exception(pytest.skip.Exception("needs a device: %s" % text[:200]))
