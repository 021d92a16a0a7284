import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "accelerate-cuda_amd"), os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


@pytest.fixture
def tuned(A, ctx):
    """tuned("name=value,..."): tuning knobs for the instances the test creates from then on in `ctx` (and for
    previews), put back when the test ends.  Nothing touches the environment."""
    stack = []

    def set_knobs(text):
        t = A.tuning(text, ctx)
        t.__enter__()
        stack.append(t)
    yield set_knobs
    for t in reversed(stack):
        t.__exit__()


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.build()
    return oracle
