import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# Engines whose step kernels write every slot of the result themselves (no fill of the result
# before a pass) first set the result to a value that is neither a vertex nor INVALID: a slot no
# kernel wrote then differs from the oracle instead of holding what an earlier pass left there.
os.environ.setdefault("ND_MARK_UNWRITTEN", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from tests import oracle_binding
    return oracle_binding
