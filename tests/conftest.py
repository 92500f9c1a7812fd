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
    from tests import oracle_api
    return oracle_api.load_oracle()


@pytest.fixture(scope="session")
def hq():
    """The product package on a GPU box; fails loudly if libhq.so is missing."""
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    import hecbench_amd
    hecbench_amd.init()
    return hecbench_amd


@pytest.fixture
def tunable():
    """Sets launch-shape knobs of the library through hq_set_tunable and clears them afterwards."""
    from hecbench_amd import _lib
    lib = _lib.load()
    touched = []

    def set_(name, value):
        rc = lib.hq_set_tunable(name.encode(), int(value), 0)
        assert rc == 0, (name, rc)
        touched.append(name)

    yield set_
    for name in touched:
        lib.hq_set_tunable(name.encode(), 0, 1)
