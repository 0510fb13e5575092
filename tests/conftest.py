import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


@pytest.fixture(scope="session")
def ct():
    """The ctypes binding of the C-ABI library (built in tree; never a fallback)."""
    import __graft_entry__ as entry

    return entry.load_package()


@pytest.fixture(scope="session")
def oracle():
    import oracle as o

    return o


@pytest.fixture()
def fake_hip():
    """A binding of the TESTING library (the product library's objects plus the recording stand-in for the HIP
    runtime), routed to that stand-in for one test."""
    import __graft_entry__ as entry

    ct = entry.load_package(testing=True)
    ct.check(ct.lib().cutile_testing_use_fake_hip(1))
    ct.lib().cutile_testing_clear_log()
    ct.tuning_reload("")            # the variant choices asserted on this runtime are the table's own, not a record's
    yield ct
    ct.tuning_reload(None)
    ct.check(ct.lib().cutile_testing_use_real_hip())


@pytest.fixture(scope="session")
def dev():
    import torch

    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return torch.device("cuda:0")
