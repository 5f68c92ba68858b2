import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "bi-kv_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lib():
    """The built HIP library. Built once if missing; never replaced by a fallback."""
    import __graft_entry__ as entry
    entry.ensure_built()
    from bikv_pagecopy import _lib
    return _lib.load()


@pytest.fixture(scope="session")
def oracle():
    from oracle import pagecopy_oracle
    pagecopy_oracle.clib()
    return pagecopy_oracle


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this process")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _default_tuning_after_each_test():
    """Launch knobs are process-wide: a test that changes them (and then fails before putting them
    back) must not leak its settings into the tests that follow."""
    yield
    from bikv_pagecopy import _lib
    if _lib._lib is not None:
        _lib.reset_tuning()
