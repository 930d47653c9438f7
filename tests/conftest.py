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
    from oracle.oracle import Oracle
    return Oracle(fast=False)


@pytest.fixture(scope="session")
def oracle_fast():
    from oracle.oracle import Oracle
    return Oracle(fast=True)


def pytest_sessionfinish(session, exitstatus):
    """Writes the parity errors the GPU tests measured (tests/helpers.py: MEASURED) to
    parity_measured.json in $SB_PARITY_OUT, when that names a directory."""
    import json
    out = os.environ.get("SB_PARITY_OUT")
    try:
        from helpers import MEASURED
    except ImportError:
        try:
            from tests.helpers import MEASURED
        except ImportError:
            return
    if out and os.path.isdir(out) and MEASURED:
        with open(os.path.join(out, "parity_measured.json"), "w") as f:
            json.dump(MEASURED, f, indent=0)
