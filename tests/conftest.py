import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an AMD GPU (run on the MI355X box)")


def pytest_sessionfinish(session, exitstatus):
    """Writes the parity margins that tests.helpers.assert_close collected (one record per compared tensor) to the
    file named by BIMAMBA2_PARITY_MARGINS, if that variable is set."""
    path = os.environ.get("BIMAMBA2_PARITY_MARGINS")
    if not path:
        return
    import json
    from tests import helpers
    with open(path, "w") as f:
        json.dump(helpers.MARGINS, f)
