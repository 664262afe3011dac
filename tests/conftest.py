import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
# the library's split-K test hooks (bfaintb_debug_control: withheld partial sums, the wait's limit) only work in a
# process that asks for them before the library reads its environment
os.environ.setdefault("BFAINTB_TEST_HOOKS", "1")
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir():
    return os.path.join(ROOT, "tests", "golden")


def pytest_sessionfinish(session, exitstatus):
    """After a GPU session: what the acceptance checks found (outputs outside the 2-ULP bound per call), for the report."""
    import json
    try:
        import helpers
    except ImportError:
        return
    if not helpers.ACCEPTANCE_LOG:
        return
    out = os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "acceptance_counts.json"), "w") as f:
            json.dump(helpers.ACCEPTANCE_LOG, f, indent=0)
    except OSError:
        pass
