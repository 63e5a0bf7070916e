import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    # Load what is built; build only when nothing is there (hipcc cross-compiles without a GPU).
    # A missing library is an error, never a reason to skip or to fall back.
    from dopt_amd import build as hip_build
    if not os.path.exists(hip_build.LIB_PATH):
        hip_build.build()
    import oracle
    oracle.build()          # no-op when liboracle.so exists


@pytest.fixture(scope="session")
def kats():
    with open(os.path.join(ROOT, "tests", "golden", "reference_kats.json")) as f:
        return json.load(f)


def pytest_sessionfinish(session, exitstatus):
    """The configuration tests record the largest error they saw per quantity; the table is written to the directory
    DOPT_TEST_REPORT_DIR names (nothing is written when it is not set)."""
    try:
        import util
    except ImportError:
        return
    out_dir = os.environ.get("DOPT_TEST_REPORT_DIR", "")
    if not util.ERROR_ROWS or not out_dir or not os.path.isdir(out_dir):
        return
    with open(os.path.join(out_dir, "parity_errors.txt"), "w") as f:
        f.write("%-34s %-40s %12s %14s %12s\n" % ("case", "quantity", "max|err|", "err/(a+r|w|)", "max|want|"))
        for case, what, err, ratio, mag in util.ERROR_ROWS:
            f.write("%-34s %-40s %12.3e %14.3f %12.3e\n" % (case, what, err, ratio, mag))
