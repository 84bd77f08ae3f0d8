import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import deepbind_oracle
    return deepbind_oracle


def pytest_terminal_summary(terminalreporter):
    """Worst elementwise relative error per benchmark configuration, as recorded by the GPU parity tests."""
    try:
        from tests import gpu_util
    except Exception:
        return
    if not gpu_util.REPORT:
        return
    import json
    tr = terminalreporter
    tr.write_line("")
    tr.write_line("parity: worst elementwise relative error, |got-ref| / max(|ref|, %g x block max); share = elements within tol with no floor"
                  % gpu_util.FLOOR_FRAC)
    rows = {}
    for (config, kind), e in sorted(gpu_util.REPORT.items()):
        tr.write_line("parity: %-34s %-12s worst %.2e (tol %.0e)  share %.4f  n=%d"
                      % (config, kind, e["worst_rel_err"], e["tol"], e["share_within"], e["elements"]))
        rows["%s/%s" % (config, kind)] = e
    out = os.path.join(ROOT, "gpurun_out")
    if os.path.isdir(out):
        with open(os.path.join(out, "parity_elementwise.json"), "w") as f:
            json.dump(rows, f, indent=1, sort_keys=True)
