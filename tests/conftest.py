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
    if not (gpu_util.REPORT or gpu_util.VS_F32 or gpu_util.ARGMAX):
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
    if gpu_util.VS_F32:
        tr.write_line("parity: distance from the float64 result relative to the block's largest value: HIP float32 next to the oracle "
                      "run in float32 in reference order (asserted: HIP <= %g x max(f32 reference, 2^-22))" % gpu_util.C_F32)
        for (config, kind), e in sorted(gpu_util.VS_F32.items()):
            tr.write_line("parity: %-34s %-12s HIP %.2e  f32 reference %.2e  worst ratio %.2f  blocks=%d"
                          % (config, kind, e["hip_err"], e["f32_ref_err"], e["worst_ratio"], e["blocks"]))
            rows["vs_f32/%s/%s" % (config, kind)] = e
    for config, e in sorted(gpu_util.ARGMAX.items()):
        tr.write_line("parity: %-34s argmax moved vs float32 reference order: %d of %d" % (config, e["moved"], e["total"]))
        rows["argmax/%s" % config] = e
    out = os.path.join(ROOT, "gpurun_out")
    if os.path.isdir(out):
        with open(os.path.join(out, "parity_elementwise.json"), "w") as f:
            json.dump(rows, f, indent=1, sort_keys=True)
