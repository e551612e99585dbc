import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def pytest_terminal_summary(terminalreporter):
    """Strict parameter metrics of the fp32-parameter comparisons, worst case per test:
    max |dev - ref| / |ref| over all elements, how many elements exceed 1e-6, the same ratio
    over the elements whose parameter is at least as large as its step (asserted <= 1e-6),
    the error in ulps of the step over the others, and the absolute tolerance that would make
    |dev - ref| <= atol + 1e-6 * |ref| hold everywhere."""
    try:
        from tests.q4_testlib import STRICT_LOG
    except Exception:
        return
    if not STRICT_LOG:
        return
    agg = {}
    for label, m in STRICT_LOG:
        a = agg.setdefault(label, dict(n=0, max_rel=0.0, above=0, dom=0.0, step_ulps=0.0, atol=0.0, calls=0))
        a["n"] += m["n"]
        a["above"] += m["above"]
        a["calls"] += 1
        for k in ("max_rel", "dom", "step_ulps", "atol"):
            a[k] = max(a[k], m[k])
    tr = terminalreporter
    tr.write_sep("=", "strict fp32 parameter metrics (one step from identical inputs)")
    tr.write_line(f"{'elements':>14} {'max rel':>10} {'> 1e-6':>10} {'frac':>9} {'max rel, |p|>=|step|':>21} "
                  f"{'step ulps, else':>16} {'atol@rtol1e-6':>14}  test")
    tot = dict(n=0, above=0, max_rel=0.0, dom=0.0, step_ulps=0.0, atol=0.0)
    for label, a in agg.items():
        tr.write_line(f"{a['n']:>14d} {a['max_rel']:>10.3g} {a['above']:>10d} {a['above'] / max(a['n'], 1):>9.2e} "
                      f"{a['dom']:>21.3g} {a['step_ulps']:>16.2f} {a['atol']:>14.3g}  {label}")
        tot["n"] += a["n"]
        tot["above"] += a["above"]
        for k in ("max_rel", "dom", "step_ulps", "atol"):
            tot[k] = max(tot[k], a[k])
    tr.write_line(f"{tot['n']:>14d} {tot['max_rel']:>10.3g} {tot['above']:>10d} {tot['above'] / max(tot['n'], 1):>9.2e} "
                  f"{tot['dom']:>21.3g} {tot['step_ulps']:>16.2f} {tot['atol']:>14.3g}  ALL")
