import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session", autouse=True)
def _oracle_threads():
    """The oracle is bit-identical for any thread count; use the cores we have for speed."""
    from oracle import cpu_ref
    cpu_ref.set_threads(min(16, os.cpu_count() or 1))
    yield


def pytest_terminal_summary(terminalreporter):
    """What the parity checks actually observed, per tolerance class: the worst relative L2 error, the largest fraction of
    elements outside the per-element bound and the worst single error as a multiple of its bound."""
    from tests import gpu_util
    if not gpu_util.OBSERVED:
        return
    tr = terminalreporter
    tr.section("observed parity errors (tests/gpu_util.py assert_close)")
    for kind in ("f32 kernel", "bf16 kernel", "bf16 step"):
        rows = [r for r in gpu_util.OBSERVED if r["kind"] == kind]
        if not rows:
            continue
        by_l2 = max(rows, key=lambda r: r["rel_l2"])
        by_frac = max(rows, key=lambda r: r["frac_outside"])
        by_worst = max(rows, key=lambda r: r["worst_ratio"])
        tr.write_line(f"{kind}: {len(rows)} comparisons, {sum(r['n'] for r in rows)} elements")
        tr.write_line(f"  worst relative L2      {by_l2['rel_l2']:.3g}  ({by_l2['name']})")
        tr.write_line(f"  most elements outside  {by_frac['frac_outside']:.3g} of {by_frac['n']}  ({by_frac['name']})")
        tr.write_line(f"  worst error / bound    {by_worst['worst_ratio']:.3g}  ({by_worst['name']})")
