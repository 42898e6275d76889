import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "grad.cpp_amd"))
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def ckpt_dir(tmp_path_factory):
    return tmp_path_factory.mktemp("ckpt")


def pytest_terminal_summary(terminalreporter):
    """Puts the margins of the logits rule on record: the worst observed share of
    each allowance per labelled comparison of the run."""
    try:
        from helpers import WORST
    except Exception:
        return
    if not WORST:
        return
    terminalreporter.write_line("logits rule, worst share of the allowance (max-norm, per-element):")
    named = {k: v for k, v in WORST.items() if k[:2] in ("c0", "c1", "c2", "c3", "c4")}
    for label in sorted(named):
        a, b = named[label][:2]
        terminalreporter.write_line(f"  {label}: {a:.3f} {b:.3f}")
    rest = {k: v for k, v in WORST.items() if k not in named}
    if rest:
        wa = max(rest, key=lambda k: rest[k][0])
        wb = max(rest, key=lambda k: rest[k][1])
        terminalreporter.write_line(f"  other comparisons ({len(rest)} labels): max-norm {rest[wa][0]:.3f} ({wa}), "
                                    f"per-element {rest[wb][1]:.3f} ({wb})")
        terminalreporter.write_line(f"    that element: {rest[wb][2]}")
