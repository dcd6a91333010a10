import os
import re
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def _has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_terminal_summary(terminalreporter, exitstatus, config):
    """Tolerance headroom: worst err/bound of every tensor compared through tests.util.assert_close in this
    run, against the bound in force and against the purely elementwise relative bound."""
    from tests import util
    if not util.HEADROOM:
        return
    terminalreporter.section("tolerance headroom (worst err/bound per compared tensor)")
    rows = sorted(util.HEADROOM.items(), key=lambda kv: -kv[1][0])
    terminalreporter.write_line(f"{len(rows)} tensors compared; the 40 with the least headroom (all of them: "
                                "headroom.json in the folder SMX_TEST_REPORT_DIR names, when set)")
    n_all = sum(r[1][2] for r in rows)
    n_over = sum(r[1][3] for r in rows)
    terminalreporter.write_line(f"{n_over} of {n_all} compared elements ({n_over / max(n_all, 1):.2e}) lie outside the plain "
                                "elementwise bound rel * |ref| and pass on the RMS floor or the summation-ulp allowance")
    by_group = {}
    for (test, what), (_, _, n, over) in rows:
        m = re.search(r"test_full_size_workload\[(\d)\]", test)
        group = f"cfg{m.group(1)} full size" if m else ("full-size drop-in flow" if "full_size_dropin" in test else "other tests")
        a = by_group.setdefault(group, [0, 0])
        a[0] += n
        a[1] += over
    for group in sorted(by_group):
        n, over = by_group[group]
        terminalreporter.write_line(f"    {group}: {over} of {n} elements ({over / max(n, 1):.2e})")
    terminalreporter.write_line("  in force  elementwise  outside/elements  test :: tensor")
    for (test, what), (with_floor, pure, n, over) in rows[:40]:
        terminalreporter.write_line(f"{with_floor:9.3g} {pure:9.3g}  {over:>7d}/{n:<9d} {test} :: {what}")
    out_dir = os.environ.get("SMX_TEST_REPORT_DIR")
    if out_dir and os.path.isdir(out_dir):
        import json
        with open(os.path.join(out_dir, "headroom.json"), "w") as f:
            json.dump([[t, w, a, b, n, over] for (t, w), (a, b, n, over) in rows], f, indent=0)
