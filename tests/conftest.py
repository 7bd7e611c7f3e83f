import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def _ledger():
    from tests import parity
    return parity.LEDGER


# the folder for what a test run leaves behind (not under version control)
LEDGER_DIR = os.environ.get("FAITH_TEST_OUTPUT", "gpurun_out")


def pytest_sessionfinish(session, exitstatus):
    """Keeps the parity concessions of the run (tests/parity.py) where the run's output is kept."""
    import json
    led = _ledger()
    if not led["comparisons"]:
        return
    out = os.path.join(ROOT, LEDGER_DIR)
    try:
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "parity_ledger.json"), "w") as f:
            json.dump(led, f, indent=1)
    except OSError:
        pass


def pytest_terminal_summary(terminalreporter):
    led = _ledger()
    if not led["comparisons"]:
        return
    kinds, per_test = {}, {}
    for c in led["concessions"]:
        kinds[c["kind"]] = kinds.get(c["kind"], 0) + 1
        fn = c["test"].split("[")[0]
        per_test[(fn, c["kind"], c["tensor"])] = per_test.get((fn, c["kind"], c["tensor"]), 0) + 1
    terminalreporter.write_line(
        f"parity ledger: {led['comparisons']} harness comparisons, {led['plain']} on the plain bar "
        f"(rtol 1e-5 / atol 1e-6), concessions: {kinds if kinds else 'none'} (each one in {LEDGER_DIR}/parity_ledger.json)")
    for (fn, kind, tensor), n in sorted(per_test.items()):
        terminalreporter.write_line(f"  {n:4d} x {kind:<24s} {tensor:<6s} {fn}")
    # every contraction tensor, conceded or not: the worst distance from float64 per test, GPU and fp32 oracle, in
    # units of the plain bar, and the worst ratio among the tensors whose GPU error is at least a quarter of the bar
    worst = {}
    for c in led.get("contractions", []):
        fn = c["test"].split("[")[0]
        w = worst.setdefault(fn, dict(n=0, gpu=0.0, oracle=0.0, ratio=0.0))
        w["n"] += 1
        w["gpu"] = max(w["gpu"], c["gpu_err_of_bar"])
        w["oracle"] = max(w["oracle"], c["oracle_err_of_bar"])
        if c["gpu_err_of_bar"] >= 0.25:
            w["ratio"] = max(w["ratio"], c["ratio"])
    if worst:
        terminalreporter.write_line("contractions against float64, worst per test (units of the plain bar): tensors, GPU, fp32 "
                                    "oracle, worst GPU / oracle ratio where the GPU error reaches a quarter of the bar")
        for fn, w in sorted(worst.items()):
            terminalreporter.write_line(f"  {w['n']:5d}  gpu {w['gpu']:8.3f}  oracle {w['oracle']:8.3f}  ratio {w['ratio']:6.2f}  {fn}")
