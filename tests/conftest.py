import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_terminal_summary(terminalreporter):
    """How often the attention checks needed their one allowance (a row one rounding flip
    away from the oracle, proven by recomputation): per check and in total; also written as
    parity_allowance.txt into the folder KVX_TEST_REPORT_DIR names (default: the run's output
    folder at the repository root) where that folder exists."""
    gpulib = sys.modules.get("gpulib")
    log = getattr(gpulib, "ALLOWANCE_LOG", None)
    if not log:
        return
    explained = sum(n for _, n, _ in log)
    rows = sum(total for _, _, total in log)
    lines = [f"attention rows above tolerance, each proven one rounding flip from the oracle: "
             f"{explained} of {rows} rows in {len(log)} checks"]
    lines += [f"  {n:4d} of {total:6d}  {label}" for label, n, total in log if n]
    terminalreporter.write_line("\n".join(lines))
    out = os.environ.get("KVX_TEST_REPORT_DIR", os.path.join(ROOT, "gpurun_out"))
    if os.path.isdir(out):
        with open(os.path.join(out, "parity_allowance.txt"), "w") as f:
            f.write("\n".join(lines) + "\n")
