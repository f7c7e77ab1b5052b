import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The oracle's attention functions spread a tile's independent rows over the host's cores
    while the suite runs (same results, computed row by row as ever; a one-GPU box's share of
    its host is 16 cores)."""
    from oracle import kvoracle as ko
    ko.set_threads(max(1, min(16, len(os.sched_getaffinity(0)))))


def pytest_terminal_summary(terminalreporter):
    """How often the attention checks needed their one allowance (a row one rounding flip
    away from the oracle, proven by recomputation): per check and in total; also written as
    parity_allowance.txt into the folder KVX_TEST_REPORT_DIR names, where that is set and exists."""
    gpulib = sys.modules.get("gpulib")
    log = getattr(gpulib, "ALLOWANCE_LOG", None)
    if not log and not getattr(gpulib, "DEVIATION_LOG", None):
        return
    log = log or []
    measured = [f"score deviation of the matrix-core kernels from the oracle, {name}: max {worst_max:.2e}, "
                f"max + log(sum) {worst_lse:.2e} over {samples} split statistics; flip slack {slack:.2e}"
                for name, samples, worst_max, worst_lse, slack in getattr(gpulib, "DEVIATION_LOG", None) or []]
    explained = sum(n for _, n, _ in log)
    rows = sum(total for _, _, total in log)
    lines = [f"attention rows above tolerance, each proven one rounding flip from the oracle: "
             f"{explained} of {rows} rows in {len(log)} checks"]
    lines += [f"  {n:4d} of {total:6d}  {label}" for label, n, total in log if n]
    lines += measured
    terminalreporter.write_line("\n".join(lines))
    out = os.environ.get("KVX_TEST_REPORT_DIR")
    if out and os.path.isdir(out):
        with open(os.path.join(out, "parity_allowance.txt"), "w") as f:
            f.write("\n".join(lines) + "\n")
