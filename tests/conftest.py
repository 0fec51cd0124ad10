import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
if os.path.dirname(os.path.abspath(__file__)) not in sys.path:
    sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_terminal_summary(terminalreporter):
    """The errors that labelled comparisons achieved in this run: with the 0.1 RMS floor in the denominator (what the
    tests assert on) and as plain relative errors over the elements above that floor."""
    import helpers
    if not helpers.ACHIEVED:
        return
    # the rows of the sweeps over fused-layer variants first, the BASELINE configurations and the batch-norm input gradients
    # last: a reader who only keeps the end of the output keeps those
    labels = sorted(helpers.ACHIEVED, key=lambda l: (not l.startswith("fused "), l))
    lines = ["achieved max relative errors (label: floored | plain over |ref| > floor | elements)"]
    for label in labels:
        e, plain, n = helpers.ACHIEVED[label]
        lines.append("  %-60s %.3e | %.3e | %d" % (label, e, plain, n))
    for line in lines:
        terminalreporter.write_line(line)
    # the whole table as a file beside the run's other output
    out_dir = os.path.join(ROOT, "gpurun_out")
    try:
        os.makedirs(out_dir, exist_ok=True)
        with open(os.path.join(out_dir, "parity_achieved.txt"), "w") as f:
            f.write("\n".join(lines) + "\n")
    except OSError:
        pass
