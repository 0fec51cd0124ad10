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
    terminalreporter.write_line("achieved max relative errors (label: floored | plain over |ref| > floor | elements)")
    for label in sorted(helpers.ACHIEVED):
        e, plain, n = helpers.ACHIEVED[label]
        terminalreporter.write_line("  %-60s %.3e | %.3e | %d" % (label, e, plain, n))
