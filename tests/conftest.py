import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def pytest_terminal_summary(terminalreporter):
    try:
        import trace_tools
    except ImportError:
        return
    if trace_tools.OBSERVED:
        terminalreporter.write_line("largest errors observed, as a share of the largest logit of the plain implementation:")
        for group in sorted(trace_tools.OBSERVED):
            terminalreporter.write_line(f"  {group}: {trace_tools.OBSERVED[group]:.2e}")
