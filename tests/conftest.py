import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def _memoise_workloads():
    """Several tests build the same scaled-down workload graph; generate each once per session (the tests get
    copies, so none can disturb another)."""
    from artifact_amd import graphgen

    raw, cache = graphgen.make_workload, {}

    def make_workload(name, scale_down=0):
        key = (name, scale_down)
        if key not in cache:
            ip, ix = raw(name, scale_down)
            if len(ix) > 20_000_000:      # full-size graphs are built by one module each: not worth the memory
                return ip, ix
            cache[key] = (ip, ix)
        ip, ix = cache[key]
        return ip.copy(), ix.copy()

    graphgen.make_workload = make_workload


_memoise_workloads()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, where no GPU exists (the CPU suite runs with -m 'not gpu')."""
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as O
    O.lib()
    return O


def pytest_terminal_summary(terminalreporter):
    """How often the fp32 parity checks needed the summation term of their tolerance (helpers.close_fp32)."""
    try:
        from helpers import FP32_BAR_STATS as st
    except ImportError:
        return
    if st["compared"]:
        terminalreporter.write_line(
            f"fp32 parity: {st['compared']} elements compared against float64 / the fp32 restatement; "
            f"{st['beyond_strict']} ({100.0 * st['beyond_strict'] / st['compared']:.5f} %) beyond the strict bar "
            f"1e-6 + 1e-5*|want| and inside the summation bound; largest error there {st['max_excess_ratio']:.2f}x the "
            f"strict bar ({st['max_excess_abs']:.2e} above it)")
