import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "metaattention_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: test needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def pytest_runtest_setup(item):
    # A kernel fault can end the whole box before pytest reports anything: name the GPU test that is about to run, flushed,
    # where the tail of the run's output will show it.
    if "gpu" in item.keywords:
        capman = item.config.pluginmanager.getplugin("capturemanager")
        if capman is not None:
            with capman.global_and_fixture_disabled():      # (past pytest's capture: a captured line dies with the process)
                sys.stderr.write(f"[gpu test] {item.nodeid}\n")
                sys.stderr.flush()
