import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")
    config.addinivalue_line("markers", "perf: a speed floor on the GPU (leave out with -m 'gpu and not perf')")


@pytest.fixture(scope="session", autouse=True)
def built_library():
    """The tests load the library that is built in-tree; only a tree where nothing has been built
    yet (a fresh clone) compiles it first."""
    from flextrain_amd import _C
    if not os.path.exists(_C.LIB_PATH):
        from flextrain_amd.build import build_library
        build_library()
    return _C.LIB_PATH


@pytest.fixture(scope="session")
def oracle():
    """The CPU checker (test infrastructure)."""
    import oracle as _oracle
    _oracle.lib()
    return _oracle


@pytest.fixture(scope="session")
def cuda():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU in this environment")
    return torch.device("cuda", 0)


# Facts a passing test wants on record (how much of a configuration a machine could hold, say):
# `pytest -q` drops the output of passing tests, the terminal summary stays.
_SUMMARY_LINES = []


@pytest.fixture
def summary_line():
    """Callable that puts one line into the run's terminal summary."""
    return _SUMMARY_LINES.append


def pytest_terminal_summary(terminalreporter):
    if _SUMMARY_LINES:
        terminalreporter.section("coverage notes")
        for line in _SUMMARY_LINES:
            terminalreporter.write_line(line)
