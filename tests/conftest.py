import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402

# Launch sequences of fewer than six steps run without a hipGraph by default (a replay costs more
# than that few direct launches).  The suite's small graphs are there to test capture and replay
# as well: they run captured unless a test says otherwise
# (test_short_launch_sequences_run_uncaptured covers the default).
os.environ.setdefault("ODLA_HIP_GRAPH_MIN_STEPS", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (runs through libodla_hip.so)")


@pytest.fixture(scope="session")
def pkg():
    return entry.load()


@pytest.fixture(scope="session")
def odla(pkg):
    return pkg.odla


@pytest.fixture(scope="session")
def models(pkg):
    return pkg.models


@pytest.fixture(scope="session")
def ref():
    return entry.load_oracle()
