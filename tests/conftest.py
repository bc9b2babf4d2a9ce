"""Shared pytest setup: the `gpu` marker and import paths."""
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


import pytest  # noqa: E402


@pytest.fixture
def test_options():
    """Setter for the library's test hooks (lpp_set_test_option); every option is back at its default afterwards."""
    from lighterpp_amd import capi
    yield capi.set_test_option
    capi.reset_test_options()
