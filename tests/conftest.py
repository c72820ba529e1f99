import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))

import __graft_entry__ as entry  # noqa: E402

entry.load_package()
entry.load_oracle()


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import gufo_oracle
    gufo_oracle.lib()
    return gufo_oracle


@pytest.fixture(scope="session")
def ref_oracle(oracle):
    if not oracle.ref_available():
        pytest.skip("oracle/_ref was not built (reference sources absent)")
    oracle.ref()
    return oracle


@pytest.fixture(scope="session")
def hip():
    """The initialised library.  No fallback: a missing library or device fails."""
    from gufo_npu_amd import capi
    capi.load_library()
    capi.init(0)
    yield capi
    capi.synchronize()


GOLDEN = ROOT / "tests" / "golden"
