import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lib():
    """The C-ABI library, loaded through the package loader (fails loudly if unbuilt)."""
    from flashsvd_amd import _lib
    return _lib.load()


@pytest.fixture(autouse=True)
def _runtime_flags_do_not_leak():
    """Runtime switches are process-wide environment variables; a test that sets them (configure_runtime does) must
    not change what the next test runs."""
    keep = {k: v for k, v in os.environ.items() if k.startswith(("FLASH_SVD", "SVDLLM_", "FLASHSVD_AMD"))}
    yield
    for k in [k for k in os.environ if k.startswith(("FLASH_SVD", "SVDLLM_", "FLASHSVD_AMD"))]:
        if k not in keep:
            del os.environ[k]
    os.environ.update(keep)
