import pathlib
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session", autouse=True)
def built_library():
    """The tests load the library that is built; only when none is there do they build it (hipcc cross-compiles
    without a GPU).  The package itself never builds or falls back: without the library it raises."""
    from pam_amd import build as builder
    if not builder.LIB.exists():
        builder.build()
    return builder.LIB


@pytest.fixture(scope="session")
def oracle():
    from oracle import pam_oracle
    pam_oracle.build()
    return pam_oracle
