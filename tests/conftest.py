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
    """The tests load the library that is built, provided it was built from this tree's sources (it carries their
    hash); a missing or stale one is rebuilt first (hipcc cross-compiles without a GPU).  The package itself never
    builds or falls back: without the library it raises."""
    from pam_amd import build as builder
    lib, stamp = builder.ensure_built()
    print(f"libpam_hip.so built from sources {stamp}")
    return lib


@pytest.fixture(scope="session")
def oracle():
    from oracle import pam_oracle
    pam_oracle.build()
    return pam_oracle
