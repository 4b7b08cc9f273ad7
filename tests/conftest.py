import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (str(ROOT), str(ROOT / "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle_lib
    return oracle_lib.load_oracle()


@pytest.fixture(scope="session")
def reference():
    import oracle_lib
    lib = oracle_lib.load_reference()
    if lib is None:
        pytest.skip("oracle/_ref/libsaltref.so not built (make -C oracle ref)")
    return lib


@pytest.fixture(scope="session")
def pkg():
    from __graft_entry__ import load_package
    return load_package()
