import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from checkers import Oracle
    return Oracle()


@pytest.fixture(scope="session")
def ref():
    from checkers import Ref
    if not Ref.available():
        pytest.skip("oracle/_ref/libboltref.so not built or host lacks avx512_vnni")
    return Ref()
