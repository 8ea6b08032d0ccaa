import os
import sys

import pytest

# The tests name the search strategy they mean; everything else runs on the
# scanning kernels, whatever the size (the library's own default would bin
# the large cases).
os.environ.setdefault("PCA_SEARCH_STRATEGY", "scan")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line(
        "markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    import oracle as _oracle
    _oracle._load()
    return _oracle


@pytest.fixture(scope="session")
def ref(oracle):
    if not oracle.have_ref():
        pytest.skip("oracle/_ref is not built (needs the reference sources)")
    return oracle
