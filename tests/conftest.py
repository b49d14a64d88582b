import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    return oracle


@pytest.fixture(scope="session")
def gc():
    """The package with its library loaded.  What is built in-tree is used as it is; only a tree in
    which nothing has been built yet (a fresh checkout) is built here - the package itself never
    builds or falls back, it raises."""
    import graphchallenge21_amd
    driver = os.path.join(os.path.dirname(graphchallenge21_amd.lib_path()), "spdnn_network")
    if not os.path.exists(graphchallenge21_amd.lib_path()) or not os.path.exists(driver):
        graphchallenge21_amd.build()
    graphchallenge21_amd.load_library()
    return graphchallenge21_amd
