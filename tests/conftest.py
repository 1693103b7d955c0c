import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    # use the library that is built; compile it only when there is none
    import __graft_entry__

    __graft_entry__.ensure_built()


@pytest.fixture(scope="session")
def lib():
    import pika_h3_flex_amd as pk

    return pk._lib.load()
