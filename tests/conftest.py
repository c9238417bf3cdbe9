import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (runs through libgnnagg.so on cuda:0)")


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_index_map_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def reference_op():
    """The reference's own compiled native op (oracle/_ref), or skip."""
    from oracle import spmm as ospmm

    mod = ospmm.load_reference_op()
    if mod is None:
        pytest.skip("oracle/_ref is not built (or the host lacks AVX-512)")
    return mod
