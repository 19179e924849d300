import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import pyoracle

    pyoracle.lib()
    pyoracle.set_round_mode(pyoracle.ROUND_HALF_AWAY)
    return pyoracle


@pytest.fixture(scope="session")
def golden():
    import json

    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def hipq():
    from torsh_amd import hipq as mod

    mod.load()
    return mod


@pytest.fixture(scope="session")
def ctx(hipq):
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    c = hipq.Context(0)
    yield c
    torch.cuda.synchronize()
    c.close()
