import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "g-core-gh_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "exhaustive: minutes-long exhaustive sweeps, enabled with LOWP_EXHAUSTIVE=1")


def pytest_collection_modifyitems(config, items):
    import torch

    has_gpu = torch.cuda.is_available()
    for item in items:
        if "gpu" in item.keywords and not has_gpu:
            item.add_marker(pytest.mark.skip(reason="no GPU visible"))
        if "exhaustive" in item.keywords and os.environ.get("LOWP_EXHAUSTIVE") != "1":
            item.add_marker(pytest.mark.skip(reason="set LOWP_EXHAUSTIVE=1 to run"))


@pytest.fixture(scope="session")
def corc():
    """The scalar C oracle, built on demand with gcc."""
    from oracle import c_oracle

    c_oracle.build()
    return c_oracle
