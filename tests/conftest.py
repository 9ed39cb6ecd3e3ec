import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_dirs(tmp_path_factory):
    """Model folders of the two tiny configurations, random weights, made once a session."""
    from helpers import TINY, TINY_MFMA, make_model_dir
    out = {}
    for name in list(TINY) + list(TINY_MFMA):
        out[name] = make_model_dir(name, str(tmp_path_factory.mktemp(f"tiny_{name}")))
    return out


@pytest.fixture(scope="session")
def plain_models(model_dirs):
    """name -> (config dict, weights as float64 arrays) read by the plain implementation."""
    import plain_llama
    return {name: plain_llama.read_model(d) for name, d in model_dirs.items()}
