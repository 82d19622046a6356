import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def tiny_dirs(tmp_path_factory):
    """Model folders (config.json + model.safetensors) of the tiny test configurations."""
    import helpers
    return helpers.TinyModels(tmp_path_factory.mktemp("models"))
