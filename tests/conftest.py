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


@pytest.fixture(autouse=True)
def _library_is_the_backend(request):
    """A GPU test grades the kernel library, whatever a test before it installed in its place (the host tests run the
    engine over plain PyTorch stand-ins through ``ops.set_backend``); and no test leaves a stand-in behind."""
    from tempura_amd.kernels import ops
    if request.node.get_closest_marker("gpu") is not None:
        ops.set_backend(None)
    yield
    ops.set_backend(None)
