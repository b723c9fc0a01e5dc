import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# The package directory is `torq-compiler_amd`; `torq_compiler_amd` is a symlink to it so that
# it can be imported.  Recreate the import name if the link did not survive a copy.
_link = os.path.join(ROOT, "torq_compiler_amd")
if not os.path.exists(_link):
    import importlib.util

    spec = importlib.util.spec_from_file_location(
        "torq_compiler_amd", os.path.join(ROOT, "torq-compiler_amd", "__init__.py"),
        submodule_search_locations=[os.path.join(ROOT, "torq-compiler_amd")])
    mod = importlib.util.module_from_spec(spec)
    sys.modules["torq_compiler_amd"] = mod
    spec.loader.exec_module(mod)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 GPU (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def device():
    """The GPU under test.  Fails loudly (never skips to a CPU path) when libthip.so or the GPU is missing."""
    import torq_compiler_amd as thip

    dev = thip.Device(0)
    assert dev.name() == "gfx950"
    yield dev
    dev.close()
