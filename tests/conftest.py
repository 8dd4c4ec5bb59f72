import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "msccl-tools_amd")
for p in (ROOT, PKG, os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def mscclx_lib():
    """The built C-ABI library; built on first use only if no build exists."""
    from msccl.executor import binding
    if not os.path.exists(binding.LIB_PATH):
        sys.path.insert(0, binding.CSRC_DIR)
        import build as _build
        _build.build(force=True, verbose=False)
    return binding.load_library()
