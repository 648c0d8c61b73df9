import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "flash-attention_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def lib():
    """The C-ABI library, built in-tree beforehand; built here only if nothing is there."""
    from flash_attn import flash_attn_gfx950 as be
    if not os.path.exists(be.LIB_PATH):
        sys.path.insert(0, PKG)
        import build as _build
        _build.build()
    return be.load_library()
