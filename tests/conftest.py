import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box with -m gpu)")


def _has_gpu() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def attn_variant():
    """Force one of the attention kernel's work decompositions for a test; automatic choice again afterwards."""
    from aitemplate_amd import _kernels

    lib = _kernels.load()

    def force(variant):
        _kernels.check(lib.aitamd_attention_set_variant(int(variant)), "aitamd_attention_set_variant")

    yield force
    lib.aitamd_attention_set_variant(-1)
