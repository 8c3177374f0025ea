import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session", autouse=True)
def _libraries_are_built():
    """The tests load the libraries that are in the tree; they are compiled here only when none is."""
    from energonai_amd import build
    build.ensure_built()


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


# shape and lengths of the reference's own kernel test
# (tests/test_kernel/test_transpose_pad_fusion_kernel.py:6-11)
REF_TEST = dict(batch=8, seq=128, heads=12, head_dim=64, lens=[24, 127, 31, 65, 24, 127, 31, 65])


@pytest.fixture
def ref_test_shape():
    return dict(REF_TEST)
