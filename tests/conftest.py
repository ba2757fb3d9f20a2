import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def cpu_ops(monkeypatch):
    """Put the plain PyTorch twins in place of the HIP operations, so that the
    engine's host logic can run without a GPU."""
    import torch_ops
    from qwen3_from_scratch_amd import ops

    for name in torch_ops.ALL:
        monkeypatch.setattr(ops, name, getattr(torch_ops, name))
    return torch_ops


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """Random-weight model folders of the tiny configurations, made once."""
    from helpers import TINY, make_folder

    root = tmp_path_factory.mktemp("models")
    return {name: make_folder(str(root / name), name) for name in TINY}
