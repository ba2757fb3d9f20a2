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


def pytest_runtest_logstart(nodeid, location):
    """Every GPU test's name goes to the real stderr, flushed, before it starts: if the process
    dies inside it, the output still says which case it was."""
    if torch.cuda.is_available():
        sys.__stderr__.write("\n[starting] %s\n" % nodeid)
        sys.__stderr__.flush()


@pytest.hookimpl(tryfirst=True)
def pytest_pyfunc_call(pyfuncitem):
    """GPU tests are called through a frame whose file name is the test's full name with its
    parameters, so that a dump of the Python stack (the fault handler's, at a fatal signal) names
    the case in the line next to the test function's own, even where the output's head is lost."""
    if "gpu" not in pyfuncitem.keywords:
        return None
    scope = {}
    exec(compile("def named_frame(function, arguments):\n    return function(**arguments)\n",
                 "<%s>" % pyfuncitem.nodeid, "exec"), scope)
    arguments = {name: pyfuncitem.funcargs[name] for name in pyfuncitem._fixtureinfo.argnames}
    scope["named_frame"](pyfuncitem.obj, arguments)
    return True


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
