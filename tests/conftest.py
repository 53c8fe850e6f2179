import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session", autouse=True)
def pipeline_bodies_cached_in_a_temporary_directory(tmp_path_factory):
    """Pipeline bodies compiled at run time are kept on disk between processes (pipeline_jit.hip). The tests keep theirs
    in a directory of their own, so that a run neither leaves files in the user's cache nor finds old ones there."""
    before = os.environ.get("DH_PIPELINE_JIT_CACHE")
    os.environ["DH_PIPELINE_JIT_CACHE"] = str(tmp_path_factory.mktemp("pipeline_bodies"))
    yield
    if before is None:
        os.environ.pop("DH_PIPELINE_JIT_CACHE", None)
    else:
        os.environ["DH_PIPELINE_JIT_CACHE"] = before


def _has_gpu() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def ctx():
    """One device context for the whole GPU test session."""
    from daphne_amd.kernels import HIPContext

    c = HIPContext(0)
    yield c
    c.destroy()
