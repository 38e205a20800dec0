import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "oracle"))
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (runs the HIP kernels in libqie.so)")
    config.addinivalue_line("markers", "slow: long-running")


def pytest_collection_modifyitems(config, items):
    """The layered-engine GPU tests run after every other module.  tests/test_gpu_tp.py drives two
    in-process ranks whose exchange kernels wait for each other: that needs the two ranks' streams
    on different hardware queues, and which queue a new stream gets depends on how many streams the
    process has created before.  Those tests were written under the stream history of the modules
    before them; modules that create many engines of their own therefore go last."""
    names = ("test_gpu_layered", "test_gpu_nodutar", "test_gpu_lugipel", "test_gpu_verelorn")
    late = [it for it in items if any(n in it.nodeid for n in names)]
    if late:
        items[:] = [it for it in items if not any(n in it.nodeid for n in names)] + late


@pytest.fixture(scope="session")
def oracle():
    import oracle as O
    O.lib()
    return O


@pytest.fixture(scope="session")
def qlib():
    from qwen_inference_engine_amd import _lib
    return _lib.load()


@pytest.fixture(autouse=True)
def _release_device_buffers():
    yield
    import gpu_util
    gpu_util.release_all()


def rng(seed=0):
    return np.random.default_rng(seed)


def pytest_sessionfinish(session, exitstatus):
    """On the GPU box, keep every end-to-end parity step's (engine error, bar) as evidence."""
    import json
    try:
        import parity
    except Exception:
        return
    if parity.REPORT and os.environ.get("GRAFT_REPO_ROOT"):
        out = os.path.join(ROOT, "gpurun_out")
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "parity_report.json"), "w") as f:
            json.dump([{"step": w, "norm_rel": r, "bar": b} for w, r, b in parity.REPORT], f, indent=0)
