import json
import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def hand_case():
    """Hand-computed 2x3 known-answer case (tests/golden/hand_2x3.json)."""
    with open(os.path.join(GOLDEN, "hand_2x3.json")) as f:
        raw = json.load(f)
    out = {}
    for k, v in raw.items():
        if k.startswith("_"):
            continue
        if k in ("spatial_shapes", "level_start_index"):
            out[k] = torch.tensor(v, dtype=torch.int64)
        else:
            out[k] = torch.tensor(np.array(v, dtype=np.float64))
    return out


@pytest.fixture(scope="session")
def gpu_device():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda", 0)


@pytest.fixture(autouse=True)
def _tuning_follows_the_environment():
    """The library reads its MXD_MSDA_* tuning variables once per process; tests that change them call
    util.set_tuning(), and after every test (monkeypatch has restored the environment by then) they are read again."""
    yield
    from drivingsdk_amd import _lib
    if _lib._lib is not None:
        _lib.reload_tuning()
