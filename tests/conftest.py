import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load_golden():
    """The reference-held vectors (tests/golden/reference_vectors.json) with "nan" strings turned into NaN."""
    import json

    def fix(x):
        if isinstance(x, str) and x == "nan":
            return float("nan")
        if isinstance(x, list):
            return [fix(y) for y in x]
        if isinstance(x, dict):
            return {k: fix(v) for k, v in x.items()}
        return x

    with open(os.path.join(GOLDEN_DIR, "reference_vectors.json")) as f:
        return fix(json.load(f))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def dev():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


@pytest.fixture(autouse=True)
def _waiting_kernels_as_the_environment_says(request):
    """Tests force time-outs of the kernels that wait inside a launch; the host mirror reacts to those by switching
    such kernels off for the process.  Every GPU test starts from what the environment says."""
    yield
    if "dev" in request.fixturenames:
        from verl_amd import _cabi
        from verl_amd.trainer.ppo import core_algos as CA

        _cabi.lib().vamd_set_waiting_kernels(-1)
        CA._WAITING_WATCH["calls"] = 0
        CA._WAITING_WATCH["seen"].clear()
