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
