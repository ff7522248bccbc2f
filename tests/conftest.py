import json
import math
import os
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (runs the HIP kernels through the C ABI)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def _num(v):
    if v == "log2":
        return math.log(2.0)
    if v == "-inf":
        return float("-inf")
    return v


def _decode(x):
    if isinstance(x, list):
        return [_decode(v) for v in x]
    return _num(x)


@pytest.fixture(scope="session")
def known_answers():
    with open(GOLDEN / "reference_known_answers.json") as f:
        data = json.load(f)
    for case in data["rejection_sampling"]:
        for k in ("prox", "old", "mask"):
            case[k] = _decode(case[k])
    return data


@pytest.fixture(scope="session")
def device():
    return torch.device("cuda:0")
