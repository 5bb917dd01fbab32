"""Shared test plumbing: the ``gpu`` marker, import paths, and the oracle/kernels handles."""

import json
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run on the GPU box only)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def embedding_norm_cases():
    with open(GOLDEN / "embedding_norm_vectors.json") as f:
        data = json.load(f)
    cases = []
    for c in data["cases"]:
        cases.append(
            {
                "name": c["name"],
                "ids": torch.tensor(c["ids"], dtype=torch.int64).reshape(c["ids_shape"]),
                "backprops": torch.tensor(c["backprops"], dtype=torch.float32).reshape(c["backprops_shape"]),
                "expected": torch.tensor(c["expected_norms"], dtype=torch.float32),
                "intermediates": c.get("intermediates"),
            }
        )
    return cases
