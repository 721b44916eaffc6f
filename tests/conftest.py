import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import matrix_fsdp_amd  # noqa: E402  (loads the package from matrix-fsdp_amd/)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run with -m gpu on an MI355X)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def golden():
    with open(os.path.join(ROOT, "tests", "golden", "reference_vectors.json")) as f:
        return json.load(f)


class P:
    """Parameter extents for oracle calls (offset / end / numel / fqn / shape)."""

    def __init__(self, fqn, offset, numel, shape=None):
        self.fqn, self.offset, self.numel = fqn, offset, numel
        self.end = offset + numel
        self.shape = tuple(shape) if shape is not None else (numel,)


def params_from_pairs(pairs):
    out, cursor = [], 0
    for name, n in pairs:
        out.append(P(name, cursor, n))
        cursor += n
    return out


def segs(triples):
    from matrix_fsdp_amd import LayoutSegment

    return tuple(tuple(LayoutSegment(*t) for t in rank) for rank in triples)
