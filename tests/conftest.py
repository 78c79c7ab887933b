import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "chill-attention_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")


# (name, args) of the mask instances the reference's own tests use (test_chill_attention.py:23-29)
# plus the BASELINE configurations and a few edge instances.
MASK_INSTANCES = [
    ("FullChillMask", ()),
    ("CausalChillMask", ()),
    ("SlidingWindowChillMask", (10, 4)),
    ("ChunkwiseChillMask", (10, 4)),
    ("PrefixLMChillMask", (10,)),
    ("SlidingWindowChillMask", (128, 128)),
    ("ChunkwiseChillMask", (128, 2)),
    ("PrefixLMChillMask", (1024,)),
    ("SlidingWindowChillMask", (0, 0)),
    ("SlidingWindowChillMask", (0, 7)),
    ("SlidingWindowChillMask", (300, 0)),
    ("ChunkwiseChillMask", (1, 3)),
    ("ChunkwiseChillMask", (100, 0)),
    ("ChunkwiseChillMask", (77, 5)),
    ("PrefixLMChillMask", (0,)),
    ("PrefixLMChillMask", (77,)),
]


def mask_id(m):
    return f"{m[0]}{m[1]}"


def make_mask(m):
    import chill_attention as ca

    return getattr(ca, m[0])(*m[1])


@pytest.fixture(autouse=True)
def _seed():
    import torch

    torch.manual_seed(20)
    yield
