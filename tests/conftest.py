"""Shared pytest setup: the ``gpu`` marker, repo-root imports, seeded inputs."""

from __future__ import annotations

import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# The library looks at its PHYAI_FP8_* tuning variables only when this switch was set before its
# first call; the tests that force kernel variants need it.
os.environ.setdefault("PHYAI_FP8_TUNING", "1")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def seeded(shape, seed, scale=1.0, dtype=torch.bfloat16):
    """CPU tensor ~ N(0, scale^2) from its own generator, so CPU and GPU see the same bits."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


@pytest.fixture(scope="session")
def dev():
    return torch.device("cuda", 0)
