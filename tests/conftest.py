"""Shared pytest setup: the ``gpu`` marker, import paths and library handles."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest

REPO_ROOT = Path(__file__).resolve().parent.parent
for extra in (REPO_ROOT, REPO_ROOT / "rl-kernel_amd", REPO_ROOT / "tests"):
    if str(extra) not in sys.path:
        sys.path.insert(0, str(extra))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def _gpu_available() -> bool:
    try:
        import torch

        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if _gpu_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def rlk_lib():
    """The C-ABI library; a missing build is a hard failure, never a skip."""
    from rl_engine import _lib

    return _lib.load()


@pytest.fixture(scope="session")
def oracle():
    from oracle import reference_math

    reference_math.build_c_oracle()
    return reference_math
