"""Test configuration: the `gpu` marker (tests that need a real MI355X), the repo root
on `sys.path`, a fixed seed per test and an empty per-session kernel cache so no
stored tuning table leaks into a test."""

import os
import sys
from pathlib import Path

import pytest
import torch

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) device")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(0)


@pytest.fixture(autouse=True, scope="session")
def _kernel_cache(tmp_path_factory):
    os.environ["KOHAKUMOSS_KERNEL_CACHE"] = str(tmp_path_factory.mktemp("kernel-cache"))
    yield
