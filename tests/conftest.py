"""Shared test plumbing: the ``gpu`` marker, paths and seeded operands."""

from __future__ import annotations

import sys
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) device")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _library_options_back_to_default(request):
    """Tests force kernels through cmi_set_option; none of that may leak into the next test."""
    yield
    if "gpu" in request.keywords:
        from coffin_amd import _native
        lib = _native.load()
        lib.cmi_set_option(b"gemm_tile", 0)
        lib.cmi_set_option(b"gemv_wholerow", -1)
        lib.cmi_set_option(b"w4_decode_waves", 0)
        lib.cmi_set_option(b"w4_decode_chain", 0)


@pytest.fixture(scope="session")
def golden():
    def load(name: str):
        return np.load(GOLDEN / f"{name}.npz", allow_pickle=False)
    return load


@pytest.fixture(scope="session")
def orc():
    from oracle import oracle
    oracle.build()
    return oracle
