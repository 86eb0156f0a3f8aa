"""Shared pytest setup: markers, import path, and the built libraries."""

from __future__ import annotations

import importlib
import pathlib
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def capi():
    """ctypes binding of libfa2_gfx950.so; builds the library only if nothing is built."""
    mod = importlib.import_module("flash-attention-triton_amd._capi")
    if not mod.LIBRARY_PATH.exists():
        importlib.import_module("flash-attention-triton_amd.build").build()
    mod.load()
    return mod


@pytest.fixture(scope="session")
def fa(capi):
    return importlib.import_module("flash_attention_triton_amd")


@pytest.fixture(scope="session")
def fa2_module(capi):
    return importlib.import_module("flash-attention-triton_amd.flash_attention_2")


@pytest.fixture(scope="session")
def workloads():
    return importlib.import_module("flash-attention-triton_amd.workloads")
