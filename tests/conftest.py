"""Shared pytest setup: registers the ``gpu`` marker and exposes the golden literals."""

import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def literals():
    with open(os.path.join(ROOT, "tests", "golden", "reference_literals.json")) as f:
        return json.load(f)


@pytest.fixture(autouse=True)
def _kernel_choice_back_to_auto():
    """Tests that pin one of two bit-identical kernels leave the process-wide choice at its default."""
    yield
    from relax_amd import _lib

    _lib.lib.relax_amd_set_kernel_choice(_lib.KERNEL_CHOICES["auto"])
