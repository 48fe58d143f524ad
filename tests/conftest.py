"""pytest configuration: the ``gpu`` marker and shared fixtures.

``-m "not gpu"`` runs on a CPU-only host (oracle checks, host logic, C-ABI
symbol export).  ``-m gpu`` needs one MI355X and calls the kernels through the
C ABI; it fails, rather than skips, when the library is not built.
"""

from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) and the built libhipengine_gfx950.so")


@pytest.fixture(scope="session")
def dev():
    """Device session: HIP runtime + loaded kernel library (gpu tests only)."""
    from tests._device import Device

    return Device()
