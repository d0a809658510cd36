"""Shared test configuration.

``-m "not gpu"`` runs everything that needs no device: the oracles against their golden vectors
and closed forms, the host policy, and the C ABI's load / symbol / argument-checking surface.
``-m gpu`` runs the parity tests proper on an MI355X, every one of them through the C ABI.
"""

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_policy():
    import json
    return json.loads((ROOT / "tests" / "golden" / "policy_a100.json").read_text())


@pytest.fixture(scope="session")
def hip_lib():
    """The loaded C-ABI library; built here only if the tree does not hold it yet."""
    from mlir_roller_amd import hip
    if not hip.LIB_PATH.exists():
        hip.build_library()
    return hip.lib()


@pytest.fixture(scope="session")
def device(hip_lib):
    """Initialised GPU context (gpu-marked tests only)."""
    from mlir_roller_amd import hip
    hip.init(0)
    return hip.device_info()
