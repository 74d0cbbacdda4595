import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def golden_ttir(name):
    with open(os.path.join(GOLDEN, name + ".ttir")) as f:
        return f.read()


@pytest.fixture(scope="session")
def native():
    """The C-ABI library through its ctypes binding (must be built: it is the product)."""
    import triton_shared_amd as tsa
    tsa._native.lib()
    return tsa._native


@pytest.fixture(scope="session")
def oracle_cpu():
    """The CPU restatement (test infrastructure); built on first use."""
    from oracle import cpu
    cpu.lib()
    return cpu


def plan_for(native, ttir_name):
    structured = native.ttir_to_structured(golden_ttir(ttir_name))
    plan_bytes, name = native.structured_to_plan(structured)
    return native.PlanHandle(plan_bytes), structured
