import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def oracle():
    import oracle_bind
    return oracle_bind.load()


@pytest.fixture(scope="session")
def gpu():
    """The HIP backend.  No fallback: a missing library or device is an error."""
    from granite_amd import get_hip_compute
    hc = get_hip_compute(0)
    print(f"[gpu] {hc.device_info().name.decode()} ({hc.device_info().arch.decode()})", flush=True)
    return hc
