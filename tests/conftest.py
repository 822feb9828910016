import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X; runs the HIP path through the C-ABI")


@pytest.fixture(scope="session")
def oracle():
    from oracle.load import load_oracle
    return load_oracle()


@pytest.fixture(scope="session")
def reference():
    """The reference's own C path (oracle/_ref), or None where it was not built."""
    from oracle.load import load_reference
    return load_reference()


@pytest.fixture(scope="session")
def product():
    """The shipped library.  GPU tests must run the HIP path: no device is an error, not a skip."""
    import picoforge_amd as pf
    api = pf.load_product()
    assert api.hip.device_count() >= 1, "no HIP device visible: GPU tests cannot run"
    return api


@pytest.fixture(scope="session")
def product_host():
    """The shipped library for tests of its host logic: no device needed, none assumed."""
    import picoforge_amd as pf
    return pf.load_product()


@pytest.fixture(scope="session")
def synth():
    import picoforge_amd as pf
    return pf.Synth()
