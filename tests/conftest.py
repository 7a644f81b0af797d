import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU and the built libsjhip.so (run on MI355X)")


@pytest.fixture(scope="session")
def c_oracle():
    """The C restatement of the oracle, built on demand (gcc, a second or two)."""
    import subprocess

    from oracle import c_oracle as co

    if not co.available():
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    co.load()
    return co
