import os
import sys

import pytest

# The library's repack cache keys a device-side copy of every weight by its pointers and ends the process when a
# launch finds other data at those addresses.  Tests build and drop weights all the time and the allocator hands the
# same addresses out again, so the suite runs with the cache off (the reference-format kernels are what most tests
# are about); tests/repack_cache_check.py covers the cache in child processes of its own.
os.environ.setdefault("TERNASPMM_REPACK_CACHE", "0")

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def coracle():
    from oracle.terna_oracle import COracle
    return COracle()
