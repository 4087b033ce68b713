"""The configuration an unmodified call site runs: no environment variable, the repack cache on.  The suite's own
process switches the cache off (tests/conftest.py), so each BitNet-2B matrix is checked in a child process with the
library's defaults: tests/default_config_check.py holds the cases."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("n,k,ws_num", [(3840, 2560, 3), (2560, 2560, 1), (13824, 2560, 2), (2560, 6912, 1)])
def test_reference_symbols_with_library_defaults(n, k, ws_num):
    env = {key: val for key, val in os.environ.items() if not key.startswith("TERNASPMM_")}
    r = subprocess.run([sys.executable, "-u", "-m", "tests.default_config_check", str(n), str(k), str(ws_num)], cwd=ROOT,
                       env=env, capture_output=True, text=True, timeout=600)
    assert r.returncode == 0 and "default configuration check ok" in r.stdout, r.stdout[-3000:] + r.stderr[-3000:]
