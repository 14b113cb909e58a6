"""The decode kernels' launch shape can be overridden through environment variables the host library reads once per
process (measurement switches). Every switch selects code that must stay correct: each setting runs the same decode
shapes against the oracle in a process of its own, one after the other."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.parametrize("env", [
    {"RLX_GEMV_WAVES": "4"},
    {"RLX_GEMV_WAVES": "16", "RLX_GEMV_WGS_PER_CU": "1"},
    {"RLX_GEMV_CONTIGUOUS": "1"},
    {"RLX_GEMV_KW": "4"},
    {"RLX_GEMV_KW": "0"},
    {"RLX_GEMV_UPI": "1"},
], ids=lambda e: ",".join(f"{k}={v}" for k, v in e.items()))
def test_gemv_measurement_switch(env):
    print("switch", env, flush=True)
    full = dict(os.environ)
    full.update(env)
    r = subprocess.run([sys.executable, "-u", os.path.join(HERE, "gemv_knob_case.py")], env=full, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "knob case ok" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
