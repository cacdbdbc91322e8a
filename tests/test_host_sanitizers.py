"""The host layer under AddressSanitizer + UBSan on the CPU (mlx-node_amd/examples/host_sanity.cpp):
hyper-parameter casts, LR schedules, table layout, null-argument refusals, and 20,000 mutated
checkpoint headers.  The instrumented binary is built by `python mlx-node_amd/build.py --sanitize`
(a couple of minutes, so not by the default build); without it the test is skipped."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BINARY = os.path.join(ROOT, "mlx-node_amd", "bin", "host_sanity_asan")


def test_host_layer_is_clean_under_asan_and_ubsan():
    if not os.path.exists(BINARY):
        pytest.skip("build it with: python mlx-node_amd/build.py --sanitize")
    env = dict(os.environ, ASAN_OPTIONS="detect_leaks=0:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1")
    proc = subprocess.run([BINARY], capture_output=True, text=True, timeout=600, env=env)
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-4000:]
    assert "host sanity ok" in proc.stdout
