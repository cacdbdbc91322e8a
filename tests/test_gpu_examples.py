"""The example programs under mlx-node_amd/examples run to completion on the GPU."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_optimizer_step_example_agrees_with_itself():
    """One step taken four ways (per-tensor loop, one launch, folded kernels, deferred accumulation)
    must give bit-identical parameters; the script exits non-zero otherwise."""
    exe = os.path.join(ROOT, "mlx-node_amd", "examples", "optimizer_step.py")
    r = subprocess.run([sys.executable, exe], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("identical") == 4 and "DIFFERENT" not in r.stdout, r.stdout
