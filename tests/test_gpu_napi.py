"""The JavaScript surface (mlx-node_amd/napi/mxopt_napi.c -> bin/mxopt.node) driven by node: the
reference's optimizer, GradientUtils, LRScheduler and accumulateGradients expectations, restated in
tests/js/optimizer_api.test.js against the same class and method names."""
import os
import shutil
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ADDON = os.path.join(ROOT, "mlx-node_amd", "bin", "mxopt.node")


def test_javascript_api():
    node = shutil.which("node")
    if node is None or not os.path.exists(ADDON):
        pytest.skip("node or the built addon is missing")
    proc = subprocess.run([node, os.path.join(ROOT, "tests", "js", "optimizer_api.test.js")], capture_output=True,
                          text=True, timeout=300)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "0 failed" in proc.stdout and proc.stdout.count("PASS") >= 20
