"""MXOPT_LOG: refused calls reach stderr at "error", nothing is printed without the variable.

The counterpart of the reference's env-filtered tracing (crates/mlx-core/src/tracing.rs:3-21)."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

REFUSED_CALL = r"""
import ctypes, os, sys
sys.path.insert(0, os.path.join(%r, "mlx-node_amd"))
from mxopt import _lib
L = _lib.load()
rc = L.mxopt_synchronize(None)
assert rc != 0, rc
print("rc", rc)
""" % ROOT


def run(code, level):
    env = dict(os.environ)
    env.pop("MXOPT_LOG", None)
    if level is not None:
        env["MXOPT_LOG"] = level
    return subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300, env=env)


@pytest.mark.parametrize("level", ["error", "debug"])
def test_refused_call_is_logged(level):
    r = run(REFUSED_CALL, level)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = [l for l in r.stderr.splitlines() if l.startswith("mxopt: ")]
    assert len(lines) == 1 and "error" in lines[0] and "mxopt_synchronize: null context" in lines[0], r.stderr


@pytest.mark.parametrize("level", [None, "off", "nonsense"])
def test_silent_unless_asked(level):
    r = run(REFUSED_CALL, level)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "mxopt:" not in r.stderr, r.stderr


@pytest.mark.gpu
def test_debug_level_names_launches_tables_and_engine_decisions():
    exe = os.path.join(ROOT, "mlx-node_amd", "examples", "optimizer_step.py")
    env = dict(os.environ, MXOPT_LOG="debug")
    r = subprocess.run([sys.executable, exe], capture_output=True, text=True, timeout=300, env=env)
    assert r.returncode == 0, r.stdout + r.stderr
    assert r.stdout.count("identical") == 4, r.stdout
    log = [l for l in r.stderr.splitlines() if l.startswith("mxopt: ")]
    assert any("table built" in l for l in log), r.stderr
    assert any("pending stream(s)" in l for l in log), r.stderr
    assert any("workgroups" in l for l in log), r.stderr
    assert not any("error" in l for l in log), r.stderr
    env.pop("MXOPT_LOG")
    quiet = subprocess.run([sys.executable, exe], capture_output=True, text=True, timeout=300, env=env)
    assert quiet.returncode == 0 and "mxopt:" not in quiet.stderr, quiet.stderr
