"""The plain-C host (mlx-node_amd/examples/cabi_demo.c, built by mlx-node_amd/build.py): known answers
of the reference's own tests through the C ABI with no Python in between, and the cost of the
updateSingle-per-tensor loop against one update_many call from compiled host code; the region-interleaved pool,
the allocation-free norm and the asynchronous engine call from plain C."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEMO = os.path.join(ROOT, "mlx-node_amd", "bin", "cabi_demo")


def test_plain_c_host_known_answers_and_timing():
    assert os.path.exists(DEMO), "run `python mlx-node_amd/build.py` first"
    proc = subprocess.run([DEMO], capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    passed = [l for l in proc.stdout.splitlines() if l.startswith("PASS")]
    assert len(passed) == 9, proc.stdout
    pool = re.search(r"POOL regions=(\d+) .* mix43_plain_gbps=(\d+) mix43_arena_gbps=(\d+)", proc.stdout)
    assert pool and int(pool.group(1)) >= 1, proc.stdout
    if int(pool.group(1)) >= 2:      # most of the device free: the arena is no slower than plain memory, which may have been lucky
        assert int(pool.group(3)) > 0.92 * int(pool.group(2)), proc.stdout
    m = re.search(r"TIMING tensors=(\d+) elements=(\d+) update_single_loop_ms=([\d.]+) \(host enqueue ([\d.]+)\) "
                  r"update_many_ms=([\d.]+)", proc.stdout)
    assert m, proc.stdout
    assert int(m.group(1)) == 310 and int(m.group(2)) == 596_049_920
    single, many = float(m.group(3)), float(m.group(5))
    print(proc.stdout)
    # 16.7 GB per step: neither path may be slower than 1.5 TB/s, the per-tensor loop within 2.5x of one launch
    assert many < 11.0 and single < 2.5 * many + 2.0
