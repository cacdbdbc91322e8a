"""bench.py's command line, without a GPU: more than one GPU is refused with a message (this path has no
multi-GPU leg), and without a GPU the benchmark says that the library has no CPU path instead of
measuring something else."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def run(*args):
    return subprocess.run([sys.executable, BENCH, *args], capture_output=True, text=True, timeout=300)


def test_more_than_one_gpu_is_refused():
    r = run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_no_gpu_means_no_number():
    import torch
    if torch.cuda.is_available():
        r = run("--workload", "cfg4", "--steps", "2", "--warmup", "1", "--cpu-sample", "0")
        assert r.returncode == 0, r.stderr
        line = json.loads(r.stdout.strip().splitlines()[-1])
        assert line["unit"] == "steps/s" and line["n_gpus"] == 1 and line["roofline"]["bound"] == "hbm"
        return
    r = run()
    assert r.returncode != 0
    assert "no CPU path" in r.stderr and r.stdout.strip() == ""
