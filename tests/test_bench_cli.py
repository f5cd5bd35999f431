"""bench.py's command line on a machine without a GPU: the one-GPU contract and the help text."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused():
    r = run("--gpus", "2")
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""
    env = dict(os.environ, WORLD_SIZE="2")
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")], capture_output=True, text=True, timeout=120, env=env)
    assert r.returncode == 2 and "one GPU" in r.stderr


def test_help_lists_the_workloads_and_switches():
    r = run("--help")
    assert r.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--config", "--matrix", "--rcm", "--wide", "--unfused", "--host-buffers"):
        assert flag in r.stdout
