"""Host-side contract of the entry points the harness calls (no GPU needed)."""
import importlib
import os
import subprocess
import sys

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(REPO, "bench.py"), *args],
                          capture_output=True, text=True, cwd=REPO, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    for args in (("--gpus", "2"), ("--gpus", "8", "--steps", "3")):
        res = run_bench(*args)
        assert res.returncode != 0
        assert "one GPU" in res.stderr and "--gpus 1" in res.stderr
        assert res.stdout.strip() == ""


def test_a_torchrun_world_is_refused_too():
    env = dict(os.environ, WORLD_SIZE="2", RANK="0", LOCAL_RANK="0")
    res = subprocess.run([sys.executable, os.path.join(REPO, "bench.py")], capture_output=True,
                         text=True, cwd=REPO, timeout=120, env=env)
    assert res.returncode != 0 and "one GPU" in res.stderr


def test_graft_entry_exposes_build_and_smoke():
    sys.path.insert(0, REPO)
    entry = importlib.import_module("__graft_entry__")
    assert callable(entry.build) and callable(entry.smoke)
