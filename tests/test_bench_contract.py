"""The command-line contract of bench.py that can be checked without a GPU."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*args, env=None):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          timeout=120, env=env)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = _run("--gpus", "2")
    assert r.returncode != 0
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_a_multi_rank_launch_is_refused():
    r = _run(env=dict(os.environ, WORLD_SIZE="2", RANK="0"))
    assert r.returncode != 0
    assert "one GPU" in r.stderr


def test_the_timed_loop_is_documented_in_the_line():
    """the run-in before the timed loops is reported, not hidden"""
    src = open(os.path.join(ROOT, "bench.py")).read()
    assert '"settle_s": SETTLE_S' in src and '"steps": a.steps' in src and '"warmup": a.warmup' in src
