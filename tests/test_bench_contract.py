"""What bench.py promises without a GPU: it is a one-GPU, one-process benchmark and says so."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def run(*args, **env):
    e = dict(os.environ)
    e.update(env)
    return subprocess.run([sys.executable, BENCH] + list(args), env=e, capture_output=True, text=True, timeout=120)


def test_more_than_one_gpu_is_refused_with_a_message():
    p = run("--gpus", "2")
    assert p.returncode == 2 and "one GPU only" in p.stderr and p.stdout == ""
    p = run("--gpus", "8", "--steps", "5", "--warmup", "1")
    assert p.returncode == 2 and "--gpus 1" in p.stderr


def test_launch_under_a_multi_process_launcher_is_refused():
    p = run(WORLD_SIZE="2", RANK="0", LOCAL_RANK="0")
    assert p.returncode == 2 and "single-process" in p.stderr


def test_flags_of_the_contract_are_accepted():
    p = run("--help")
    assert p.returncode == 0
    for flag in ("--gpus", "--steps", "--warmup", "--config", "--only-roofline", "--sweep"):
        assert flag in p.stdout
