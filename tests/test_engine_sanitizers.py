"""The engine's host logic under the host sanitizers: tests/support/sanitize_main.cpp drives the
simulated-device build (random worlds and knobs, lockstep and one thread per rank, record/replay,
failure handling, point-to-point) in a process of its own, once with AddressSanitizer +
UndefinedBehaviorSanitizer and once, every world threaded, with ThreadSanitizer.  Any report fails
the run (halt_on_error / a non-zero exit status)."""
import os
import shutil
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(ROOT, "allreduce-proto_amd", "csrc")
SUPPORT = os.path.join(HERE, "support")


def build(tmp_path, name, sanitize):
    cxx = shutil.which("g++")
    if not cxx:
        pytest.skip("no g++")
    exe = str(tmp_path / name)
    cmd = [cxx, "-O1", "-g", "-std=c++17", "-fno-omit-frame-pointer", "-pthread", "-fsanitize=" + sanitize,
           "-I", CSRC, "-I", SUPPORT, "-o", exe, os.path.join(SUPPORT, "sanitize_main.cpp"), os.path.join(SUPPORT, "sim_world.cpp")]
    p = subprocess.run(cmd, capture_output=True, text=True)
    if p.returncode != 0 and ("cannot find -l" in p.stderr or "unrecognized" in p.stderr):
        pytest.skip("sanitizer runtime not installed: " + p.stderr.strip().splitlines()[-1])
    assert p.returncode == 0, p.stderr[-3000:]
    return exe


def run(exe, args, **env):
    e = dict(os.environ)
    e.update(env)
    p = subprocess.run([exe] + [str(a) for a in args], env=e, capture_output=True, text=True, timeout=600)
    if p.returncode != 0 and "does not come first in initial library list" in p.stderr:
        pytest.skip("another preloaded library keeps the sanitizer runtime from loading first")
    return p


def test_address_and_undefined_behaviour_sanitizers(tmp_path):
    exe = build(tmp_path, "asan_sim", "address,undefined")
    p = run(exe, [16, 0], ASAN_OPTIONS="detect_leaks=1:halt_on_error=1", UBSAN_OPTIONS="halt_on_error=1:print_stacktrace=1")
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-4000:])
    assert "bad 0" in p.stdout and "ERROR" not in p.stderr and "runtime error" not in p.stderr


def test_thread_sanitizer_with_one_thread_per_rank(tmp_path):
    exe = build(tmp_path, "tsan_sim", "thread")
    p = run(exe, [12, 1, 0], TSAN_OPTIONS="halt_on_error=1")
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-4000:])
    assert "bad 0" in p.stdout and "ThreadSanitizer" not in p.stderr
