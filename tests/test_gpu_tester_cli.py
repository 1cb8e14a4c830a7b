"""The reference's integration tests (tests/allreduce_test.py:102-235), case for case, against the
loopback tester built on the drop-in C++ header (allreduce-proto_amd/examples/allreduce_tester.cpp).

The reference starts `mpiexec -np N allreduce_tester algo size init check` and asserts on the exit
status; here N is the tester's first argument and the ranks are threads sharing the GPU.  The element
type is int, the default vectors are init `i*np+p`, check `i*np*np+np*(np-1)/2`.
"""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TESTER = os.path.join(ROOT, "allreduce-proto_amd", "allreduce_tester")

IBCOMM_INVALID_ARGUMENT = 1
IBCOMM_NOT_SUPPORTED = 4
ALGO_RING = "ring"
ALGO_RABEN = "rabenseifner"


def check(np, algo, buffsize, init_expr="i*np+p", check_expr="i*np*np+np*(np-1)/2", chunksize=None):
    assert os.path.exists(TESTER), "build the tester first (__graft_entry__.build())"
    env = dict(os.environ)
    env.pop("IBCOMM_CHUNKSIZE", None)
    if chunksize is not None:
        env["IBCOMM_CHUNKSIZE"] = str(chunksize)
    cmd = ["timeout", "90s", TESTER, str(np), algo, str(buffsize), init_expr, check_expr]
    return subprocess.run(cmd, env=env, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL).returncode


def test_1proc():
    assert check(algo=ALGO_RING, np=1, buffsize=1024) == 0
    assert check(algo=ALGO_RABEN, np=1, buffsize=1024) == 0


def test_small_buffer():
    int_size = 4
    for NP in (1, 2, 3, 5):
        assert check(algo=ALGO_RING, np=NP, buffsize=NP * 2 * int_size) == 0
    assert check(algo=ALGO_RING, np=2, buffsize=2521 * int_size) == 0
    for NP in (1, 2):
        assert check(algo=ALGO_RABEN, np=NP, buffsize=NP * 2 * int_size) == 0
    for NP in (3, 5):  # non-power-of-2 np is not supported
        assert check(algo=ALGO_RABEN, np=NP, buffsize=NP * 2 * int_size) == IBCOMM_NOT_SUPPORTED
    assert check(algo=ALGO_RABEN, np=2, buffsize=2521 * int_size) == 0


def test_basic():
    for NP in (2, 3, 4):
        assert check(algo=ALGO_RING, np=NP, buffsize="128M") == 0
    assert check(algo=ALGO_RABEN, np=2, buffsize="128M") == 0
    assert check(algo=ALGO_RABEN, np=3, buffsize="128M") == IBCOMM_NOT_SUPPORTED
    assert check(algo=ALGO_RABEN, np=4, buffsize="128M") == 0


def test_chunk_size():
    for chunk in ("4", "8", "16", "32", "64", "128"):
        assert check(algo=ALGO_RING, np=4, buffsize="1k", chunksize=chunk) == 0


def test_invalid_error():
    for chunk_size in range(0, 4):
        assert check(algo=ALGO_RING, np=4, buffsize="1k", chunksize=chunk_size) == IBCOMM_INVALID_ARGUMENT
    assert check(algo=ALGO_RING, np=4, buffsize="1k", chunksize="-128") == IBCOMM_INVALID_ARGUMENT
    assert check(algo=ALGO_RING, np=4, buffsize="1k", chunksize="1k") == IBCOMM_INVALID_ARGUMENT
    assert check(algo=ALGO_RING, np=2, buffsize=4, init_expr="1", check_expr="np") == IBCOMM_NOT_SUPPORTED
    assert check(algo=ALGO_RABEN, np=2, buffsize=4, init_expr="1", check_expr="np") == IBCOMM_NOT_SUPPORTED


def test_a_wrong_answer_is_reported_in_the_exit_status():
    # every rank's check fails -> exit status = number of ranks (allreduce_tester.cpp:396-405)
    assert check(algo=ALGO_RING, np=4, buffsize="1k", check_expr="i*np*np+1") == 4


@pytest.mark.slow
def test_aging():
    # the reference repeats each 100 times (tests/allreduce_test.py:227-235); a few keep the suite short
    for _ in range(3):
        assert check(algo=ALGO_RING, np=4, buffsize="128M") == 0
    for _ in range(3):
        assert check(algo=ALGO_RABEN, np=4, buffsize="128M") == 0
