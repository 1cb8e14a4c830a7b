"""The loopback counterpart of the reference's example program (examples/allreduce.cpp), built on the
drop-in C++ header: every rank must print "rank: r OK" (its result equals the exact integer sum),
rank 0's time is reported in the reference's format, and the exit status counts failed ranks."""
import os
import re
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXAMPLE = os.path.join(ROOT, "allreduce-proto_amd", "allreduce_example")


def run(*args, chunksize=None, **extra_env):
    assert os.path.exists(EXAMPLE), "build the example first (__graft_entry__.build())"
    env = dict(os.environ)
    env.update(extra_env)
    env.pop("IBCOMM_CHUNKSIZE", None)
    if chunksize is not None:
        env["IBCOMM_CHUNKSIZE"] = str(chunksize)
    p = subprocess.run(["timeout", "120s", EXAMPLE] + [str(a) for a in args], env=env, capture_output=True, text=True)
    return p.returncode, p.stdout, p.stderr


@pytest.mark.parametrize("np_,algo,n", [(4, "ring", 4194304), (8, "ring", 1048577), (8, "rabenseifner", 2097152),
                                        (3, "ring", 1000003), (1, "ring", 4096)])
def test_every_rank_reports_ok(np_, algo, n):
    rc, out, err = run(np_, algo, n)
    assert rc == 0, (out[-2000:], err[-2000:])
    lines = out.splitlines()
    assert lines[:np_] == ["rank: %d OK" % r for r in range(np_)]
    m = re.fullmatch(r"elapsed time : (\d\.\d{6}e[-+]\d\d) \[s\]", lines[np_])
    assert m and float(m.group(1)) > 0


def test_reference_sized_run_with_its_chunking():
    # 256 MiB per rank as in the reference example (ARRAY_LENGTH 67108864), 8 ranks, 8 MiB chunks
    rc, out, err = run(8, "ring", 67108864, chunksize=8388608)
    assert rc == 0, (out[-2000:], err[-2000:])
    assert out.count(" OK") == 8


@pytest.mark.parametrize("algo", ["ring", "rabenseifner"])
def test_several_timed_runs_through_the_blocking_calls(algo):
    # the optional fourth argument repeats the timed call: 3 warm-ups (eager, recorded, replayed) and 6 more replays of
    # the world the 8 rank threads' blocking calls meet in; every rank still checks every element of its last result
    rc, out, err = run(8, algo, 4194304, 6, chunksize=1048576)
    assert rc == 0, (out[-2000:], err[-2000:])
    lines = out.splitlines()
    assert lines[:8] == ["rank: %d OK" % r for r in range(8)]
    first = float(lines[8].split(":")[1].split()[0])
    m = re.fullmatch(r"elapsed times of 6 timed runs \[s\] :((?: \d\.\d{6}e[-+]\d\d){6})", lines[9])
    assert m, lines[9]
    runs = [float(x) for x in m.group(1).split()]
    assert runs[0] == first and all(0 < t < 0.1 for t in runs)
    # with one engine per rank thread instead of the meeting point the program behaves the same
    rc, out2, err2 = run(4, algo, 1048576, 2, IBCOMM_HIP_RENDEZVOUS="0")
    assert rc == 0, (out2[-2000:], err2[-2000:])
    assert out2.count(" OK") == 4


def test_library_errors_end_the_process_with_the_reference_codes():
    rc, _, err = run(3, "rabenseifner", 4096)  # not a power of two: NOT_SUPPORTED
    assert rc == 4 and "Error occured at" in err
    rc, _, err = run(4, "ring", 4096, chunksize=3)  # not a multiple of sizeof(float): INVALID_ARGUMENT
    assert rc == 1
    rc, _, _ = run(4, "bogus", 4096)
    assert rc == 1
    rc, _, _ = run(4, "ring", 4096, 0)  # no timed run at all
    assert rc == 1


def test_the_example_names_every_public_call_of_the_bring_up():
    # PrepareMemoryPool() is public in the reference's class under USE_CUDA (ibverbs_communicator.h:116):
    # the example calls it, so the binary that the tests above ran was compiled against a header that has it
    src = open(os.path.join(ROOT, "allreduce-proto_amd", "examples", "allreduce.cpp")).read()
    assert "->PrepareMemoryPool()" in src
    hdr = open(os.path.join(ROOT, "allreduce-proto_amd", "ibcomm", "ibverbs_communicator.h")).read()
    assert "void PrepareMemoryPool()" in hdr
