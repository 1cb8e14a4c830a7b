"""Point-to-point messaging through self-wired queue pairs: the bring-up of the reference's
tests/sendrecv_test.cpp (one communicator of world size 2 whose queue pair for peer 1 is connected
to its own queue pair for peer 0), driven through the drop-in C++ class by
allreduce-proto_amd/examples/sendrecv_selfloop.cpp."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PROG = os.path.join(ROOT, "allreduce-proto_amd", "sendrecv_selfloop")


def run(*args):
    assert os.path.exists(PROG), "build the examples first (__graft_entry__.build())"
    return subprocess.run(["timeout", "60s", PROG] + list(args), capture_output=True, text=True)


def test_messages_sent_to_one_pair_arrive_on_the_pair_wired_to_it():
    p = run()
    assert p.returncode == 0, (p.stdout[-2000:], p.stderr[-2000:])
    assert "sendrecv_selfloop: OK" in p.stdout


def test_second_nonblocking_send_before_sendwait_is_not_supported():
    # ibcomm/ibverbs_communicator.cpp:375-378: exit status 4 and the reference's message
    p = run("twice")
    assert p.returncode == 4
    assert "SendWait must be called before next non-blocking send." in p.stderr
