"""Committed known answers (tests/golden/allreduce_golden.json, made by tests/golden/make_golden.py from
numpy closed forms) against the CPU oracle and, on a GPU, against the HIP library."""
import hashlib
import json
import os

import numpy as np
import pytest

import oracle_lib as O

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = json.load(open(os.path.join(HERE, "golden", "allreduce_golden.json")))


def inputs(g):
    return [(np.random.default_rng(7000 + 100 * g["case"] + r).standard_normal(g["elements"]) * g["scale"]).astype(g["dtype"])
            for r in range(g["ranks"])]


def matches(result, g):
    bits = result.view(np.uint32)
    return (hashlib.sha256(result.tobytes()).hexdigest() == g["sha256"] and [int(x) for x in bits[:4]] == g["head_bits"]
            and [int(x) for x in bits[-4:]] == g["tail_bits"])


@pytest.mark.parametrize("g", GOLDEN, ids=lambda g: "%s-%d-%d-%s" % (g["algo"], g["ranks"], g["elements"], g["chunksize"]))
def test_oracle_reproduces_golden(g):
    algos = (O.RING_CPU, O.RING_GPU) if g["algo"] == "ring" else (O.RABEN_GPU,)
    for algo in algos:
        rc, recv, _ = O.allreduce(algo, inputs(g), g["chunksize"])
        assert rc == 0
        for r in range(g["ranks"]):
            assert matches(recv[r], g), "rank %d" % r


@pytest.mark.gpu
@pytest.mark.parametrize("g", GOLDEN, ids=lambda g: "%s-%d-%d-%s" % (g["algo"], g["ranks"], g["elements"], g["chunksize"]))
def test_hip_reproduces_golden(g):
    torch = pytest.importorskip("torch")
    import gpu_util as G
    import hip_lib as H
    algo = H.RING if g["algo"] == "ring" else H.RABENSEIFNER
    with H.World(g["ranks"]) as w:
        send = G.to_device(inputs(g))
        recv = [G.poisoned_like(t) for t in send]
        assert G.run_world(w, algo, send, recv, g["chunksize"]) == 0, H.last_error()
        for r in range(g["ranks"]):
            assert matches(recv[r].cpu().numpy(), g), "rank %d" % r
        # and one rank through the blocking per-rank calls on threads
        recv2 = [G.poisoned_like(t) for t in send]
        assert G.run_world(w, algo, send, recv2, g["chunksize"], threads=True) == 0, H.last_error()
        assert matches(recv2[g["ranks"] - 1].cpu().numpy(), g)
