#!/usr/bin/env python3
"""Writes tests/golden/allreduce_golden.json: known answers for the two allreduce schedules.

The reference ships no fixture files for this path, so these vectors are derived from what the
schedules must compute, using numpy only (no code of the oracle or of the HIP library is involved):
inputs come from numpy's PCG64 with the seeds below, the expected result is the ring left fold that
starts at the owner of each element's chunk group, or the balanced pairwise tree over rank index,
evaluated with explicit numpy float32/int32 adds.  Stored per case: SHA-256 of the result's bytes and
its first and last four elements (as raw bit patterns).  Regenerate with `python tests/golden/make_golden.py`.
"""
import hashlib
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
from oracle_lib import np_ring, np_tree  # numpy closed forms only  # noqa: E402

CASES = [
    # algo, ranks, elements, IBCOMM_CHUNKSIZE, dtype, scale
    ("ring", 2, 2521, None, "float32", 1.0),
    ("ring", 3, 1003, None, "float32", 1.0),
    ("ring", 4, 65543, None, "float32", 1.0),
    ("ring", 4, 65536, 4096, "float32", 1.0),
    ("ring", 5, 1003, 40, "float32", 1e-3),
    ("ring", 8, 262151, None, "float32", 1.0),
    ("ring", 8, 262144, 8192, "float32", 1.0),
    ("ring", 4, 4099, None, "int32", 3e8),
    ("rabenseifner", 2, 2521, None, "float32", 1.0),
    ("rabenseifner", 4, 65543, None, "float32", 1e-2),
    ("rabenseifner", 8, 262151, None, "float32", 1e-2),
    ("rabenseifner", 8, 262144, 8192, "float32", 1e-2),
    ("rabenseifner", 16, 1048583, 16384, "float32", 1e-2),
    ("rabenseifner", 4, 4099, None, "int32", 3e8),
]


def inputs(case_index, ranks, n, dtype, scale):
    return [(np.random.default_rng(7000 + 100 * case_index + r).standard_normal(n) * scale).astype(dtype)
            for r in range(ranks)]


def main():
    out = []
    for k, (algo, ranks, n, chunk, dtype, scale) in enumerate(CASES):
        bufs = inputs(k, ranks, n, dtype, scale)
        want = np_ring(bufs, chunk) if algo == "ring" else np_tree(bufs)
        bits = want.view(np.uint32)
        out.append({"case": k, "algo": algo, "ranks": ranks, "elements": n, "chunksize": chunk, "dtype": dtype, "scale": scale,
                    "sha256": hashlib.sha256(want.tobytes()).hexdigest(),
                    "head_bits": [int(x) for x in bits[:4]], "tail_bits": [int(x) for x in bits[-4:]]})
    with open(os.path.join(HERE, "allreduce_golden.json"), "w") as f:
        json.dump(out, f, indent=1)
    print("wrote %d cases" % len(out))


if __name__ == "__main__":
    main()
