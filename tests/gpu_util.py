"""Helpers shared by the GPU tests: device buffers come from torch (plumbing only), every compute
call goes through the C ABI of libibcomm_hip.so, every expected value comes from the CPU oracle or
from plain torch fp32 adds in the reference's association order."""
import os
from contextlib import contextmanager

import numpy as np
import torch

import hip_lib as H
import oracle_lib as O

TORCH_DT = {H.F32: torch.float32, H.I32: torch.int32, H.F64: torch.float64, H.I64: torch.int64}
NP_TO_H = {np.dtype(np.float32): H.F32, np.dtype(np.int32): H.I32, np.dtype(np.float64): H.F64,
           np.dtype(np.int64): H.I64}
ORACLE_ALGO = {H.RING: O.RING_GPU, H.RABENSEIFNER: O.RABEN_GPU}


@contextmanager
def env(**kw):
    """Temporarily set (value) or unset (None) environment knobs such as IBCOMM_CHUNKSIZE."""
    saved = {k: os.environ.get(k) for k in kw}
    try:
        for k, v in kw.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = str(v)
        yield
    finally:
        for k, v in saved.items():
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = v


def to_device(arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrays]


def poisoned_like(t):
    out = torch.empty_like(t)
    out.view(torch.uint8).fill_(0x55)
    return out


def bits_equal(a, b):
    """Bit-exact comparison of two device tensors of the same dtype."""
    it = {4: torch.int32, 8: torch.int64}[a.element_size()]
    return torch.equal(a.view(it), b.view(it))


def run_world(world, algo, send, recv, chunksize=None, threads=False):
    """send/recv: lists of device tensors.  Returns the status code (0 = ok)."""
    n = send[0].numel()
    dt = {torch.float32: H.F32, torch.int32: H.I32, torch.float64: H.F64, torch.int64: H.I64}[send[0].dtype]
    torch.cuda.synchronize()
    with env(IBCOMM_CHUNKSIZE=chunksize):
        if threads:
            rcs, msgs = world.allreduce_threads(algo, dt, [t.data_ptr() for t in send], [t.data_ptr() for t in recv], n)
            rc = next((r for r in rcs if r), 0)
        else:
            rc = world.allreduce_ptrs(algo, dt, [t.data_ptr() for t in send], [t.data_ptr() for t in recv], n)
    torch.cuda.synchronize()
    return rc


def check_against_oracle(world, algo, host_bufs, chunksize=None, threads=False, in_place=False):
    send = to_device(host_bufs)
    recv = send if in_place else [poisoned_like(t) for t in send]
    rc = run_world(world, algo, send, recv, chunksize, threads)
    assert rc == 0, H.last_error()
    orc, want, _ = O.allreduce(ORACLE_ALGO[algo], host_bufs, chunksize)
    assert orc == 0
    for r in range(len(host_bufs)):
        got = recv[r].cpu().numpy()
        assert np.array_equal(O.bits(got), O.bits(want[r])), "rank %d differs from the oracle" % r
    if not in_place:
        for r in range(len(host_bufs)):
            assert np.array_equal(O.bits(send[r].cpu().numpy()), O.bits(host_bufs[r])), "sendbuf of rank %d was modified" % r


def device_ring_fold(send, span, owner):
    """Left fold over ranks starting at `owner` on elements [span), with torch fp32 adds (IEEE, one per hop)."""
    s, e = span
    n = len(send)
    acc = send[owner][s:e].clone()
    for j in range(1, n):
        acc += send[(owner + j) % n][s:e]
    return acc


def device_tree(send, span):
    s, e = span
    level = [t[s:e] for t in send]
    while len(level) > 1:
        level = [level[i] + level[i + 1] for i in range(0, len(level), 2)]
    return level[0]
