"""Pins orc_reduce_inplace (allreduce_cpu_impl.h:16-21) against numpy's IEEE-754 / wrapping adds."""
import numpy as np

import oracle_lib as O


def run(dtype_code, a, b):
    r = a.copy()
    O.lib().orc_reduce_inplace(dtype_code, r.ctypes.data, b.ctypes.data, r.size)
    return r


def test_f32_random_bit_exact():
    rng = np.random.default_rng(1)
    for n in (0, 1, 3, 4, 5, 127, 1000, 65537):
        a = rng.standard_normal(n).astype(np.float32) * np.float32(1e3)
        b = rng.standard_normal(n).astype(np.float32)
        assert np.array_equal(O.bits(run(O.F32, a, b)), O.bits(a + b))


def test_f32_special_values():
    tiny = np.float32(1e-45)          # smallest denormal
    dn = np.float32(5.9e-39)          # denormal
    mx = np.finfo(np.float32).max
    a = np.array([0.0, -0.0, -0.0, tiny, dn, mx, -mx, np.inf, 1.0, 16777216.0, 1e-38], dtype=np.float32)
    b = np.array([-0.0, -0.0, 0.0, tiny, dn, mx, -mx, 1.0, -1.0, 1.0, -1.1e-38], dtype=np.float32)
    with np.errstate(over="ignore"):
        want = a + b
    got = run(O.F32, a, b)
    assert np.array_equal(O.bits(got), O.bits(want))
    assert got[3] == np.float32(2.8e-45) and got[3] != 0  # denormals are kept, not flushed
    assert np.isinf(got[5]) and np.isinf(got[6])
    assert got[9] == np.float32(16777216.0)               # round-to-nearest-even at 2^24 + 1


def test_f32_nan_propagates():
    a = np.array([np.nan, 1.0, np.inf], dtype=np.float32)
    b = np.array([1.0, np.nan, -np.inf], dtype=np.float32)
    assert np.isnan(run(O.F32, a, b)).all()


def test_f64_bit_exact():
    rng = np.random.default_rng(2)
    a = rng.standard_normal(5001)
    b = rng.standard_normal(5001) * 1e-9
    assert np.array_equal(O.bits(run(O.F64, a, b)), O.bits(a + b))


def test_integers_wrap():
    a = np.array([2**31 - 1, -2**31, 5, -7], dtype=np.int32)
    b = np.array([1, -1, 6, 7], dtype=np.int32)
    with np.errstate(over="ignore"):
        assert np.array_equal(run(O.I32, a, b), a + b)
    assert run(O.I32, a, b)[0] == -2**31
    a = np.array([2**63 - 1, 11], dtype=np.int64)
    b = np.array([1, 31], dtype=np.int64)
    with np.errstate(over="ignore"):
        assert np.array_equal(run(O.I64, a, b), a + b)
