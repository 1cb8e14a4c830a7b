"""Pins the oracle's restatement of ibcomm/util.h (ceilDiv, GetExpOfTwo, error codes)."""
import pytest

import oracle_lib as O


def test_get_exp_of_two_reference_known_answers():
    # tests/unittest.cpp:65-71 (written there against the old name get_exp_of_two)
    L = O.lib()
    assert L.orc_get_exp_of_two(0) == 0
    assert L.orc_get_exp_of_two(2) == 1
    assert L.orc_get_exp_of_two(128) == 7
    assert L.orc_get_exp_of_two(127) == 0
    assert L.orc_get_exp_of_two(129) == 0


def test_get_exp_of_two_is_log2_on_powers_and_zero_elsewhere():
    L = O.lib()
    for n in range(0, 5000):
        want = n.bit_length() - 1 if n > 0 and n & (n - 1) == 0 else 0
        assert L.orc_get_exp_of_two(n) == want  # note: 1 -> 0, same as "not a power"
    assert L.orc_get_exp_of_two(1 << 30) == 30


def test_ceil_div_closed_form():
    L = O.lib()
    for a in list(range(0, 200)) + [2521, 67108864, 536870911, 2**40 + 1]:
        for b in [1, 2, 3, 4, 7, 8, 16, 128, 316, 2097152]:
            assert L.orc_ceil_div(a, b) == -(-a // b)


def test_error_code_values():
    # tests/allreduce_test.py:13-16 and ibcomm/util.h:32-42
    assert (O.INVALID_ARGUMENT, O.IBVERBS_ERROR, O.CUDA_ERROR, O.NOT_SUPPORTED) == (1, 2, 3, 4)


def test_against_reference_util_h_build():
    R = O.ref_util()
    if R is None:
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    L = O.lib()
    for n in range(-3, 70000):
        if n < 0:
            continue  # n % 2 on negatives never reaches 1 in the reference; not a meaningful input
        assert L.orc_get_exp_of_two(n) == R.ref_get_exp_of_two(n)
    for a in range(0, 300):
        for b in range(1, 40):
            assert L.orc_ceil_div(a, b) == R.ref_ceil_div(a, b)
    assert [R.ref_error_code(i) for i in range(4)] == [1, 2, 3, 4]
