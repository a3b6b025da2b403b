"""Philox4x32-10 against the published Random123 known-answer vectors, and the
derived Bernoulli/uniform helpers against their stated distributions."""

import numpy as np
import pytest

from oracle import gtm_oracle as o

KAT = [
    ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
    ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
    ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0),
     (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
]


@pytest.mark.parametrize("counter,key,want", KAT)
def test_known_answers(counter, key, want):
    got = o.philox4x32(*counter, *key)
    assert tuple(int(x) for x in got) == want


def test_vectorised_equals_scalar():
    c0 = np.arange(7)
    got = o.philox4x32(c0, 3, 9, 4, 123, 456)
    for i in range(7):
        one = o.philox4x32(i, 3, 9, 4, 123, 456)
        assert [int(g[i]) for g in got] == [int(x) for x in one]


def test_feedback_threshold_values():
    assert o.feedback_threshold(1.0) == 65536  # s = 1: every bit set
    assert o.feedback_threshold(10.0) == 6553
    assert o.feedback_threshold(0.5) == 65536
    assert o.q_threshold(1.0, 2) == 2**32 and o.q_threshold(1.0, 11) == int(0.1 * 2**32)


@pytest.mark.parametrize("s", [1.0, 2.0, 10.0, 15.0])
def test_feedback_bits_are_bernoulli_one_over_s(s):
    bits = o.feedback_bits(seed=99, step=5, bank_id=0, class_id=3, clauses=400, chunks=8, threshold16=o.feedback_threshold(s))
    ones = int(o._popcount32(bits).sum())
    n = 400 * 8 * 32
    p = 1.0 / s
    if s == 1.0:
        assert ones == n
    else:
        assert abs(ones - n * p) < 5 * np.sqrt(n * p * (1 - p))
    # different classes / steps / banks give different streams
    other = o.feedback_bits(99, 5, 0, 4, 400, 8, o.feedback_threshold(2.0))
    assert not np.array_equal(other, o.feedback_bits(99, 5, 1, 4, 400, 8, o.feedback_threshold(2.0)))
    assert not np.array_equal(other, o.feedback_bits(99, 6, 0, 4, 400, 8, o.feedback_threshold(2.0)))
