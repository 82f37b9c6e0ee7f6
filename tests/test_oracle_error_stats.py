"""Pins the CPU oracle of error_stats (error_stats.cu:13-75): closed forms and numpy."""
import numpy as np
import pytest

import oracle
from helpers import rng


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_closed_forms(dtype):
    a = np.zeros(1280, dtype)
    b = np.zeros(1280, dtype)
    assert np.array_equal(oracle.error_stats(a, b), np.zeros(3, np.float32))
    b[:] = 0.5                       # constant difference
    assert np.allclose(oracle.error_stats(a, b), [0.25, 0.5, 0.5], rtol=0, atol=0)
    b[:] = 0
    b[77] = -3.0                     # one spike: mse = 9/n, max = 3, mae = 3/n
    assert np.allclose(oracle.error_stats(a, b), [9 / 1280, 3, 3 / 1280], rtol=1e-7)


def test_tail_beyond_the_last_full_multiple_of_128_is_not_visited():
    a = np.zeros(1000, np.float32)   # 1000 = 7 * 128 + 104
    b = np.zeros(1000, np.float32)
    b[896:] = 5.0                    # only unvisited elements differ
    assert np.array_equal(oracle.error_stats(a, b), np.zeros(3, np.float32))
    b[895] = 2.0                     # the last visited one; means still divide by 1000
    assert np.allclose(oracle.error_stats(a, b), [4 / 1000, 2, 2 / 1000], rtol=1e-7)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_against_numpy(dtype):
    g = rng(900)
    n = 128 * 333
    a = g.standard_normal(n).astype(dtype)
    b = (a.astype(np.float64) + g.standard_normal(n) * 0.01).astype(dtype)
    d = (a.astype(np.float32) - b.astype(np.float32)).astype(np.float64)
    want = [np.mean(d ** 2), np.max(np.abs(d)), np.mean(np.abs(d))]
    got = oracle.error_stats(a, b)
    assert np.allclose(got, want, rtol=1e-5) and got[1] == np.float32(want[1])
