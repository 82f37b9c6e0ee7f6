"""Pins the CPU oracle of softmax_rows (normalize.cu:147-220) without the reference: closed
forms, invariants and an independent float64 evaluation."""
import numpy as np
import pytest

import oracle
from helpers import rng, ulp_diff_f16


def f64_softmax(x, temp):
    v = x.astype(np.float64) / np.float64(np.float32(temp))
    e = np.exp(v - v.max(axis=-1, keepdims=True))
    return e / e.sum(axis=-1, keepdims=True)


@pytest.mark.parametrize("mode", [0, 1])
def test_closed_forms(mode):
    # a uniform row of 2^k entries is exactly 2^-k
    for w in (1, 2, 64, 1024):
        x = np.full((3, w), 0.37, np.float16)
        assert np.all(oracle.softmax_rows(x, 1.0, mode) == np.float16(1.0 / w))
    # two values a, b: the logistic function of their difference
    x = np.array([[1.5, -0.25]], np.float16)
    p = 1.0 / (1.0 + np.exp(-(1.5 + 0.25) / 0.7))
    got = oracle.softmax_rows(x, 0.7, mode).astype(np.float64)
    assert abs(got[0, 0] - p) <= 2.0 ** -11 and abs(got[0, 1] - (1 - p)) <= 2.0 ** -11
    # -inf entries (the causal mask) are exactly zero, the rest renormalise
    x = np.array([[0.5, -np.inf, 0.5, -np.inf]], np.float16)
    assert np.array_equal(oracle.softmax_rows(x, 1.0, mode), np.array([[0.5, 0, 0.5, 0]], np.float16))
    # a dominant entry: 1 and zeros (exp underflows)
    x = np.array([[60000.0, 0.0, -60000.0]], np.float16)
    assert np.array_equal(oracle.softmax_rows(x, 1.0, mode), np.array([[1, 0, 0]], np.float16))


@pytest.mark.parametrize("w", [1, 7, 255, 256, 257, 2048, 3000])
@pytest.mark.parametrize("temp", [1.0, 0.5, 3.0])
def test_against_float64_and_invariants(w, temp):
    g = rng(700 + w)
    x = (g.standard_normal((5, w)) * 3).astype(np.float16)
    want = f64_softmax(x, temp)
    for mode in (0, 1):
        got = oracle.softmax_rows(x, temp, mode)
        assert np.max(ulp_diff_f16(got, want.astype(np.float16))) <= 1, mode
        assert np.allclose(got.astype(np.float64).sum(-1), 1.0, atol=w * 2.0 ** -12 + 1e-3)
    # the reference order (mode 0) and float64 (mode 1) agree within one fp16 step
    assert np.max(ulp_diff_f16(oracle.softmax_rows(x, temp, 0), oracle.softmax_rows(x, temp, 1))) <= 1
    # temperature: softmax(x, T) == softmax(x / T, 1) when the division by T is exact
    if temp == 0.5:
        small = (x / 4).astype(np.float16)
        assert np.array_equal(oracle.softmax_rows(small, 0.5, 1), oracle.softmax_rows(small * 2, 1.0, 1))
    # order: a permutation of the row permutes the result (float64 mode is order independent
    # up to summation order; compare within one step)
    perm = g.permutation(w)
    assert np.max(ulp_diff_f16(oracle.softmax_rows(x[:, perm], temp, 1),
                               oracle.softmax_rows(x, temp, 1)[:, perm])) <= 1
