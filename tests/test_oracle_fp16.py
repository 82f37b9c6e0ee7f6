"""Pins the oracle's integer-only fp16 soft-float against numpy's float16 (an independent,
correctly-rounded implementation).  CPU only."""
import numpy as np

import oracle
from helpers import rng

import ctypes as C


def _f2h(x32):
    out = np.empty(x32.size, np.uint16)
    oracle.lib().adr_o_f2h_n(out.ctypes.data_as(C.POINTER(C.c_uint16)),
                             x32.ctypes.data_as(C.POINTER(C.c_float)), x32.size)
    return out


def _d2h(x64):
    out = np.empty(x64.size, np.uint16)
    oracle.lib().adr_o_d2h_n(out.ctypes.data_as(C.POINTER(C.c_uint16)),
                             x64.ctypes.data_as(C.POINTER(C.c_double)), x64.size)
    return out


def _same_f16_bits(got_u16, ref_f16):
    ref_u16 = ref_f16.view(np.uint16)
    nan = np.isnan(ref_f16)
    assert np.array_equal(np.isnan(got_u16.view(np.float16)), nan)
    assert np.array_equal(got_u16[~nan], ref_u16[~nan])


def test_h2f_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    out = np.empty(65536, np.float32)
    oracle.lib().adr_o_h2f_n(out.ctypes.data_as(C.POINTER(C.c_float)),
                             bits.ctypes.data_as(C.POINTER(C.c_uint16)), 65536)
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(out), nan)
    assert np.array_equal(out.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])


def test_f2h_random_bit_patterns():
    g = rng(1)
    x = g.integers(0, 2**32, size=2_000_000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    with np.errstate(over="ignore"):
        _same_f16_bits(_f2h(x), x.astype(np.float16))


def test_f2h_half_range_and_subnormals():
    g = rng(2)
    # values spread over the whole fp16 exponent range, including below the smallest subnormal
    e = g.uniform(-30, 17, size=1_000_000)
    x = (np.exp2(e) * g.choice([-1.0, 1.0], size=e.size)).astype(np.float32)
    with np.errstate(over="ignore"):
        _same_f16_bits(_f2h(x), x.astype(np.float16))


def test_d2h_all_midpoints_and_neighbours():
    """Every tie between adjacent fp16 values must go to the even neighbour; a nudge either
    way must go to the nearer one.  Covers normal, subnormal, carry into the next binade and
    overflow to infinity."""
    pos = np.arange(0, 0x7C00, dtype=np.uint16)  # all finite non-negative fp16
    lo = pos.view(np.float16).astype(np.float64)
    hi = (pos + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    hi[-1] = 65536.0  # the value after the largest finite fp16, were the format wider
    mid = (lo + hi) / 2  # exact in float64
    for sign in (1.0, -1.0):
        for nudge in (0.0, 1e-9, -1e-9):
            x = sign * mid * (1.0 + nudge)
            with np.errstate(over="ignore"):
                _same_f16_bits(_d2h(x), x.astype(np.float16))


def test_d2h_specials():
    x = np.array([0.0, -0.0, np.inf, -np.inf, 65504.0, 65519.99, 65520.0, 1e300, -1e300, 5e-324,
                  2.0**-25, 2.0**-25 * (1 + 1e-12), 2.0**-24, 2.0**-14, np.nan])
    with np.errstate(over="ignore"):
        _same_f16_bits(_d2h(x), x.astype(np.float16))


def test_hmul_hadd_match_numpy_half_arithmetic():
    g = rng(3)
    L = oracle.lib()
    a = g.integers(0, 65536, size=40000, dtype=np.uint32).astype(np.uint16)
    b = g.integers(0, 65536, size=40000, dtype=np.uint32).astype(np.uint16)
    af, bf = a.view(np.float16).astype(np.float64), b.view(np.float16).astype(np.float64)
    with np.errstate(all="ignore"):
        ref_mul = (af * bf).astype(np.float16)   # exact product in f64, one rounding
        ref_add = (af + bf).astype(np.float16)   # exact sum in f64, one rounding
    got_mul = np.array([L.adr_o_hmul(int(x), int(y)) for x, y in zip(a, b)], np.uint16)
    got_add = np.array([L.adr_o_hadd(int(x), int(y)) for x, y in zip(a, b)], np.uint16)
    _same_f16_bits(got_mul, ref_mul)
    _same_f16_bits(got_add, ref_add)
