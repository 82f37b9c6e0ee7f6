"""Pins the oracle's u8 absmax format functions (adrastea_kernels/cpp/quantize.cu:3-56,
matmul_nt_fp16u8.cu:4-24, matmul_nt_wmma_16x128x256_fp16u8.cu:5-7,43-83).  CPU only.

The reference holds no fixture for these; the pins are: an exhaustive dequant table against an
independent float64 evaluation, closed-form quantise rows, the round-trip bound, and the identity
"u8 matmul == fp16 matmul on the dequantised weights"."""
import hashlib
import os

import numpy as np

import oracle
from helpers import rng, randn_f16, max_rel_err

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _expected_table():
    q = np.arange(256, dtype=np.float64)[:, None] - 127.5
    s = np.arange(65536, dtype=np.uint16).view(np.float16).astype(np.float64)[None, :]
    with np.errstate(all="ignore"):
        return (q * s).astype(np.float16)  # exact f64 product, one rounding


def test_dequant_table_exhaustive():
    table = oracle.dequant_table()
    ref = _expected_table()
    nan = np.isnan(ref)
    assert np.array_equal(np.isnan(table.view(np.float16)), nan)
    assert np.array_equal(table[~nan], ref.view(np.uint16)[~nan])
    # inf scales give signed infinities, never NaN (q - 127.5 is never zero)
    assert table[0, 0x7C00] == 0xFC00 and table[255, 0x7C00] == 0x7C00
    # subnormal scale: (255 - 127.5) * 2^-24 = 127.5 * 2^-24 -> 128 * 2^-24 (ties to even)
    assert table[255, 0x0001] == 128 and table[0, 0x0001] == 0x8000 | 128


def test_dequant_table_hash_fixture():
    """The committed digest lets the GPU parity test compare a 16.7 M-entry device result
    without shipping the table; NaN patterns are canonicalised first."""
    table = oracle.dequant_table().copy()
    table[np.isnan(table.view(np.float16))] = 0x7E00
    digest = hashlib.sha256(table.tobytes()).hexdigest()
    with open(os.path.join(GOLDEN, "dequant_table.sha256")) as f:
        assert f.read().split()[0] == digest


def test_dequantize_indexing_uses_the_rows_own_scale_block():
    g = rng(30)
    rows, cols, bs = 5, 96, 32
    q = g.integers(0, 256, size=(rows, cols), dtype=np.uint16).astype(np.uint8)
    s = g.uniform(0.001, 0.02, size=(rows, cols // bs)).astype(np.float16)
    got = oracle.dequantize_absmax_u8(q, s, bs)
    ref = ((q.astype(np.float64) - 127.5) * np.repeat(s.astype(np.float64), bs, axis=1))
    assert np.array_equal(got.view(np.uint16), ref.astype(np.float16).view(np.uint16))


def test_quantize_closed_forms():
    bs = 32
    x = np.zeros((4, 64), np.float16)
    x[0, :32] = 3.0                     # all equal: every element is +absmax -> 255
    x[0, 32:] = -3.0                    # -> 0
    x[1, 5] = 10.0                      # single spike; zeros sit at round(127.5) = 128
    x[2, :32] = np.linspace(-1, 1, 32).astype(np.float16)
    x[3, 32:] = np.float16(6.1e-5)      # smallest normal: subnormal scale
    q, s = oracle.quantize_absmax_u8(x, bs)
    assert np.all(q[0, :32] == 255) and np.all(q[0, 32:] == 0)
    assert s[0, 0] == np.float16(np.float32(3.0) / np.float32(127.5))
    assert q[1, 5] == 255 and np.all(np.delete(q[1, :32], 5) == 128)
    # closed form on a ramp: q = round_half_away(127.5 + x / s)
    sc = np.float64(s[2, 0])
    v = 127.5 + x[2, :32].astype(np.float64) / sc
    v32 = (np.float32(127.5) + x[2, :32].astype(np.float32) / np.float32(s[2, 0])).astype(np.float64)
    ref = np.floor(np.abs(v32) + 0.5) * np.sign(v32)
    assert np.array_equal(q[2, :32].astype(np.float64), ref)
    assert np.max(np.abs(v - v32)) < 1e-4
    assert q[2, 0] == 0 and q[2, 31] == 255
    assert s[3, 1] == np.float16(np.float32(np.float16(6.1e-5)) / np.float32(127.5))


def test_quantize_dequantize_round_trip_bound():
    g = rng(31)
    bs = 32
    x = randn_f16(g, (16, 256), 0.02)
    q, s = oracle.quantize_absmax_u8(x, bs)
    dq = oracle.dequantize_absmax_u8(q, s, bs).astype(np.float64)
    sc = np.repeat(s.astype(np.float64), bs, axis=1)
    err = np.abs(dq - x.astype(np.float64))
    # half a quantisation step, plus the fp16 roundings of the scale and of the result
    assert np.all(err <= sc * 0.5 + np.abs(x.astype(np.float64)) * 2.0 ** -10 + 1e-7)


def test_u8_matmul_equals_fp16_matmul_on_dequantised_weights():
    g = rng(32)
    M, K, N, bs = 5, 128, 24, 32
    a = randn_f16(g, (M, K))
    q = g.integers(0, 256, size=(N, K), dtype=np.uint16).astype(np.uint8)
    s = g.uniform(0.001, 0.02, size=(N, K // bs)).astype(np.float16)
    prev = randn_f16(g, (M, N))
    for beta in (0.0, 0.5):
        out = prev.copy()
        oracle.matmul_nt_fp16u8(out, a, q, s, bs, beta=beta)
        w = oracle.dequantize_absmax_u8(q, s, bs)
        out2 = prev.copy()
        oracle.matmul_nt_f16(out2, a, w, beta=beta)
        assert np.array_equal(out.view(np.uint16), out2.view(np.uint16))
        # the general matmul on the NT view agrees too (beta = 0 only: it has no plain beta op)
        if beta == 0.0:
            out3 = np.zeros(M * N, np.float16)
            oracle.matmul_f16(out3, a, w, 1, M, K, N, (1, N, 0), (1, K, 0), (K, 1, 0),
                              mode=oracle.EXACT)
            assert np.array_equal(out3.reshape(M, N).view(np.uint16), out.view(np.uint16))
        ref = a.astype(np.float64) @ w.astype(np.float64).T + beta * prev.astype(np.float64)
        assert max_rel_err(out, ref) <= 2.0 ** -10
        # the naive kernel's double-precision product differs only by the weight rounding
        out4 = prev.copy()
        oracle.matmul_nt_fp16u8(out4, a, q, s, bs, beta=beta, naive=True)
        assert max_rel_err(out4, ref) <= 1e-2
        wd = (q.astype(np.float64) - 127.5) * np.repeat(s.astype(np.float64), bs, axis=1)
        ref_naive = a.astype(np.float64) @ wd.T + beta * prev.astype(np.float64)
        assert max_rel_err(out4, ref_naive) <= 2.0 ** -9
