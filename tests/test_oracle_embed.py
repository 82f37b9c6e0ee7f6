"""Pins oracle.embed_uint8 (embed_uint8.cu:3-19): it is the gather of the already pinned
dequantisation (exhaustive table, tests/test_oracle_quant.py), so the check is that identity plus
the index arithmetic on constructed tables."""
import numpy as np

import oracle
from helpers import rng


def test_embed_is_a_gather_of_the_dequantised_table():
    g = rng(5)
    vocab, n_dim, bs = 50, 96, 32
    table = g.integers(0, 256, size=(vocab, n_dim)).astype(np.uint8)
    scales = np.exp2(g.integers(-9, -3, size=(vocab, n_dim // bs))).astype(np.float16)
    ids = np.array([0, 49, 7, 7, 13, 1], np.int16)
    got = oracle.embed_uint8(ids, table, scales, bs)
    full = oracle.dequantize_absmax_u8(table, scales, bs)
    assert np.array_equal(got.view(np.uint16), full[ids].view(np.uint16))
    # closed form on one entry: (q - 127.5) * s, exact here (power-of-two scale)
    t, i = 2, 70
    want = (float(table[ids[t], i]) - 127.5) * float(scales[ids[t], i // bs])
    assert float(got[t, i]) == want


def test_embed_block_index_uses_the_row_of_the_id():
    # a table whose scale differs per (row, block): a wrong row or block index shows
    vocab, n_dim, bs = 4, 16, 8
    table = np.full((vocab, n_dim), 255, np.uint8)            # q - 127.5 = 127.5
    scales = np.array([[1, 2], [4, 8], [16, 32], [64, 128]], np.float16) / 128
    got = oracle.embed_uint8(np.array([3, 1], np.int16), table, scales, bs).astype(np.float64)
    assert np.all(got[0, :8] == 127.5 * 64 / 128) and np.all(got[0, 8:] == 127.5)
    assert np.all(got[1, :8] == 127.5 * 4 / 128) and np.all(got[1, 8:] == 127.5 * 8 / 128)
