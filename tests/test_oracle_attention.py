"""Pins oracle.attention_f16: its float64 form against torch's own attention routine and closed
forms, and its restatement of the reference's three-call sequence (llama.rs:541-554) against that
float64 form within the fp16 rounding the sequence applies in between."""
import numpy as np
import pytest
import torch

import oracle
from helpers import rng, randn_f16


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("shape", [(2, 40, 50, 64), (1, 77, 77, 64), (3, 65, 33, 128)])
def test_exact_form_matches_torch_sdpa(shape, causal):
    heads, m, n, d = shape
    g = rng(m * 31 + n)
    q, k, v = randn_f16(g, (heads, m, d)), randn_f16(g, (heads, n, d)), randn_f16(g, (heads, n, d))
    scale = float(np.float16(0.125))
    got = oracle.attention_f16(q, k, v, scale, 1.0,
                               oracle.MASK_CAUSAL if causal else oracle.MASK_NONE, exact=True)
    qt, kt, vt = (torch.from_numpy(t).double() for t in (q, k, v))
    # the reference's mask removes x > y by absolute index (matmul.cu:182-184): a boolean
    # mask handed to torch, not its is_causal flag (which aligns differently when m != n)
    keep = torch.arange(n)[None, :] <= torch.arange(m)[:, None] if causal else None
    want = torch.nn.functional.scaled_dot_product_attention(qt, kt, vt, attn_mask=keep,
                                                            scale=scale).numpy()
    assert np.abs(got.astype(np.float64) - want).max() <= 2 ** -11 * np.abs(want).max() + 1e-7


def test_three_call_restatement_against_exact_form_and_temperature():
    g = rng(9)
    heads, m, n, d = 2, 96, 96, 128
    q, k, v = randn_f16(g, (heads, m, d)), randn_f16(g, (heads, n, d)), randn_f16(g, (heads, n, d))
    scale = 1.0 / np.sqrt(d)
    for temp in (1.0, 0.6):
        steps = oracle.attention_f16(q, k, v, scale, temp, oracle.MASK_CAUSAL)
        exact = oracle.attention_f16(q, k, v, scale, temp, oracle.MASK_CAUSAL, exact=True)
        err = np.abs(steps.astype(np.float64) - exact.astype(np.float64)).max()
        assert 0 < err <= 4e-3 * np.abs(exact.astype(np.float64)).max()
    # a dropped temperature would show: the two temperatures give different results
    a = oracle.attention_f16(q, k, v, scale, 1.0, oracle.MASK_NONE, exact=True)
    b = oracle.attention_f16(q, k, v, scale, 0.6, oracle.MASK_NONE, exact=True)
    assert np.abs(a.astype(np.float64) - b.astype(np.float64)).max() > 0.05


def test_closed_forms():
    g = rng(3)
    heads, n, d = 2, 64, 64
    v = randn_f16(g, (heads, n, d))
    k = randn_f16(g, (heads, n, d))
    zero_q = np.zeros((heads, 8, d), np.float16)
    for exact in (False, True):
        # equal scores: the mean of the value rows
        out = oracle.attention_f16(zero_q, k, v, 0.125, 1.0, oracle.MASK_NONE, exact=exact)
        mean = v.astype(np.float64).mean(axis=1, keepdims=True)
        assert np.abs(out.astype(np.float64) - mean).max() <= 2e-3
        # causal: query row y averages value rows 0..y; row 0 is value row 0 exactly
        out = oracle.attention_f16(zero_q, k, v, 0.125, 1.0, oracle.MASK_CAUSAL, exact=exact)
        assert np.array_equal(out[:, 0], v[:, 0])
        cum = np.cumsum(v.astype(np.float64), axis=1)[:, :8] / np.arange(1, 9)[None, :, None]
        assert np.abs(out.astype(np.float64) - cum).max() <= 2e-3
