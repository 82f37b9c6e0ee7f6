"""fp16 skinny matmul (few activation rows, the per-token call of llama.rs:485-591) through
adr_matmul_f16: the streaming dot-product kernel (m <= 8) and the matrix-core kernel whose
wavefronts split K (m = 9..32) against the CPU oracle."""
import numpy as np
import pytest
import torch

import oracle
from helpers import rng, randn_f16, max_rel_err
from gpu_common import to_dev, to_np, raw_matmul, oracle_matmul, plan

pytestmark = pytest.mark.gpu

TOL = 1e-2
PLAN = "gemv_f16_dot2_stream"
PLAN_MFMA = "skinny_f16_mfma16_regstream"


def nt(M, K, N):
    return (1, N, M * N), (1, K, M * K), (K, 1, K * N)


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 9, 16])
@pytest.mark.parametrize("K,N", [(512, 1030), (4096, 259), (4104, 131), (11008, 50), (12288, 44),
                                 # five to sixteen segments of 512: eight wavefronts with one or two each
                                 (2560, 420), (5120, 230), (6664, 90), (8192, 140),
                                 (4096, 1100), (11008, 400)])
def test_matches_oracle_and_is_exact_on_exact_inputs(m, K, N):
    so, sl, sr = nt(m, K, N)
    # one and two rows: dot products; three to eight: dot products only where K is no multiple
    # of 128 (or the matrix is small); more: other kernels
    mfma = K % 128 == 0 and K >= 1024 and N * K >= (1 << 22) and m >= 3
    if mfma:
        assert plan(1, m, K, N, so, sl, sr) == PLAN_MFMA
    elif m <= 8:
        assert plan(1, m, K, N, so, sl, sr) == PLAN
    g = rng(2000 + m * 31 + K + N)
    l, r = randn_f16(g, m * K), randn_f16(g, K * N, K ** -0.5)
    o_t = to_dev(np.full(m * N, 3.0, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), 1, m, K, N, so, sl, sr) == 0
    want = oracle_matmul(np.zeros(m * N, np.float16), l, r, 1, m, K, N, so, sl, sr)
    assert max_rel_err(to_np(o_t), want.astype(np.float64)) <= 2e-3
    # k/64 values in [-1/8, 1/8]: every partial sum is exact in fp32, any order gives the same bits
    l = (g.integers(-8, 9, size=m * K) / 64.0).astype(np.float16)
    r = (g.integers(-8, 9, size=K * N) / 64.0).astype(np.float16)
    o_t = to_dev(np.zeros(m * N, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), 1, m, K, N, so, sl, sr) == 0
    want = (l.reshape(m, K).astype(np.float64) @ r.reshape(N, K).astype(np.float64).T)
    assert np.array_equal(to_np(o_t).view(np.uint16), want.astype(np.float16).reshape(-1).view(np.uint16))


STORES = [oracle.STORE_IDENTITY, oracle.STORE_SCALE, oracle.STORE_ADD, oracle.STORE_BETA_BIAS,
          oracle.STORE_QUICK_GELU_BIAS, oracle.STORE_BETA_GELU_BIAS]


@pytest.mark.parametrize("store", STORES)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
def test_operators_and_mask(store, mask):
    m, K, N = 6, 1032, 520
    so, sl, sr = nt(m, K, N)
    assert plan(1, m, K, N, so, sl, sr, store=store, mask=mask) == PLAN
    g = rng(2100 + store * 5 + mask)
    l, r = randn_f16(g, m * K), randn_f16(g, K * N, K ** -0.5)
    prev, bias = randn_f16(g, m * N), randn_f16(g, N)
    scale = 0.25 if store == oracle.STORE_SCALE else 1.0
    o_t = to_dev(prev)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), 1, m, K, N, so, sl, sr,
                      bias_t=to_dev(bias), beta=0.75, scale=scale, store=store, mask=mask) == 0
    want = oracle_matmul(prev, l, r, 1, m, K, N, so, sl, sr, bias=bias, beta=0.75, scale=scale,
                         store=store, mask=mask)
    got = to_np(o_t)
    masked = np.isneginf(want.astype(np.float32))
    assert np.array_equal(np.isneginf(got.astype(np.float32)), masked)
    assert mask == oracle.MASK_NONE or masked.any()
    err = np.abs(got[~masked].astype(np.float64) - want[~masked].astype(np.float64))
    ref = np.abs(want[~masked].astype(np.float64))
    assert np.max(err / np.maximum(ref, np.sqrt(np.mean(ref ** 2)))) <= TOL


def test_padded_rows_and_transposed_output():
    """Row pitches larger than the row (views into wider tensors) and an output written
    column-major; nothing outside the views may change."""
    m, K, N = 4, 2048, 300
    ldl, ldr = K + 64, K + 8
    g = rng(2200)
    l, r = randn_f16(g, m * ldl), randn_f16(g, N * ldr, K ** -0.5)
    so, sl, sr = (m + 2, 1, 0), (1, ldl, 0), (ldr, 1, 0)   # out[y, x] at x * (m + 2) + y
    assert plan(1, m, K, N, so, sl, sr) == PLAN
    out0 = np.full(N * (m + 2), 5.0, np.float16)
    o_t = to_dev(out0)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), 1, m, K, N, so, sl, sr) == 0
    want = oracle_matmul(out0, l, r, 1, m, K, N, so, sl, sr)
    got = to_np(o_t)
    assert max_rel_err(got.reshape(N, m + 2)[:, :m], want.reshape(N, m + 2)[:, :m].astype(np.float64)) <= 2e-3
    assert np.all(got.reshape(N, m + 2)[:, m:] == 5.0)


def test_nt_entry_point_with_beta():
    """adr_matmul_nt_f16 (out = acc + beta * out, the accumulator not narrowed first) takes the
    same kernel for a few rows."""
    from adrastea_amd import _ffi
    m, K, N = 3, 4096, 256
    g = rng(2300)
    l, r, prev = randn_f16(g, m * K), randn_f16(g, N * K, K ** -0.5), randn_f16(g, m * N)
    o_t, l_t, r_t = to_dev(prev), to_dev(l), to_dev(r)
    stream = torch.cuda.current_stream().cuda_stream
    assert _ffi.lib().adr_matmul_nt_f16(stream, o_t.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), m, K,
                                        N, 0.5) == 0
    want = (l.reshape(m, K).astype(np.float64) @ r.reshape(N, K).astype(np.float64).T
            + 0.5 * prev.reshape(m, N).astype(np.float64))
    assert max_rel_err(to_np(o_t).reshape(m, N), want) <= 2e-3


@pytest.mark.parametrize("m,K,N,tiled", [(32, 1280, 51865, True), (32, 2048, 12288, True), (64, 1536, 8192, True),
                                         (17, 1024, 16384, True), (32, 1024, 4096, False),
                                         (16, 1280, 51864, False), (32, 4096, 12288, False)])
def test_short_k_from_17_rows_on_a_wide_matrix_takes_the_tiled_kernels(m, K, N, tiled):
    """Ten macro steps split badly over the kernel's eight wavefronts: from 17 rows on, with
    K < 4096 and more than one workgroup per compute unit, the product is a tiled one (the
    Whisper decoder's logits for a 32-token prefix: 43 us here, 30 there)."""
    so, sl, sr = nt(m, K, N)
    name = plan(1, m, K, N, so, sl, sr)
    assert name.startswith("gemm_nt_mfma") if tiled else name == PLAN_MFMA


@pytest.mark.parametrize("m,K,N", [(9, 1024, 4100), (16, 4096, 1030), (13, 11008, 400), (17, 8192, 520),
                                   (32, 11008, 390), (25, 12288, 350), (20, 1024, 4096),
                                   (30, 1152, 4096),
                                   # one, two and three groups of 16 weight rows per workgroup
                                   (9, 2048, 4100), (16, 4096, 6200), (12, 5120, 10300),
                                   (11, 8192, 1000), (16, 4096, 12288),
                                   # macro-step counts that do not divide by the eight wavefronts
                                   # (K 11008: 86 steps), fewer steps than wavefronts + 1
                                   (16, 11008, 4096), (10, 2176, 6200), (14, 4992, 10300), (9, 10368, 800),
                                   (16, 13824, 5120), (12, 6656, 700),
                                   # 17 to 32 rows: two blocks of activations
                                   (17, 4096, 6200), (32, 2048, 4096), (25, 3072, 4000), (32, 4096, 12288),
                                   (20, 3968, 4096), (32, 11008, 4096), (19, 8192, 6200), (27, 5120, 10300),
                                   # 33 to 64 rows: three and four blocks (four: at most two row groups)
                                   (33, 4096, 4100), (48, 4096, 6200), (49, 3968, 4000), (64, 11008, 4096),
                                   (40, 10368, 1000), (64, 4096, 8192), (48, 5120, 5000), (64, 13824, 1000),
                                   (48, 8192, 12288), (33, 2048, 4096),
                                   # one to four rows where K is beyond the dot-product kernel's reach
                                   (2, 13824, 1000), (4, 16384, 600), (1, 12416, 520),
                                   # three and four rows on narrow matrices, five to eight rows
                                   (3, 4096, 4096), (4, 2048, 4000), (4, 3072, 3072),
                                   (5, 4096, 4100), (8, 11008, 4096), (7, 1152, 4000)])
def test_matrix_core_kernel_for_five_to_sixty_four_rows(m, K, N):
    so, sl, sr = nt(m, K, N)
    assert plan(1, m, K, N, so, sl, sr) == PLAN_MFMA
    g = rng(2400 + m + K + N)
    l = (g.integers(-8, 9, size=m * K) / 64.0).astype(np.float16)
    r = (g.integers(-8, 9, size=K * N) / 64.0).astype(np.float16)
    o_t = to_dev(np.full(m * N, 2.0, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), 1, m, K, N, so, sl, sr) == 0
    want = (l.reshape(m, K).astype(np.float64) @ r.reshape(N, K).astype(np.float64).T)
    assert np.array_equal(to_np(o_t).view(np.uint16), want.astype(np.float16).reshape(-1).view(np.uint16))
    # random inputs, an operator that reads the previous output and the bias, the causal mask
    l, r = randn_f16(g, m * K), randn_f16(g, K * N, K ** -0.5)
    prev, bias = randn_f16(g, m * N), randn_f16(g, N)
    o_t = to_dev(prev)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), 1, m, K, N, so, sl, sr,
                      bias_t=to_dev(bias), beta=0.5, store=oracle.STORE_BETA_BIAS,
                      mask=oracle.MASK_CAUSAL) == 0
    want = oracle_matmul(prev, l, r, 1, m, K, N, so, sl, sr, bias=bias, beta=0.5,
                         store=oracle.STORE_BETA_BIAS, mask=oracle.MASK_CAUSAL)
    got = to_np(o_t)
    masked = np.isneginf(want.astype(np.float32))
    assert masked.any() and np.array_equal(np.isneginf(got.astype(np.float32)), masked)
    err = np.abs(got[~masked].astype(np.float64) - want[~masked].astype(np.float64))
    ref = np.abs(want[~masked].astype(np.float64))
    assert np.max(err / np.maximum(ref, np.sqrt(np.mean(ref ** 2)))) <= TOL


def test_more_rows_or_short_k_stay_on_the_tiled_kernels():
    for m, K, N in [(65, 4096, 4096), (65, 11008, 4096), (33, 2000, 8192), (12, 960, 8192),
                    (64, 4096, 12288)]:
        so, sl, sr = nt(m, K, N)
        assert plan(1, m, K, N, so, sl, sr).startswith("gemm_nt_mfma")
