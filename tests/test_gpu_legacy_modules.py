"""GPU parity of the legacy-symbol code objects (adrastea_amd/lib/legacy/*.co): launched through
the HIP module API exactly as the reference's host code launches its own kernels -- same symbol
names, same argument tuple, same grid and block shapes (adrastea_models/src/kernels.rs:783-792,
849-863, 968-993) -- and compared with the CPU oracle."""
import itertools
import os

import numpy as np
import pytest
import torch

import oracle
import refgpu
from adrastea_amd import build
from helpers import rng, randn_f16, max_rel_err, largest_address
from gpu_common import to_dev, to_np, oracle_matmul, nan_canon

pytestmark = pytest.mark.gpu

TOL = 1e-2  # max relative error against the float64 product, as for the library's MFMA path


@pytest.fixture(scope="module")
def legacy():
    for name in build.LEGACY_MODULES:
        assert os.path.exists(os.path.join(build.LEGACY_DIR, name)), "run the build first"
    return refgpu.RefKernels(build.LEGACY_DIR)


def nt(M, K, N):
    return (1, N, M * N), (1, K, M * K), (K, 1, K * N)


CASES = [
    # name, B, M, K, N, strides(out, lhs, rhs) builder
    ("nt_weights_tails", 1, 77, 768, 100, nt),
    ("nt_k_tail_of_32", 2, 33, 72, 50, nt),
    ("nt_k_not_8", 1, 20, 75, 40, nt),  # per-output path
    ("row_major_rhs", 2, 40, 64, 48, lambda M, K, N: ((1, N, M * N), (1, K, M * K), (1, N, K * N))),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
@pytest.mark.parametrize("kernel", ["matmul_f16", "matmul_f16_fast"])
def test_matmul_symbols_match_oracle(legacy, case, kernel):
    _, B, M, K, N, mk = case
    so, sl, sr = mk(M, K, N)
    g = rng(900 + M + K)
    l, r = randn_f16(g, B * M * K), randn_f16(g, B * K * N, K ** -0.5)
    o_t, l_t, r_t = to_dev(np.full(B * M * N, 7.0, np.float16)), to_dev(l), to_dev(r)
    getattr(legacy, kernel)(o_t.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, so, sl, sr)
    torch.cuda.synchronize()
    got = to_np(o_t)
    want = oracle_matmul(np.zeros(B * M * N, np.float16), l, r, B, M, K, N, so, sl, sr,
                         mode=oracle.FAITHFUL)
    if kernel == "matmul_f16":  # the reference's arithmetic step for step
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    else:
        exact = oracle_matmul(np.zeros(B * M * N, np.float16), l, r, B, M, K, N, so, sl, sr)
        assert max_rel_err(got, exact.astype(np.float64)) <= TOL


STORES = [oracle.STORE_IDENTITY, oracle.STORE_SCALE, oracle.STORE_ADD, oracle.STORE_BETA_BIAS,
          oracle.STORE_QUICK_GELU_BIAS, oracle.STORE_BETA_GELU_BIAS]


@pytest.mark.parametrize("store", STORES)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
@pytest.mark.parametrize("load", [oracle.LOAD_IDENTITY, oracle.LOAD_SCALE])
def test_fast_symbol_operators(legacy, store, mask, load):
    B, M, K, N = 2, 45, 96, 70
    so, sl, sr = nt(M, K, N)
    g = rng(1000 + store * 7 + mask * 3 + load)
    l, r = randn_f16(g, B * M * K), randn_f16(g, B * K * N, K ** -0.5)
    prev, bias = randn_f16(g, B * M * N), randn_f16(g, N)
    scale = 0.5 if (load == oracle.LOAD_SCALE or store == oracle.STORE_SCALE) else 1.0
    o_t, l_t, r_t, b_t = to_dev(prev), to_dev(l), to_dev(r), to_dev(bias)
    legacy.matmul_f16_fast(o_t.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, so, sl, sr,
                           bias_ptr=b_t.data_ptr(), beta=0.75, scale=scale, store=store, load=load,
                           mask=mask)
    torch.cuda.synchronize()
    want = oracle_matmul(prev, l, r, B, M, K, N, so, sl, sr, bias=bias, beta=0.75, scale=scale,
                         store=store, load=load, mask=mask)
    got = to_np(o_t)
    masked = np.isneginf(want.astype(np.float32))
    assert np.array_equal(np.isneginf(got.astype(np.float32)), masked)
    err = np.abs(got[~masked].astype(np.float64) - want[~masked].astype(np.float64))
    ref = np.abs(want[~masked].astype(np.float64))
    assert np.max(err / np.maximum(ref, np.sqrt(np.mean(ref ** 2)))) <= TOL


def test_fast_symbol_exact_on_dyadic_inputs_and_attention_views(legacy):
    """QK^T on the interleaved head views of llama.rs:534-546: exact sums, bit for bit."""
    H, S, D = 3, 50, 64
    ld = H * D
    g = rng(1100)
    q = (g.integers(-8, 9, size=S * ld) / 64.0).astype(np.float16)
    k = (g.integers(-8, 9, size=S * ld) / 64.0).astype(np.float16)
    so, sl, sr = (1, S, S * S), (1, ld, D), (ld, 1, D)
    o_t, q_t, k_t = to_dev(np.zeros(H * S * S, np.float16)), to_dev(q), to_dev(k)
    legacy.matmul_f16_fast(o_t.data_ptr(), q_t.data_ptr(), k_t.data_ptr(), H, S, D, S, so, sl, sr,
                           scale=0.125, store=oracle.STORE_SCALE, mask=oracle.MASK_CAUSAL)
    torch.cuda.synchronize()
    want = oracle_matmul(np.zeros(H * S * S, np.float16), q, k, H, S, D, S, so, sl, sr, scale=0.125,
                         store=oracle.STORE_SCALE, mask=oracle.MASK_CAUSAL)
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))


def test_raw_symbol(legacy):
    B, M, K, N = 1, 19, 40, 23
    so, sl, sr = nt(M, K, N)
    g = rng(1200)
    l, r = randn_f16(g, B * M * K), randn_f16(g, B * K * N, K ** -0.5)
    o_t, l_t, r_t = to_dev(np.zeros(B * M * N, np.float16)), to_dev(l), to_dev(r)
    legacy.matmul_f16_raw(o_t.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, so, sl, sr)
    torch.cuda.synchronize()
    want = oracle_matmul(np.zeros(B * M * N, np.float16), l, r, B, M, K, N, so, sl, sr,
                         mode=oracle.FAITHFUL)
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_error_stats_symbols(legacy, dtype):
    n = 1 << 20
    gen = torch.Generator(device="cuda").manual_seed(5)
    a = torch.randn(n + 77, generator=gen, device="cuda").to(dtype)
    b = (a.float() + 0.01 * torch.randn(n + 77, generator=gen, device="cuda")).to(dtype)
    out = torch.zeros(3, device="cuda")
    legacy.error_stats(out, a, b)
    torch.cuda.synchronize()
    want = oracle.error_stats(a.cpu().numpy(), b.cpu().numpy())
    got = out.cpu().numpy()
    assert got[1] == want[1]
    assert abs(got[0] - want[0]) <= 1e-5 * want[0] and abs(got[2] - want[2]) <= 1e-5 * want[2]
