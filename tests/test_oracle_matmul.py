"""Pins oracle.matmul_f16 (the restatement of adrastea_kernels/cpp/matmul.cu:186-222 and the
operator structs :26-184) by what the mathematics fixes -- the reference has no matmul test or
golden vector.  CPU only.

Each check is chosen so that a plausible mistake fails it: swapped strides or operands
(stride brute force, non-square shapes), a dropped rounding (epilogue closed forms on inputs
whose accumulator is exactly known), a wrong mask orientation (causal on a non-square output),
reading the output after writing it (in-place Add), mis-broadcast batches (stride_z = 0).
"""
import itertools

import numpy as np
import pytest

import oracle
from helpers import rng, view, largest_address, randn_f16, ulp_diff_f16, max_rel_err


def small_ints(g, shape, lim=4):
    return g.integers(-lim, lim + 1, size=shape).astype(np.float16)


def dyadic(g, shape):
    """fp16 values k/64 in [-4, 4]: products are multiples of 2^-12 and every partial sum of
    a few hundred of them is exact in float32 and float64, whatever the summation order."""
    return (g.integers(-256, 257, size=shape) / 64.0).astype(np.float16)


def run(out, lhs, rhs, B, M, K, N, so, sl, sr, **kw):
    return oracle.matmul_f16(out, lhs, rhs, B, M, K, N, so, sl, sr, **kw)


def contiguous(B, M, K, N):
    return (1, N, M * N), (1, K, M * K), (1, N, K * N)


@pytest.mark.parametrize("mode", [oracle.FAITHFUL, oracle.EXACT])
def test_integer_inputs_are_bit_exact(mode):
    g = rng(10)
    B, M, K, N = 3, 17, 40, 23  # K * 4 * 4 = 640 < 2048: all sums are exact fp16 integers
    a, b = small_ints(g, (B, M, K)), small_ints(g, (B, K, N))
    out = np.zeros(B * M * N, np.float16)
    run(out, a, b, B, M, K, N, *contiguous(B, M, K, N), mode=mode)
    ref = np.einsum("bmk,bkn->bmn", a.astype(np.int64), b.astype(np.int64))
    assert np.array_equal(out.reshape(B, M, N).astype(np.int64), ref)


def test_identity_and_permutation_operands_copy_bits():
    g = rng(11)
    M, K = 9, 12
    a = g.integers(0, 0x7C00, size=(M, K), dtype=np.uint32).astype(np.uint16).view(np.float16)
    perm = g.permutation(K)
    p = np.zeros((K, K), np.float16)
    p[perm, np.arange(K)] = 1.0  # out[:, j] = a[:, perm[j]]
    out = np.zeros(M * K, np.float16)
    run(out, a, p, 1, M, K, K, (1, K, 0), (1, K, 0), (1, K, 0))
    assert np.array_equal(out.reshape(M, K).view(np.uint16), a[:, perm].view(np.uint16))


def test_exact_mode_matches_float64_on_dyadic_inputs():
    g = rng(12)
    B, M, K, N = 2, 13, 96, 11
    a, b = dyadic(g, (B, M, K)), dyadic(g, (B, K, N))
    for mode in (oracle.FAITHFUL, oracle.EXACT):
        out = np.zeros(B * M * N, np.float16)
        run(out, a, b, B, M, K, N, *contiguous(B, M, K, N), mode=mode)
        ref = np.einsum("bmk,bkn->bmn", a.astype(np.float64), b.astype(np.float64))
        if mode == oracle.EXACT:
            assert np.array_equal(out.reshape(B, M, N).view(np.uint16),
                                  ref.astype(np.float32).astype(np.float16).view(np.uint16))
        else:
            # fp16-rounded products: |product| <= 16 loses at most half an fp16 step at 16
            # (2^-7) each; the fp32 running sum stays exact; then one final rounding
            err = np.abs(out.reshape(B, M, N).astype(np.float64) - ref)
            assert np.all(err <= K * 2.0 ** -7 + np.abs(ref) * 2.0 ** -11)
            assert np.any(err > 0)  # and the product rounding is really there


def test_faithful_mode_against_numpy_half_arithmetic():
    """Independent evaluation with numpy's own float16 multiply (one rounding per product)
    and a sequential float32 sum, as matmul.cu:214-218 does."""
    g = rng(13)
    M, K, N = 5, 37, 6
    a, b = randn_f16(g, (M, K)), randn_f16(g, (K, N), 0.3)
    out = np.zeros(M * N, np.float16)
    run(out, a, b, 1, M, K, N, (1, N, 0), (1, K, 0), (1, N, 0), mode=oracle.FAITHFUL)
    ref = np.zeros((M, N), np.float16)
    for y in range(M):
        for x in range(N):
            s = np.float32(0)
            for i in range(K):
                s = np.float32(s + np.float32(np.float16(a[y, i] * b[i, x])))
            ref[y, x] = np.float16(s)
    assert np.array_equal(out.reshape(M, N).view(np.uint16), ref.view(np.uint16))


def test_random_matches_float64_within_tolerance():
    g = rng(14)
    M, K, N = 33, 300, 29
    a, b = randn_f16(g, (M, K)), randn_f16(g, (K, N), K ** -0.5)
    ref = a.astype(np.float64) @ b.astype(np.float64)
    # the north-star tolerance (max relative error <= 1e-2 against an fp32/fp64 GEMM) must hold
    # for the reference-faithful arithmetic too; the exact mode is only final-rounding away
    for mode, tol in ((oracle.FAITHFUL, 1e-2), (oracle.EXACT, 2.0 ** -10)):
        out = np.zeros(M * N, np.float16)
        run(out, a, b, 1, M, K, N, (1, N, 0), (1, K, 0), (1, N, 0), mode=mode)
        assert max_rel_err(out.reshape(M, N), ref) <= tol


def test_all_stride_permutations_brute_force():
    """Every assignment of (z, y, x) to memory order, for all three tensors, with padding."""
    g = rng(15)
    B, M, K, N = 2, 3, 5, 4
    perms = list(itertools.permutations(range(3)))

    def layout(shape, perm, pad):
        # memory order perm[0] slowest ... perm[2] fastest, innermost stride `pad`
        strides = [0, 0, 0]
        s = pad
        for d in reversed(perm):
            strides[d] = s
            s *= shape[d] + 1  # +1: gaps between rows, catches off-by-one stride use
        return strides

    for po, pl, pr in itertools.product(perms, perms, perms):
        so3, sl3, sr3 = layout((B, M, N), po, 1), layout((B, M, K), pl, 2), layout((B, K, N), pr, 1)
        lbuf = dyadic(g, largest_address((B, M, K), sl3) + 1 + 3)
        rbuf = dyadic(g, largest_address((B, K, N), sr3) + 1 + 2)
        obuf = np.full(largest_address((B, M, N), so3) + 1 + 1, 7.0, np.float16)
        before = obuf.copy()
        # (x, y, z) triples; offsets exercise non-zero base pointers
        run(obuf, lbuf, rbuf, B, M, K, N, (so3[2], so3[1], so3[0]), (sl3[2], sl3[1], sl3[0]),
            (sr3[2], sr3[1], sr3[0]), mode=oracle.EXACT, offsets=(1, 3, 2))
        lv = view(lbuf, 3, (B, M, K), sl3).astype(np.float64)
        rv = view(rbuf, 2, (B, K, N), sr3).astype(np.float64)
        ref = np.einsum("bmk,bkn->bmn", lv, rv).astype(np.float32).astype(np.float16)
        got = view(obuf, 1, (B, M, N), so3)
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), (po, pl, pr)
        # nothing outside the output view is written
        touched = np.zeros(obuf.size, bool)
        idx = (1 + np.arange(B)[:, None, None] * so3[0] + np.arange(M)[None, :, None] * so3[1] +
               np.arange(N)[None, None, :] * so3[2])
        touched[idx.reshape(-1)] = True
        assert np.array_equal(obuf[~touched], before[~touched])


def test_weight_nt_and_attention_views():
    """The three canonical layouts of the callers: W[N,K].permute([1,0]) (llama.rs:503-508),
    and the QK^T / PV head views of llama.rs:534-554 (scaled down: S=6, heads=3, hd=4)."""
    g = rng(16)
    S, H, D = 6, 3, 4
    HD = H * D
    x, w = dyadic(g, (S, HD)), dyadic(g, (HD, HD))
    out = np.zeros(S * HD, np.float16)
    run(out, x, w, 1, S, HD, HD, (1, HD, 0), (1, HD, 0), (HD, 1, 0), mode=oracle.EXACT)
    ref = (x.astype(np.float64) @ w.astype(np.float64).T)
    assert np.array_equal(out.reshape(S, HD), ref.astype(np.float32).astype(np.float16))
    q, k, v = dyadic(g, (S, HD)), dyadic(g, (S, HD)), dyadic(g, (S, HD))
    qk = np.zeros(H * S * S, np.float16)
    # q_view [H,S,D]: (x1, y HD, z D); k_view [H,D,S]: (x HD, y 1, z D)
    run(qk, q, k, H, S, D, S, (1, S, S * S), (1, HD, D), (HD, 1, D), mode=oracle.EXACT)
    q3, k3, v3 = (t.reshape(S, H, D).astype(np.float64) for t in (q, k, v))
    ref = np.einsum("shd,thd->hst", q3, k3)
    assert np.array_equal(qk.reshape(H, S, S), ref.astype(np.float32).astype(np.float16))
    p = dyadic(g, (H, S, S))
    o = np.zeros(S * HD, np.float16)
    # PV: L contiguous [H,S,S]; v_view [H,S,D]: (x1, y HD, z D); out view the same
    run(o, p, v, H, S, S, D, (1, HD, D), (1, S, S * S), (1, HD, D), mode=oracle.EXACT)
    ref = np.einsum("hst,thd->shd", p.astype(np.float64), v3)
    assert np.array_equal(o.reshape(S, H, D), ref.astype(np.float32).astype(np.float16))


def test_batch_broadcast_stride_zero():
    g = rng(17)
    B, M, K, N = 4, 5, 8, 6
    a, b = dyadic(g, (B, M, K)), dyadic(g, (K, N))
    out0 = np.zeros(B * M * N, np.float16)
    run(out0, a, b, B, M, K, N, (1, N, M * N), (1, K, M * K), (1, N, 0))
    out1 = np.zeros(B * M * N, np.float16)
    run(out1, a, np.broadcast_to(b, (B, K, N)).copy(), B, M, K, N, *contiguous(B, M, K, N))
    assert np.array_equal(out0, out1)


def test_transposed_output_strides():
    g = rng(18)
    M, K, N = 7, 9, 5
    a, b = dyadic(g, (M, K)), dyadic(g, (K, N))
    o1 = np.zeros(M * N, np.float16)
    run(o1, a, b, 1, M, K, N, (1, N, 0), (1, K, 0), (1, N, 0))
    o2 = np.zeros(M * N, np.float16)
    run(o2, a, b, 1, M, K, N, (M, 1, 0), (1, K, 0), (1, N, 0))
    assert np.array_equal(o1.reshape(M, N), o2.reshape(N, M).T)


# ---------------------------------------------------------------- epilogues

def _exact_case(seed, M=6, K=16, N=10):
    g = rng(seed)
    a, b = small_ints(g, (M, K), 3), small_ints(g, (K, N), 3)
    acc = a.astype(np.float64) @ b.astype(np.float64)  # |acc| <= 144: exact in fp16
    return g, a, b, acc


def _epilogue(a, b, M, K, N, prev, **kw):
    out = prev.astype(np.float16).reshape(-1).copy()
    run(out, a, b, 1, M, K, N, (1, N, 0), (1, K, 0), (1, N, 0), **kw)
    return out.reshape(M, N)


def test_store_scale_is_an_fp16_multiply():
    g, a, b, acc = _exact_case(20)
    M, N = acc.shape
    K = a.shape[1]
    for scale in (0.5, 0.125, 1.0 / np.sqrt(128.0), 0.3):
        got = _epilogue(a, b, M, K, N, np.zeros((M, N)), store=oracle.STORE_SCALE, scale=scale)
        s16 = np.float64(np.float16(np.float32(scale)))
        ref = (acc * s16).astype(np.float16)  # product exact in f64 -> one rounding
        assert np.array_equal(got.view(np.uint16), ref.view(np.uint16)), scale
    # 1/sqrt(128) narrows to the fp16 value 0.08837890625 (the QK^T scale of LLaMA-7B)
    assert float(np.float16(np.float32(1.0 / np.sqrt(128.0)))) == 0.08837890625


def test_store_add_reads_previous_output_in_fp16():
    g, a, b, acc = _exact_case(21)
    M, N = acc.shape
    prev = randn_f16(g, (M, N), 30.0)
    got = _epilogue(a, b, M, a.shape[1], N, prev, store=oracle.STORE_ADD)
    ref = (acc + prev.astype(np.float64)).astype(np.float16)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("beta", [0.0, 1.0, -0.5, 0.3])
def test_store_beta_bias(beta):
    g, a, b, acc = _exact_case(22)
    M, N = acc.shape
    prev, bias = randn_f16(g, (M, N), 5.0), randn_f16(g, (N,), 2.0)
    got = _epilogue(a, b, M, a.shape[1], N, prev, store=oracle.STORE_BETA_BIAS, beta=beta,
                    bias=bias)
    ref64 = acc + bias.astype(np.float64)[None, :] + np.float64(np.float32(beta)) * prev.astype(np.float64)
    # fp32 intermediate roundings can move a near-tie by one fp16 step, never more
    assert np.max(ulp_diff_f16(got, ref64.astype(np.float16))) <= 1
    if beta in (0.0, 1.0):  # every fp32 step is exact for these: demand bit equality
        assert np.array_equal(got.view(np.uint16), ref64.astype(np.float16).view(np.uint16))


def test_store_quick_gelu_bias():
    g, a, b, acc = _exact_case(23)
    M, N = acc.shape
    acc_small = acc / 16.0  # spread values over the interesting range of the activation
    a = (a.astype(np.float64) / 16.0).astype(np.float16)
    bias = randn_f16(g, (N,), 1.0)
    got = _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), store=oracle.STORE_QUICK_GELU_BIAS,
                    bias=bias)
    v = acc_small + bias.astype(np.float64)[None, :]
    ref = v / (1.0 + np.exp(-np.float64(np.float32(1.702)) * v))
    assert np.max(ulp_diff_f16(got, ref.astype(np.float16))) <= 1


def test_store_beta_gelu_bias():
    g, a, b, acc = _exact_case(24)
    M, N = acc.shape
    acc_small = acc / 16.0
    a = (a.astype(np.float64) / 16.0).astype(np.float16)
    bias, prev = randn_f16(g, (N,), 1.0), randn_f16(g, (M, N), 1.0)
    got = _epilogue(a, b, M, a.shape[1], N, prev, store=oracle.STORE_BETA_GELU_BIAS, bias=bias,
                    beta=0.75)
    v = acc_small + bias.astype(np.float64)[None, :]
    gelu = 0.5 * v * (1.0 + np.tanh(0.7978845608028654 * (v + 0.044715 * v ** 3)))
    ref = gelu + 0.75 * prev.astype(np.float64)
    assert np.max(ulp_diff_f16(got, ref.astype(np.float16))) <= 1


def test_causal_mask_writes_negative_infinity_above_the_diagonal():
    g, a, b, acc = _exact_case(25, M=6, N=10)
    M, N = acc.shape
    plain = _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)))
    got = _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), mask=oracle.MASK_CAUSAL)
    y, x = np.mgrid[0:M, 0:N]
    assert np.all(got.view(np.uint16)[x > y] == 0xFC00)
    assert np.array_equal(got[x <= y], plain[x <= y])
    # masked elements ignore the store operator (matmul.cu:210-213 returns before it)
    got = _epilogue(a, b, M, a.shape[1], N, np.ones((M, N)), mask=oracle.MASK_CAUSAL,
                    store=oracle.STORE_ADD)
    assert np.all(got.view(np.uint16)[x > y] == 0xFC00)
    assert np.array_equal(got[x <= y], (plain.astype(np.float64) + 1.0).astype(np.float16)[x <= y])


def test_load_scale_scales_both_operands_in_fp16():
    g, a, b, acc = _exact_case(26)
    M, N = acc.shape
    got = _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), load=oracle.LOAD_SCALE, scale=0.5,
                    mode=oracle.EXACT)
    assert np.array_equal(got, (acc * 0.25).astype(np.float16))
    # a non power-of-two scale: operands are rounded to fp16 after scaling
    s = 128.0 ** -0.25
    s16 = np.float16(np.float32(s))
    a2 = (a.astype(np.float64) * np.float64(s16)).astype(np.float16)
    b2 = (b.astype(np.float64) * np.float64(s16)).astype(np.float16)
    ref = (a2.astype(np.float64) @ b2.astype(np.float64)).astype(np.float32).astype(np.float16)
    got = _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), load=oracle.LOAD_SCALE, scale=s,
                    mode=oracle.EXACT)
    assert np.array_equal(got.view(np.uint16), ref.view(np.uint16))


def test_load_and_store_scale_share_one_value():
    """kernels.rs:837-843 merges both scales into one float, which the device then applies at
    load (twice) and at store: the product ends up scaled three times."""
    g, a, b, acc = _exact_case(27)
    M, N = acc.shape
    got = _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), load=oracle.LOAD_SCALE,
                    store=oracle.STORE_SCALE, scale=0.5, mode=oracle.EXACT)
    assert np.array_equal(got, (acc * 0.125).astype(np.float16))


def test_invalid_requests_are_rejected():
    g, a, b, acc = _exact_case(28)
    M, N = acc.shape
    with pytest.raises(ValueError):  # GeluBias lowers from Rust but has no device case
        _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), store=oracle.STORE_GELU_BIAS,
                  bias=np.zeros(N, np.float16))
    with pytest.raises(ValueError):  # bias operator without a bias vector
        _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), store=oracle.STORE_BETA_BIAS)
    with pytest.raises(ValueError):
        _epilogue(a, b, M, a.shape[1], N, np.zeros((M, N)), store=7)


def test_overflow_saturates_to_infinity():
    a = np.full((1, 4), 200.0, np.float16)
    b = np.full((4, 1), 200.0, np.float16)
    out = np.zeros(1, np.float16)
    run(out, a, b, 1, 1, 4, 1, (1, 1, 0), (1, 4, 0), (1, 1, 0), mode=oracle.EXACT)
    assert out.view(np.uint16)[0] == 0x7C00


@pytest.mark.parametrize("mkn", [(1, 1, 1), (5, 300, 7), (64, 256, 64), (70, 513, 131), (130, 64, 3)])
def test_blocked_sgemm_baseline_matches_numpy(mkn):
    """The OpenMP fp32 GEMM that bench.py times as a CPU baseline: ragged panels in all three
    dimensions against numpy's float64 product, and small integers exactly."""
    m, k, n = mkn
    g = rng(7000 + m + k + n)
    a = g.standard_normal((m, k)).astype(np.float32)
    b = g.standard_normal((n, k)).astype(np.float32)
    got = oracle.sgemm_nt(a, b, threads=4)
    ref = a.astype(np.float64) @ b.astype(np.float64).T
    assert np.max(np.abs(got - ref)) <= 1e-4 * max(1.0, np.max(np.abs(ref)))
    ai = g.integers(-8, 9, size=(m, k)).astype(np.float32)
    bi = g.integers(-8, 9, size=(n, k)).astype(np.float32)
    assert np.array_equal(oracle.sgemm_nt(ai, bi, threads=3), ai @ bi.T)
