"""GPU parity of the fp16 matmul entry points (through the C ABI) against the CPU oracle, the
reference's own naive kernel (oracle/_ref, when built) and an fp32/fp64 GEMM.

Bars: bit-exact where the arithmetic is exactly determined (dyadic inputs, fp16-only operators,
mask pattern, the step-for-step slow kernel); max relative error <= 1e-2 against an fp32/fp64
GEMM on random inputs (the stated tolerance of this path: fp16 output, fp32 accumulation).
"""
import itertools

import numpy as np
import pytest
import torch

import oracle
from adrastea_amd import _ffi
from helpers import rng, randn_f16, ulp_diff_f16, max_rel_err, largest_address, view
from gpu_common import to_dev, to_np, raw_matmul, oracle_matmul, plan

pytestmark = pytest.mark.gpu

TOL = 1e-2  # max relative error vs an fp32/fp64 GEMM (fp16 output, fp32 accumulation)


def dyadic(g, shape):
    return (g.integers(-256, 257, size=shape) / 64.0).astype(np.float16)


def nt_strides(M, K, N):
    # output row-major, lhs row-major, rhs = W[N,K].permute([1,0])
    return (1, N, 0), (1, K, 0), (K, 1, 0)


@pytest.fixture(scope="module")
def ref():
    import refgpu
    if not refgpu.available():
        pytest.skip("oracle/_ref code objects not built")
    return refgpu.RefKernels()


# ------------------------------------------------------------------ slow (step-for-step) kernel

STORES_EXACT = [oracle.STORE_IDENTITY, oracle.STORE_SCALE, oracle.STORE_ADD]
STORES_F32 = [oracle.STORE_BETA_BIAS, oracle.STORE_QUICK_GELU_BIAS, oracle.STORE_BETA_GELU_BIAS]


def _random_layout_case(g, B, M, K, N):
    perms = list(itertools.permutations(range(3)))

    def layout(shape, perm, pad):
        strides, s = [0, 0, 0], pad
        for d in reversed(perm):
            strides[d] = s
            s *= shape[d] + 1
        return strides
    po, pl, pr = (perms[i] for i in g.integers(0, 6, size=3))
    so3 = layout((B, M, N), po, 1)
    sl3 = layout((B, M, K), pl, int(g.integers(1, 3)))
    sr3 = layout((B, K, N), pr, int(g.integers(1, 3)))
    return so3, sl3, sr3


@pytest.mark.parametrize("store", STORES_EXACT + STORES_F32)
@pytest.mark.parametrize("load", [oracle.LOAD_IDENTITY, oracle.LOAD_SCALE])
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
def test_slow_kernel_matches_faithful_oracle(store, load, mask):
    g = rng(100 + store * 10 + load * 2 + mask)
    B, M, K, N = 3, 19, 45, 21
    so3, sl3, sr3 = _random_layout_case(g, B, M, K, N)
    lbuf = randn_f16(g, largest_address((B, M, K), sl3) + 4)
    rbuf = randn_f16(g, largest_address((B, K, N), sr3) + 3, 0.2)
    obuf = randn_f16(g, largest_address((B, M, N), so3) + 2)
    bias = randn_f16(g, N)
    so, sl, sr = (so3[2], so3[1], so3[0]), (sl3[2], sl3[1], sl3[0]), (sr3[2], sr3[1], sr3[0])
    kw = dict(beta=0.6, scale=0.37, store=store, load=load, mask=mask, offsets=(1, 3, 2))
    want = oracle_matmul(obuf, lbuf, rbuf, B, M, K, N, so, sl, sr, bias=bias,
                         mode=oracle.FAITHFUL, **kw)
    o_t, l_t, r_t, b_t = to_dev(obuf), to_dev(lbuf), to_dev(rbuf), to_dev(bias)
    rc = raw_matmul("adr_matmul_f16_slow", o_t, l_t, r_t, B, M, K, N, so, sl, sr, bias_t=b_t, **kw)
    assert rc == 0
    got = to_np(o_t)
    if store in STORES_EXACT:
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    else:
        # fp32 epilogue: the device may fuse a multiply-add or use its own expf/tanhf
        assert np.max(ulp_diff_f16(got, want)) <= 2


@pytest.mark.parametrize("store", STORES_EXACT + STORES_F32)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
def test_oracle_and_slow_kernel_match_reference_naive_kernel(ref, store, mask):
    """The reference's own matmul_f16 kernel, compiled for gfx950, on the same inputs: pins the
    C restatement (faithful mode) and the slow kernel to the real thing."""
    g = rng(200 + store * 2 + mask)
    B, M, K, N = 2, 37, 70, 41
    so3, sl3, sr3 = _random_layout_case(g, B, M, K, N)
    lbuf = randn_f16(g, largest_address((B, M, K), sl3) + 1)
    rbuf = randn_f16(g, largest_address((B, K, N), sr3) + 1, 0.2)
    obuf = randn_f16(g, largest_address((B, M, N), so3) + 1)
    bias = randn_f16(g, N)
    so, sl, sr = (so3[2], so3[1], so3[0]), (sl3[2], sl3[1], sl3[0]), (sr3[2], sr3[1], sr3[0])
    kw = dict(beta=-0.4, scale=0.2, store=store, load=oracle.LOAD_IDENTITY, mask=mask)
    l_t, r_t, b_t = to_dev(lbuf), to_dev(rbuf), to_dev(bias)
    o_ref = to_dev(obuf)
    ref.matmul_f16(o_ref.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, so, sl, sr,
                   bias_ptr=b_t.data_ptr(), **kw)
    torch.cuda.synchronize()
    want = to_np(o_ref)
    o_t = to_dev(obuf)
    assert raw_matmul("adr_matmul_f16_slow", o_t, l_t, r_t, B, M, K, N, so, sl, sr, bias_t=b_t,
                      **kw) == 0
    got = to_np(o_t)
    orc = oracle_matmul(obuf, lbuf, rbuf, B, M, K, N, so, sl, sr, bias=bias, mode=oracle.FAITHFUL,
                        **kw)
    if store in STORES_EXACT:
        assert np.array_equal(orc.view(np.uint16), want.view(np.uint16))
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    else:
        assert np.max(ulp_diff_f16(orc, want)) <= 2
        assert np.max(ulp_diff_f16(got, want)) <= 2


def test_reference_tiled_kernel_agrees_with_its_naive_kernel(ref):
    """matmul_f16_fast (the production kernel of the reference) sums in the same k order with the
    same fp16 products: the two reference kernels, and therefore the oracle, must agree."""
    g = rng(210)
    B, M, K, N = 2, 50, 75, 70  # K % 32 != 0 exercises its scalar tail loop
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, K * N)
    l, r = randn_f16(g, B * M * K), randn_f16(g, B * K * N, 0.2)
    l_t, r_t = to_dev(l), to_dev(r)
    o1, o2 = to_dev(np.zeros(B * M * N, np.float16)), to_dev(np.zeros(B * M * N, np.float16))
    ref.matmul_f16(o1.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, so, sl, sr)
    ref.matmul_f16_fast(o2.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, so, sl, sr)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(o1).view(np.uint16), to_np(o2).view(np.uint16))


# ------------------------------------------------------------------ fast (MFMA) path

SHAPES = [
    # (B, M, K, N): tails in every dimension, every tile configuration
    (1, 77, 768, 2304),     # benchmark config 1 (CLIP text QKV)
    (1, 64, 64, 64),
    (1, 1, 8, 1),
    (1, 33, 72, 130),
    (1, 300, 200, 520),
    (1, 515, 136, 1100),
    (3, 129, 96, 257),
    (1, 2056, 256, 1024),   # config-2-like M tail with the large tile
    (1, 1000, 320, 2040),   # 128x64 tiles (256 of them), ragged in M and N
    (1, 2056, 320, 1024),   # 128x128 tiles, three stages, K tail of the 3-slice loop
]


@pytest.mark.parametrize("shape", SHAPES)
def test_fast_nt_bit_exact_on_dyadic_inputs(shape):
    B, M, K, N = shape
    g = rng(300 + M + N)
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, K * N)
    assert plan(B, M, K, N, so, sl, sr).startswith("gemm_nt_mfma")
    # k/64 values in [-1/8, 1/8]: sums of up to 768 products stay exact in fp32
    l = (g.integers(-8, 9, size=B * M * K) / 64.0).astype(np.float16)
    r = (g.integers(-8, 9, size=B * K * N) / 64.0).astype(np.float16)
    o_t = to_dev(np.full(B * M * N, 9.0, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr) == 0
    want = np.einsum("bmk,bnk->bmn", l.reshape(B, M, K).astype(np.float64),
                     r.reshape(B, N, K).astype(np.float64)).astype(np.float32).astype(np.float16)
    assert np.array_equal(to_np(o_t).reshape(B, M, N).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("shape", SHAPES)
def test_fast_nt_random_within_tolerance_and_close_to_oracle(shape):
    B, M, K, N = shape
    g = rng(400 + M + N)
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, K * N)
    l, r = randn_f16(g, B * M * K), randn_f16(g, B * K * N, K ** -0.5)
    o_t = to_dev(np.zeros(B * M * N, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr) == 0
    got = to_np(o_t).reshape(B, M, N)
    ref64 = np.einsum("bmk,bnk->bmn", l.reshape(B, M, K).astype(np.float64),
                      r.reshape(B, N, K).astype(np.float64))
    assert max_rel_err(got, ref64) <= TOL
    # exact products + fp32 accumulation: within one fp16 step of the correctly rounded result
    assert np.max(ulp_diff_f16(got, ref64.astype(np.float16))) <= 1 or max_rel_err(got, ref64) <= 2e-3


@pytest.mark.parametrize("store", STORES_EXACT + STORES_F32)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
def test_fast_nt_epilogues_match_oracle(store, mask):
    g = rng(500 + store * 2 + mask)
    B, M, K, N = 2, 150, 64, 200
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, K * N)
    assert plan(B, M, K, N, so, sl, sr, store=store, mask=mask).startswith("gemm_nt_mfma")
    l = (g.integers(-16, 17, size=B * M * K) / 16.0).astype(np.float16)
    r = (g.integers(-16, 17, size=B * K * N) / 16.0).astype(np.float16)
    prev, bias = randn_f16(g, B * M * N), randn_f16(g, N)
    kw = dict(beta=0.7, scale=0.2, store=store, load=oracle.LOAD_IDENTITY, mask=mask)
    want = oracle_matmul(prev, l, r, B, M, K, N, so, sl, sr, bias=bias, mode=oracle.EXACT, **kw)
    o_t = to_dev(prev)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr,
                      bias_t=to_dev(bias), **kw) == 0
    got = to_np(o_t)
    if store in STORES_EXACT:
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    else:
        assert np.max(ulp_diff_f16(got, want)) <= 2
    if mask == oracle.MASK_CAUSAL:
        y, x = np.mgrid[0:M, 0:N]
        assert np.all(got.reshape(B, M, N).view(np.uint16)[:, x > y] == 0xFC00)


@pytest.mark.parametrize("store", STORES_EXACT + STORES_F32)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
@pytest.mark.parametrize("shape", [(2, 150, 64, 201, 0), (1, 300, 128, 333, 1), (3, 70, 192, 1001, 1),
                                   (1, 448, 128, 2047, 0)], ids=lambda v: str(v))
def test_fast_nt_epilogues_into_rows_of_an_odd_length(store, mask, shape):
    """A dense [M, N] result with an odd N (the 51865 logits of the Whisper decoder): its rows
    start at any even address, so chunks go out piecewise (the operators that read nothing back)
    or element by element; the output may start at an odd element too.  Same bits as aligned
    rows would get, and nothing written outside the rows."""
    B, M, K, N, off = shape
    g = rng(700 + store * 2 + mask + N)
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, K * N)
    assert plan(B, M, K, N, so, sl, sr, store=store, mask=mask).startswith("gemm_nt_mfma")
    l = (g.integers(-16, 17, size=B * M * K) / 16.0).astype(np.float16)
    r = (g.integers(-16, 17, size=B * K * N) / 16.0).astype(np.float16)
    prev, bias = randn_f16(g, off + B * M * N + 3), randn_f16(g, N)
    kw = dict(beta=0.7, scale=0.2, store=store, load=oracle.LOAD_IDENTITY, mask=mask)
    want = oracle_matmul(prev, l, r, B, M, K, N, so, sl, sr, bias=bias, mode=oracle.EXACT,
                         offsets=(off, 0, 0), **kw)
    o_t = to_dev(prev)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr,
                      bias_t=to_dev(bias), offsets=(off, 0, 0), **kw) == 0
    got = to_np(o_t)
    assert np.array_equal(got[:off].view(np.uint16), prev[:off].view(np.uint16))
    assert np.array_equal(got[-3:].view(np.uint16), prev[-3:].view(np.uint16))
    if store in STORES_EXACT:
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    else:
        # (the fp32 operator may fuse its multiply and add: a third step only where v + beta * prev
        # cancels to almost nothing)
        steps = ulp_diff_f16(got, want)
        assert np.count_nonzero(steps > 2) <= 1e-5 * steps.size
        assert np.max(steps) <= 8


def test_up_to_64_rows_against_a_little_more_than_one_small_tile_per_cu():
    """280 tiles of 64 x 64 on 256 compute units leave most of a second round empty: one 128 x 128
    tile per CU takes such products; 500 tiles fill both rounds and stay."""
    def nt(M, K, N):
        return (1, N, 0), (1, K, 0), (K, 1, 0)
    assert plan(1, 64, 4096, 17920, *nt(64, 4096, 17920)) == "gemm_nt_mfma_dma_128x128x64"
    assert plan(1, 40, 3072, 24576, *nt(40, 3072, 24576)) == "gemm_nt_mfma_dma_128x128x64"
    assert plan(1, 64, 4096, 32000, *nt(64, 4096, 32000)) == "gemm_nt_mfma_dma_64x64x64"
    M, K, N = 50, 3072, 17000
    so, sl, sr = nt(M, K, N)
    assert plan(1, M, K, N, so, sl, sr) == "gemm_nt_mfma_dma_128x128x64"
    gen = torch.Generator(device="cuda").manual_seed(77)   # small integers: every sum is exact
    l = torch.randint(-3, 4, (M, K), generator=gen, device="cuda").half()
    r = torch.randint(-2, 3, (N, K), generator=gen, device="cuda").half()
    out = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16", out, l, r, 1, M, K, N, so, sl, sr) == 0
    want = (l.double() @ r.double().t()).half()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_fast_nt_load_scale():
    g = rng(520)
    B, M, K, N = 1, 100, 128, 90
    so, sl, sr = (1, N, 0), (1, K, 0), (K, 1, 0)
    l, r = randn_f16(g, M * K), randn_f16(g, K * N, 0.1)
    scale = 64.0 ** -0.25  # Whisper's d_head^-0.25 (whisper.rs:424-430)
    want = oracle_matmul(np.zeros(M * N, np.float16), l, r, B, M, K, N, so, sl, sr,
                         load=oracle.LOAD_SCALE, scale=scale, mode=oracle.EXACT)
    o_t = to_dev(np.zeros(M * N, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr,
                      load=oracle.LOAD_SCALE, scale=scale) == 0
    assert np.max(ulp_diff_f16(to_np(o_t), want)) <= 1


def test_attention_views_qk_and_pv():
    """llama.rs:534-554 with S=160, 4 heads, head_dim 64: QK^T with Scale + Causal on the
    interleaved-head views, then P.V into the strided output view."""
    g = rng(530)
    S, H, D = 192, 4, 64
    HD = H * D
    q, k, v = (dyadic(g, S * HD) for _ in range(3))
    scale = 1.0 / np.sqrt(D)
    so, sl, sr = (1, S, S * S), (1, HD, D), (HD, 1, D)
    assert plan(H, S, D, S, so, sl, sr, store=4, mask=1).startswith("gemm_nt_mfma")
    kw = dict(store=oracle.STORE_SCALE, scale=scale, mask=oracle.MASK_CAUSAL)
    want = oracle_matmul(np.zeros(H * S * S, np.float16), q, k, H, S, D, S, so, sl, sr,
                         mode=oracle.EXACT, **kw)
    qk_t = to_dev(np.zeros(H * S * S, np.float16))
    assert raw_matmul("adr_matmul_f16", qk_t, to_dev(q), to_dev(k), H, S, D, S, so, sl, sr, **kw) == 0
    assert np.array_equal(to_np(qk_t).view(np.uint16), want.view(np.uint16))
    # P.V: probabilities k/64 in [0, 1/8]
    p = (g.integers(0, 9, size=H * S * S) / 64.0).astype(np.float16)
    so, sl, sr = (1, HD, D), (1, S, S * S), (1, HD, D)
    # the general kernel rounds each product to fp16 like the reference; a tiled kernel does not
    mode = oracle.FAITHFUL if plan(H, S, S, D, so, sl, sr) == "matmul_general" else oracle.EXACT
    want = oracle_matmul(np.zeros(S * HD, np.float16), p, v, H, S, S, D, so, sl, sr, mode=mode)
    o_t = to_dev(np.zeros(S * HD, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(p), to_dev(v), H, S, S, D, so, sl, sr) == 0
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))


PV_SHAPES = [
    # (heads, S, T, D, extra elements before the first probability, kernel)
    (12, 77, 77, 64, 0, "128x64x64"),        # CLIP text: rows of 154 bytes
    (16, 257, 257, 64, 0, "32x64x64_k4"),    # CLIP vision, one image
    (3, 300, 301, 128, 1, "32x64x64_k4"),    # odd pitch and an odd first address
    (2, 1500, 1500, 64, 0, "32x64x64_k4"),   # Whisper: rows aligned to 8 bytes, K ends inside a chunk
    (2, 130, 1999, 128, 3, "32x64x64_k4"),   # a long odd K
    (2, 200, 1000, 128, 0, "32x64x64_k4"),   # 16-byte aligned rows, K no multiple of 64
    (20, 5, 1500, 64, 0, "32x64x64_k4"),     # the first steps of the Whisper decoder against 1500 frames
    (32, 1, 2047, 128, 1, "32x64x64_k4"),    # one query row against a long context
    (32, 1, 2048, 128, 0, "32x64x64_k4"),    # ... whose length is a multiple of 64
    (20, 448, 1536, 64, 0, "64x64x64_k4"),
    (32, 300, 333, 64, 1, "64x64x64_k4"),    # more 32-row tiles than compute units
    (20, 448, 1500, 64, 0, "64x64x64_k4"),   # the last steps of the Whisper decoder
    (40, 500, 200, 64, 1, "128x64x64"),      # more 64-row tiles than compute units, heads of 64
    (8, 1100, 257, 128, 0, "128x64x64"),     # heads of 128 on few tiles: 64-column tiles
    (16, 1100, 321, 128, 1, "128x128x64"),
    (4, 600, 130, 72, 0, "128x64x64"),       # 72 columns: a full and a ragged column tile
    (3, 70, 500, 200, 1, "32x64x64_k4"),     # 200 columns: three full column tiles and 8 columns
]


def _pv_case(H, S, T, D, off, pitch=None, gen=None):
    """Probabilities (multiples of 1/64 up to 1/8) as [H, S, T] rows of `pitch` elements that end
    with the buffer, values (multiples of 1/16), the output and the strides of the head views."""
    pitch = pitch or T
    HD = H * D
    pbuf = (torch.randint(0, 9, (off + (H * S - 1) * pitch + T,), generator=gen, device="cuda").float() / 64).half()
    v = (torch.randint(-8, 9, (T, HD), generator=gen, device="cuda").float() / 16).half()
    out = torch.full((S, HD), 3.0, dtype=torch.float16, device="cuda")
    return pbuf, v, out, ((1, HD, D), (1, pitch, S * pitch), (1, HD, D))


def _pv_want(pbuf, v, H, S, T, D, off, pitch=None):
    pitch = pitch or T
    p = torch.as_strided(pbuf, (H, S, T), (S * pitch, pitch, 1), off).double()
    return torch.bmm(p, v.view(T, H, D).permute(1, 0, 2).double()).permute(1, 0, 2).reshape(S, H * D).half()


@pytest.mark.parametrize("H,S,T,D,off,kernel", PV_SHAPES, ids=lambda v: str(v))
def test_pv_of_sequence_lengths_that_are_no_multiple_of_64(H, S, T, D, off, kernel):
    """P.V on the views of llama.rs:552-554 / clip.rs:385-388 / whisper.rs:433-436 when the
    probabilities' rows start at any even address and K = T ends inside a slice: the tiled kernel
    that shifts the left operand into place, on every tile it has, on inputs whose fp32 sums are
    exact; the last probability is the last element of its buffer (nothing may be read past it
    that matters)."""
    gen = torch.Generator(device="cuda").manual_seed(H * S + T)
    pbuf, v, out, (so, sl, sr) = _pv_case(H, S, T, D, off, gen=gen)
    assert plan(H, S, T, D, so, sl, sr) == "gemm_nn_mfma_anyrow_" + kernel
    assert raw_matmul("adr_matmul_f16", out, pbuf, v, H, S, T, D, so, sl, sr, offsets=(0, off, 0)) == 0
    want = _pv_want(pbuf, v, H, S, T, D, off)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


# K from one slice to many: the kernel runs a steady loop of two slices a trip from its fifth
# slice on (per group of wavefronts: from K > 1024 where four groups share K) and a tail of up to
# four; every remainder of both, K ending on a slice, one element behind and one before it
_PV_K = {
    "32x64x64_k4": (3, 40, 64, [193, 255, 257, 319, 511, 700, 1024, 1025, 1100, 1281, 1345,
                                1537, 1601, 1857, 1999, 2305, 2560]),
    "64x64x64_k4": (32, 300, 64, [193, 255, 321, 449, 1025, 1088, 1282, 1409]),
    "128x64x64": (40, 500, 64, [193, 255, 257, 321, 385, 449, 513]),
    "128x128x64": (16, 1100, 128, [193, 255, 258, 322, 385]),
}


@pytest.mark.parametrize("kernel,T", [(k, t) for k, (_, _, _, ts) in _PV_K.items() for t in ts],
                         ids=lambda v: str(v))
def test_pv_anyrow_tiles_every_remainder_of_their_loops(kernel, T):
    H, S, D, _ = _PV_K[kernel]
    gen = torch.Generator(device="cuda").manual_seed(T)
    off = T % 2
    pbuf, v, out, (so, sl, sr) = _pv_case(H, S, T, D, off, gen=gen)
    assert plan(H, S, T, D, so, sl, sr) == "gemm_nn_mfma_anyrow_" + kernel
    assert raw_matmul("adr_matmul_f16", out, pbuf, v, H, S, T, D, so, sl, sr, offsets=(0, off, 0)) == 0
    want = _pv_want(pbuf, v, H, S, T, D, off)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("H,S,T,D,off", [(1, 1, 12, 8, 0), (1, 1, 13, 8, 1), (1, 2, 7, 8, 0),
                                          (1, 3, 5, 16, 1), (2, 1, 9, 8, 0), (1, 1, 5, 8, 0),
                                          (1, 2, 3, 8, 1), (1, 1, 1, 8, 0)], ids=lambda v: str(v))
def test_pv_of_a_handful_of_probabilities(H, S, T, D, off):
    """Left operands of a few bytes that end with their buffer: the tiled kernel (whose 16-byte
    loads start up to 12 bytes before the last dword) from 12 elements on, another kernel below
    that; the same sums either way."""
    gen = torch.Generator(device="cuda").manual_seed(T)
    pbuf, v, out, (so, sl, sr) = _pv_case(H, S, T, D, off, gen=gen)
    tiled = plan(H, S, T, D, so, sl, sr).startswith("gemm_nn_mfma_anyrow")
    assert tiled == ((H * S - 1) * T + T >= 12)
    assert raw_matmul("adr_matmul_f16", out, pbuf, v, H, S, T, D, so, sl, sr, offsets=(0, off, 0)) == 0
    want = _pv_want(pbuf, v, H, S, T, D, off)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("H,S,T,D,pitch,kernel", [(2, 140, 70, 64, 75, "128x64x64"),
                                                  (2, 140, 326, 64, 331, "32x64x64_k4"),
                                                  (40, 330, 1030, 64, 1033, "64x64x64_k4")],
                         ids=lambda v: str(v))
def test_pv_anyrow_kernel_ignores_what_follows_k(H, S, T, D, pitch, kernel):
    """Non-finite values right behind a row's K elements (the next row's first probabilities, or
    whatever follows the tensor) must not reach the sums: rows of T probabilities inside a
    longer pitch, the elements in between set to NaN."""
    HD = H * D
    gen = torch.Generator(device="cuda").manual_seed(3)
    pbuf = torch.full((H * S * pitch,), float("nan"), dtype=torch.float16, device="cuda")
    p = (torch.randint(0, 9, (H, S, T), generator=gen, device="cuda").float() / 64).half()
    pbuf.view(H, S, pitch)[:, :, :T] = p
    v = (torch.randint(-8, 9, (T, HD), generator=gen, device="cuda").float() / 16).half()
    out = torch.zeros(S, HD, dtype=torch.float16, device="cuda")
    so, sl, sr = (1, HD, D), (1, pitch, S * pitch), (1, HD, D)
    assert plan(H, S, T, D, so, sl, sr) == "gemm_nn_mfma_anyrow_" + kernel
    assert raw_matmul("adr_matmul_f16", out, pbuf, v, H, S, T, D, so, sl, sr) == 0
    want = torch.bmm(p.double(), v.view(T, H, D).permute(1, 0, 2).double()).permute(1, 0, 2).reshape(S, HD).half()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


SHORTK = [
    # (B, M, K, N): at least 512 tiles of 128x128 so that the persistent kernel is selected
    (9, 1000, 128, 1000),    # ragged tiles in M and N, 64 tiles per batch
    (40, 500, 64, 450),      # K = 64 variant, 16 tiles per batch
    (3, 1700, 128, 1800),    # more tiles than workgroups per batch, odd tile counts
]


@pytest.mark.parametrize("shape", SHORTK, ids=lambda c: "B%d_M%d_K%d_N%d" % c)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
def test_persistent_short_k_kernel_head_views(shape, mask):
    """QK^T-shaped products (K = head size) on interleaved head views as in llama.rs:534-545:
    every workgroup walks several tiles, including ragged, diagonal and fully masked ones."""
    B, M, K, N = shape
    g = rng(900 + B + M + mask)
    HD = B * K
    # heads interleaved in the rows of [S, H*D] buffers; output [H, M, N] with padded rows
    NP = N + 8
    so, sl, sr = (1, NP, M * NP), (1, HD, K), (HD, 1, K)
    assert plan(B, M, K, N, so, sl, sr, store=oracle.STORE_SCALE, mask=mask).startswith(
        "gemm_nt_mfma_persistent")
    l, r = dyadic(g, M * HD), dyadic(g, N * HD)
    prev = randn_f16(g, B * M * NP)
    kw = dict(store=oracle.STORE_SCALE, scale=0.125, mask=mask)
    want = oracle_matmul(prev, l, r, B, M, K, N, so, sl, sr, mode=oracle.EXACT, **kw)
    o_t = to_dev(prev)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr, **kw) == 0
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("pad", [1, 3, 4], ids=["rows_aligned_to_8_bytes", "to_4_bytes", "to_2_bytes"])
def test_persistent_short_k_kernel_causal_rows_not_16_byte_aligned(pad):
    """The causal score product into rows that no 16-byte store may touch (a sequence length that
    is not a multiple of 8): the tiles go out in 8-, 4- or 2-byte pieces, the run of -inf right of
    the diagonal tile element by element, to the same bits."""
    B, M, K, N = 9, 1000, 128, 1003
    g = rng(930 + pad)
    HD = B * K
    NP = N + pad
    so, sl, sr = (1, NP, M * NP), (1, HD, K), (HD, 1, K)
    kw = dict(store=oracle.STORE_SCALE, scale=0.125, mask=oracle.MASK_CAUSAL)
    assert plan(B, M, K, N, so, sl, sr, store=oracle.STORE_SCALE,
                mask=oracle.MASK_CAUSAL).startswith("gemm_nt_mfma_persistent")
    l, r = dyadic(g, M * HD), dyadic(g, N * HD)
    prev = randn_f16(g, B * M * NP)
    want = oracle_matmul(prev, l, r, B, M, K, N, so, sl, sr, mode=oracle.EXACT, **kw)
    o_t = to_dev(prev)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr, **kw) == 0
    got = to_np(o_t)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    # the padding between rows keeps what it held
    assert np.array_equal(got.reshape(B, M, NP)[:, :, N:], prev.reshape(B, M, NP)[:, :, N:])


@pytest.mark.parametrize("K,N", [(64, 1500), (128, 1000)])
def test_persistent_short_k_kernel_load_scale(K, N):
    """Whisper's score product (whisper.rs:424-430: both operands times d_head^-0.25 in fp16 before
    the product) on the persistent kernel: 1500 positions, rows of the score tensor aligned to
    8 bytes only."""
    B, M = 6, 1500
    g = rng(960 + K)
    HD = B * K
    so, sl, sr = (1, N, M * N), (1, HD, K), (HD, 1, K)
    scale = float(K) ** -0.25
    assert plan(B, M, K, N, so, sl, sr, load=oracle.LOAD_SCALE).startswith("gemm_nt_mfma_persistent")
    l, r = randn_f16(g, M * HD), randn_f16(g, N * HD)
    want = oracle_matmul(np.zeros(B * M * N, np.float16), l, r, B, M, K, N, so, sl, sr,
                         load=oracle.LOAD_SCALE, scale=scale, mode=oracle.EXACT)
    o_t = to_dev(np.zeros(B * M * N, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr,
                      load=oracle.LOAD_SCALE, scale=scale) == 0
    # the scaled operands are the same fp16 numbers; the fp32 sums run in another order, which
    # shows as a second step only where products cancel to almost nothing
    got, ref = to_np(o_t).astype(np.float64), want.astype(np.float64)
    floor = 1e-2 * np.sqrt(np.mean(ref * ref))
    assert np.max(np.abs(got - ref) / np.maximum(np.abs(ref), floor)) <= 2.0 ** -10
    assert np.count_nonzero(ulp_diff_f16(to_np(o_t), want) > 1) <= 1e-4 * want.size


@pytest.mark.parametrize("store", [oracle.STORE_ADD] + STORES_F32)
def test_persistent_short_k_kernel_epilogues(store):
    g = rng(950 + store)
    B, M, K, N = 20, 640, 128, 650
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, K * N)
    assert plan(B, M, K, N, so, sl, sr, store=store).startswith("gemm_nt_mfma_persistent")
    l = (g.integers(-16, 17, size=B * M * K) / 16.0).astype(np.float16)
    r = (g.integers(-16, 17, size=B * K * N) / 16.0).astype(np.float16)
    prev, bias = randn_f16(g, B * M * N), randn_f16(g, N)
    kw = dict(beta=0.7, scale=0.2, store=store, mask=oracle.MASK_CAUSAL)
    want = oracle_matmul(prev, l, r, B, M, K, N, so, sl, sr, bias=bias, mode=oracle.EXACT, **kw)
    o_t = to_dev(prev)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr,
                      bias_t=to_dev(bias), **kw) == 0
    got = to_np(o_t)
    if store in STORES_EXACT:
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    else:
        assert np.max(ulp_diff_f16(got, want)) <= 2


NN_SHAPES = [(2, 100, 128, 136), (1, 300, 64, 128), (3, 257, 192, 72), (1, 64, 64, 8),
             (2, 513, 256, 264),
             # few tiles and a long K: the small tiles whose wavefront groups share K
             (2, 100, 1024, 136), (2, 90, 1030, 72), (3, 200, 300, 136), (40, 300, 1088, 64)]


@pytest.mark.parametrize("shape", NN_SHAPES)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
def test_fast_nn_row_major_right_operand(shape, mask):
    """Right operand stored [K, N] row-major (n contiguous), as V is in P.V: goes through the
    transposing LDS reads.  Padded row and batch strides; dyadic inputs -> bit-exact."""
    B, M, K, N = shape
    g = rng(535 + M + N)
    ly, ry, oy = K + 8, N + 16, N + 8
    lz, rz, oz = M * ly + 16, K * ry + 8, M * oy + 24
    so, sl, sr = (1, oy, oz), (1, ly, lz), (1, ry, rz)
    assert plan(B, M, K, N, so, sl, sr, mask=mask).startswith("gemm_nn_mfma")
    lbuf = (g.integers(-8, 9, size=B * lz + 8) / 64.0).astype(np.float16)
    rbuf = (g.integers(-8, 9, size=B * rz + 8) / 64.0).astype(np.float16)
    obuf = np.full(B * oz + 8, 3.0, np.float16)
    want = oracle_matmul(obuf, lbuf, rbuf, B, M, K, N, so, sl, sr, mode=oracle.EXACT, mask=mask,
                         offsets=(8, 8, 8))
    o_t = to_dev(obuf)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(lbuf), to_dev(rbuf), B, M, K, N, so, sl, sr,
                      mask=mask, offsets=(8, 8, 8)) == 0
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))


def test_row_and_batch_strides_with_padding_on_the_fast_path():
    g = rng(540)
    B, M, K, N = 2, 70, 96, 150
    ly, rx, oy = K + 8, K + 16, N + 5
    lz, rz, oz = M * ly + 8, N * rx + 24, M * oy + 3
    so, sl, sr = (1, oy, oz), (1, ly, lz), (rx, 1, rz)
    assert plan(B, M, K, N, so, sl, sr).startswith("gemm_nt_mfma")
    lbuf, rbuf = dyadic(g, B * lz + 8), dyadic(g, B * rz + 8)
    obuf = np.full(B * oz + 8, 5.0, np.float16)
    want = oracle_matmul(obuf, lbuf, rbuf, B, M, K, N, so, sl, sr, mode=oracle.EXACT,
                         offsets=(3, 8, 8))
    o_t = to_dev(obuf)
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(lbuf), to_dev(rbuf), B, M, K, N, so, sl, sr,
                      offsets=(3, 8, 8)) == 0
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))  # gaps untouched too


@pytest.mark.parametrize("B,M,K,N,tile", [(2, 600, 1088, 6136, "128x256"), (2, 380, 1088, 6136, "128x192"),
                                          (2, 1000, 1088, 4088, "256x128"), (4, 1000, 1088, 3064, "256x192"),
                                          (3, 1000, 1088, 3064, "256x160")])
def test_batched_padded_operands_on_the_large_tiles(B, M, K, N, tile):
    """Batches with row pitches wider than the rows and batch strides wider than the matrices on
    every large tile (16 x 16 and 32 x 32 accumulator blocks), exact inputs; whatever lies between
    the rows and after the last batch of the output must stay as it was."""
    ly, rx, oy = K + 8, K + 16, N + 8
    lz, rz, oz = M * ly + 64, N * rx + 24, M * oy + 16
    so, sl, sr = (1, oy, oz), (1, ly, lz), (rx, 1, rz)
    assert plan(B, M, K, N, so, sl, sr) == f"gemm_nt_mfma_dma_{tile}x64"
    gen = torch.Generator(device="cuda").manual_seed(B * M + N)
    lbuf = (torch.randint(-4, 5, (B * lz + 8,), generator=gen, device="cuda").float() / 64).half()
    rbuf = (torch.randint(-4, 5, (B * rz + 8,), generator=gen, device="cuda").float() / 64).half()
    obuf = torch.full((B * oz + 8,), 5.0, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16", obuf, lbuf, rbuf, B, M, K, N, so, sl, sr) == 0
    want = torch.full_like(obuf, 5.0)
    for b in range(B):
        a = torch.as_strided(lbuf, (M, K), (ly, 1), b * lz).double()
        w = torch.as_strided(rbuf, (N, K), (rx, 1), b * rz).double()
        torch.as_strided(want, (M, N), (oy, 1), b * oz).copy_((a @ w.t()).half())
    assert torch.equal(obuf.view(torch.int16), want.view(torch.int16))


def test_unsupported_layouts_fall_back_and_stay_correct():
    g = rng(550)
    B, M, K, N = 1, 40, 50, 30   # K % 8 != 0
    so, sl, sr = (1, N, 0), (1, K, 0), (K, 1, 0)
    assert plan(B, M, K, N, so, sl, sr) == "matmul_general"
    l, r = dyadic(g, M * K), dyadic(g, K * N)
    want = oracle_matmul(np.zeros(M * N, np.float16), l, r, B, M, K, N, so, sl, sr,
                         mode=oracle.FAITHFUL)
    o_t = to_dev(np.zeros(M * N, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr) == 0
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))
    # misaligned base pointer on an otherwise supported layout
    K = 64
    l, r = dyadic(g, M * K + 8), dyadic(g, K * N + 8)
    sl, sr = (1, K, 0), (K, 1, 0)
    want = oracle_matmul(np.zeros(M * N, np.float16), l, r, B, M, K, N, so, sl, sr,
                         mode=oracle.FAITHFUL, offsets=(0, 1, 3))
    o_t = to_dev(np.zeros(M * N, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, to_dev(l), to_dev(r), B, M, K, N, so, sl, sr,
                      offsets=(0, 1, 3)) == 0
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))


def test_matmul_nt_f16_entry_point():
    from adrastea_amd import GpuKernels
    g = rng(560)
    M, K, N = 48, 256, 200
    a, b, prev = dyadic(g, (M, K)), dyadic(g, (N, K)), randn_f16(g, (M, N))
    for beta in (0.0, 0.5):
        want = prev.copy()
        oracle.matmul_nt_f16(want, a, b, beta=beta)
        o_t = to_dev(prev)
        GpuKernels().matmul_nt_f16(o_t, to_dev(a), to_dev(b), beta=beta)
        assert np.max(ulp_diff_f16(to_np(o_t), want)) <= (0 if beta == 0.0 else 1)


@pytest.mark.parametrize("M,K,N,tile", [(2000, 2048, 8184, "256x128"), (630, 2048, 12280, "128x256"),
                                        (380, 2048, 12280, "128x192"), (2048, 1024, 12288, "256x192"),
                                        (2000, 2048, 8186, "256x128"), (1000, 2048, 4090, "128x128")])
@pytest.mark.parametrize("beta", [1.0, 0.5])
def test_fp32_epilogues_of_the_large_tiles(M, K, N, tile, beta):
    """out = acc + beta * out on the unrounded fp32 accumulator (adr_matmul_nt_f16 with beta != 0):
    the accumulators -- 16 x 16 blocks in the 256-row and 256-column tiles, 32 x 32 blocks in
    128 x 192 -- pass through LDS as fp32; with 16-byte aligned rows a lane then owns whole chunks
    whose previous values were requested up front (N = 8184, 12280: the last tile column runs past
    the matrix; M = 2000 ...: so does the last tile row), with unaligned rows (N = 8186, 4090) the
    elements are stored one by one.  Exact on inputs whose sums are exact (the sum of two exact
    terms rounded once)."""
    so, sl, sr = nt_strides(M, K, N)
    assert plan(1, M, K, N, so, sl, sr, store=0) == f"gemm_nt_mfma_dma_{tile}x64"
    gen = torch.Generator(device="cuda").manual_seed(M + N)
    a = (torch.randint(-4, 5, (M, K), generator=gen, device="cuda").float() / 64).half()
    w = (torch.randint(-4, 5, (N, K), generator=gen, device="cuda").float() / 64).half()
    prev = (torch.randint(-64, 65, (M, N), generator=gen, device="cuda").float() / 16).half()
    want = (a.double() @ w.double().t() + beta * prev.double()).half()
    out = prev.clone()
    stream = torch.cuda.current_stream().cuda_stream
    assert _ffi.lib().adr_matmul_nt_f16(stream, out.data_ptr(), a.data_ptr(), w.data_ptr(), M, K, N,
                                        beta) == 0
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    if N % 8 and beta == 1.0:
        # unaligned rows through the plain entry point too (Identity)
        out = torch.full((M, N), 9.0, dtype=torch.float16, device="cuda")
        assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr) == 0
        want = (a.double() @ w.double().t()).half()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))


# ------------------------------------------------------------------ host API and error behaviour

def test_gpukernels_interface_and_errors():
    from adrastea_amd import (GpuKernels, TensorView, MatmulOptions, MatmulStore, MatmulMask,
                              AdrasteaError, MatmulTracer)
    g = rng(570)
    S, D = 96, 64
    kern = MatmulTracer(GpuKernels())
    x, w = dyadic(g, (S, D)), dyadic(g, (D, D))
    x_t, w_t = to_dev(x), to_dev(w)
    out = torch.zeros(S, D, dtype=torch.float16, device="cuda")
    kern.matmul_f16(TensorView.of(out), TensorView.of(x_t), TensorView.of(w_t).permute([1, 0]),
                    MatmulOptions.new())
    want = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32).astype(np.float16)
    assert np.array_equal(to_np(out), want)
    assert len(kern.shapes) == 1
    with pytest.raises(AssertionError):   # K mismatch: the reference assert_eq!-panics
        kern.matmul_f16(TensorView.of(out), TensorView.of(x_t), TensorView.of(w_t[:, :32]),
                        MatmulOptions.new())
    bias = torch.zeros(D, dtype=torch.float16, device="cuda")
    with pytest.raises(AdrasteaError) as e:  # GeluBias: device NYI in the reference
        kern.matmul_f16(TensorView.of(out), TensorView.of(x_t), TensorView.of(w_t).permute([1, 0]),
                        MatmulOptions.new().store(MatmulStore.GeluBias(TensorView.of(bias))))
    assert e.value.code == -3
    with pytest.raises(AdrasteaError) as e:  # bias operator without a bias
        kern.matmul_f16(TensorView.of(out), TensorView.of(x_t), TensorView.of(w_t).permute([1, 0]),
                        MatmulOptions.new().store(MatmulStore.BetaBias(1.0, None)))
    assert e.value.code == -4
    o_t = to_dev(np.zeros(4, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, o_t, o_t, 1, 2, 2, 2, (1, 2, 0), (1, 2, 0), (1, 2, 0),
                      store=9) == -2
    assert raw_matmul("adr_matmul_f16", o_t, o_t, o_t, 1, -2, 2, 2, (1, 2, 0), (1, 2, 0),
                      (1, 2, 0)) == -1
    # empty problems are a no-op, k == 0 stores store(0)
    assert raw_matmul("adr_matmul_f16", o_t, o_t, o_t, 1, 0, 2, 2, (1, 2, 0), (1, 2, 0), (1, 2, 0)) == 0
    o_t = to_dev(np.full(4, 3.0, np.float16))
    assert raw_matmul("adr_matmul_f16", o_t, o_t, o_t, 1, 2, 0, 2, (1, 2, 0), (1, 2, 0), (1, 2, 0)) == 0
    assert np.all(to_np(o_t) == 0)


# ------------------------------------------------------------------ benchmark sizes: properties

FULL = [
    # name, B, M, K, N  (fp16 NT weights)
    ("clip_mlp_up", 1, 2056, 1024, 4096),
    ("clip_mlp_down", 1, 2056, 4096, 1024),
    ("llama_qkv", 1, 2048, 4096, 12288),
    ("llama_o", 1, 2048, 4096, 4096),
    ("llama_gate", 1, 2048, 4096, 11008),
    ("llama_down", 1, 2048, 11008, 4096),
    ("llama_qkv_2056_rows", 1, 2056, 4096, 12288),  # issued as 2048 rows + 8 rows
]


@pytest.mark.parametrize("workspace_mode", ["pool_off", "shipped_default"], indirect=True)
@pytest.mark.parametrize("case", FULL, ids=[c[0] for c in FULL])
def test_full_size_gemm_against_fp32_gemm_and_slow_kernel(case, workspace_mode):
    """At benchmark sizes: max relative error <= 1e-2 against an fp32 GEMM of the same fp16
    inputs (torch, on the device, as the independent fp32 reference), and agreement with the
    step-for-step slow kernel on a band of rows.  Once with the library's workspace pool off and
    once exactly as a drop-in caller (and bench.py) finds the library."""
    _, B, M, K, N = case
    gen = torch.Generator(device="cuda").manual_seed(42)
    a = torch.randn(M, K, generator=gen, device="cuda").half()
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    out = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    so, sl, sr = nt_strides(M, K, N)
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr) == 0
    ref32 = a.float() @ w.float().t()
    rms = ref32.pow(2).mean().sqrt()
    rel = ((out.float() - ref32).abs() / torch.maximum(ref32.abs(), rms)).max().item()
    assert rel <= TOL, rel
    # the plain ratio |got - ref| / |ref| wherever the reference is at least of typical size
    big = ref32.abs() >= rms
    assert ((out.float() - ref32).abs()[big] / ref32.abs()[big]).max().item() <= TOL
    rows = 64
    slow = torch.zeros(rows, N, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16_slow", slow, a[M - rows:], w, 1, rows, K, N, so, sl, sr) == 0
    rel = ((out[M - rows:].float() - slow.float()).abs() /
           torch.maximum(slow.float().abs(), rms)).max().item()
    assert rel <= TOL, rel


@pytest.mark.parametrize("K", [320, 384, 448, 512, 576, 640])
def test_large_tile_kernel_every_k_tail_exact(K):
    """The 256 x 192 kernel rotates two left and four right LDS stages with a period of four
    slices, half of its wavefronts issuing the left and half the right operand's transfers:
    every remainder of that loop, on inputs whose fp32 sums are exact, must give the correctly
    rounded product bit for bit (ragged last tile row and column included)."""
    M, N = 2000, 12200
    so, sl, sr = nt_strides(M, K, N)
    assert plan(1, M, K, N, so, sl, sr) == "gemm_nt_mfma_dma_256x192x64"
    gen = torch.Generator(device="cuda").manual_seed(K)
    a = (torch.randint(-8, 9, (M, K), generator=gen, device="cuda").float() / 64).half()
    w = (torch.randint(-8, 9, (N, K), generator=gen, device="cuda").float() / 64).half()
    out = torch.full((M, N), 9.0, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr) == 0
    want = (a.double() @ w.double().t()).half()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


# (M, N, the tile the choice model gives the shape at K >= 2048)
TILE_SHAPES = [(2000, 8184, "256x128"), (630, 12280, "128x256"), (380, 12280, "128x192"),
               (2000, 5112, "256x160")]


@pytest.mark.parametrize("K", [2048, 2112, 2176, 2240, 2304, 2368])
@pytest.mark.parametrize("M,N,tile", TILE_SHAPES)
def test_large_tiles_every_k_tail_exact(K, M, N, tile):
    """The 256 x 128, 128 x 256 and 256 x 160 kernels (16x16x32 MFMAs; the last with sub-tiles five
    16-column blocks wide) and the 128 x 192 kernel (32x32x16): six consecutive K tails (every remainder of the three-slice loop of the three-stage tiles)
    on inputs whose fp32 sums are exact, ragged last tile row and column."""
    so, sl, sr = nt_strides(M, K, N)
    assert plan(1, M, K, N, so, sl, sr) == f"gemm_nt_mfma_dma_{tile}x64"
    gen = torch.Generator(device="cuda").manual_seed(K)
    a = (torch.randint(-4, 5, (M, K), generator=gen, device="cuda").float() / 64).half()
    w = (torch.randint(-4, 5, (N, K), generator=gen, device="cuda").float() / 64).half()
    out = torch.full((M, N), 9.0, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr) == 0
    want = (a.double() @ w.double().t()).half()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("K", [1536 + 64 * i for i in range(12)])
def test_256x128_tile_every_remainder_of_its_twelve_slice_period(K):
    """The 256 x 128 kernel rotates three left and four right LDS stages (period twelve slices), half
    of its wavefronts issuing the left and half the right operand's transfers: every remainder of
    that loop on inputs whose fp32 sums are exact, ragged last tile row and column."""
    M, N = 2000, 8184
    so, sl, sr = nt_strides(M, K, N)
    assert plan(1, M, K, N, so, sl, sr) == "gemm_nt_mfma_dma_256x128x64"
    gen = torch.Generator(device="cuda").manual_seed(K)
    a = (torch.randint(-4, 5, (M, K), generator=gen, device="cuda").float() / 64).half()
    w = (torch.randint(-4, 5, (N, K), generator=gen, device="cuda").float() / 64).half()
    out = torch.full((M, N), 9.0, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr) == 0
    want = (a.double() @ w.double().t()).half()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("K", [320 + 64 * i for i in range(14)])
def test_128x128_tile_every_remainder_of_its_twelve_slice_period(K):
    """The 128 x 128 kernel (eight wavefronts of 32 x 64 on 16x16x32 MFMAs) rotates three left and four
    right LDS stages like the 256 x 128 one: K of 5 to 18 slices, i.e. fewer slices than the period,
    every remainder of it and one full turn, on inputs whose fp32 sums are exact, ragged last tile
    row and column."""
    M, N = 1000, 3064
    so, sl, sr = nt_strides(M, K, N)
    assert plan(1, M, K, N, so, sl, sr) == "gemm_nt_mfma_dma_128x128x64"
    gen = torch.Generator(device="cuda").manual_seed(K)
    a = (torch.randint(-4, 5, (M, K), generator=gen, device="cuda").float() / 64).half()
    w = (torch.randint(-4, 5, (N, K), generator=gen, device="cuda").float() / 64).half()
    out = torch.full((M, N), 9.0, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr) == 0
    want = (a.double() @ w.double().t()).half()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("store", STORES_EXACT + STORES_F32)
@pytest.mark.parametrize("mask", [oracle.MASK_NONE, oracle.MASK_CAUSAL])
@pytest.mark.parametrize("M,N,tile", [(4000, 4088, "256x128"), (630, 12280, "128x256"), (380, 12280, "128x192"),
                                      (2000, 5112, "256x160")])
def test_large_tile_epilogues_against_the_slow_kernel(store, mask, M, N, tile):
    """Every store operator and the causal mask through the epilogues of the 256 x 128 and
    128 x 256 tiles (accumulators in 16 x 16 blocks, the latter's staging slots in the right
    operand's LDS stages) and of the 128 x 192 tile, compared with the step-for-step kernel on
    bands of rows (first tile row, a diagonal tile, the ragged last rows)."""
    K = 2048
    so, sl, sr = nt_strides(M, K, N)
    assert plan(1, M, K, N, so, sl, sr, store=store, mask=mask) == f"gemm_nt_mfma_dma_{tile}x64"
    gen = torch.Generator(device="cuda").manual_seed(900 + store * 2 + mask)
    a = torch.randn(M, K, generator=gen, device="cuda").half()
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    prev = torch.randn(M, N, generator=gen, device="cuda").half()
    bias = torch.randn(N, generator=gen, device="cuda").half()
    kw = dict(bias_t=bias, beta=0.7, scale=0.2, store=store, mask=mask)
    out = prev.clone()
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr, **kw) == 0
    for r0, rows in ((0, 40), (M * 3 // 8, 72), (M - 30, 30)):
        # the causal mask compares absolute row numbers: run the band as a product of its own
        # with the columns it may see shifted accordingly (a band of the full problem on the
        # slow kernel = rows r0.. of a, previous output rows r0..)
        slow = prev[r0:r0 + rows].clone()
        if mask == oracle.MASK_CAUSAL:
            # rows 0..r0+rows of the product, keep the band
            full = prev[:r0 + rows].clone()
            assert raw_matmul("adr_matmul_f16_slow", full, a[:r0 + rows], w, 1, r0 + rows, K, N, so, sl, sr,
                              **kw) == 0
            slow = full[r0:]
        else:
            assert raw_matmul("adr_matmul_f16_slow", slow, a[r0:r0 + rows], w, 1, rows, K, N, so, sl, sr,
                              **kw) == 0
        got = out[r0:r0 + rows]
        inf = torch.isinf(slow)
        assert torch.equal(torch.isinf(got), inf)
        fin = ~inf
        scale = slow[fin].float().pow(2).mean().sqrt()
        err = (got[fin].float() - slow[fin].float()).abs() / torch.maximum(slow[fin].float().abs(), scale)
        assert err.max().item() <= TOL, (store, mask, r0)


def test_row_tail_split_keeps_operator_semantics():
    """A product a few rows past a multiple of 128 goes out as two launches (2048 + 8 rows here);
    the second one must see its own rows of the previous output and the shared bias."""
    M, K, N = 2056, 4096, 12288
    so, sl, sr = nt_strides(M, K, N)
    gen = torch.Generator(device="cuda").manual_seed(7)
    a = torch.randn(M, K, generator=gen, device="cuda").half()
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    prev = torch.randn(M, N, generator=gen, device="cuda").half()
    bias = torch.randn(N, generator=gen, device="cuda").half()
    out = prev.clone()
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr, bias_t=bias, beta=0.5,
                      store=oracle.STORE_BETA_BIAS) == 0
    acc16 = (a.float() @ w.float().t()).half().float()
    want = acc16 + bias.float()[None, :] + 0.5 * prev.float()
    rms = want.pow(2).mean().sqrt()
    rel = ((out.float() - want).abs() / torch.maximum(want.abs(), rms)).max().item()
    assert rel <= TOL, rel
    # the eight tail rows against the step-for-step kernel on the same rows
    slow = prev[M - 8:].clone()
    assert raw_matmul("adr_matmul_f16_slow", slow, a[M - 8:], w, 1, 8, K, N, so, sl, sr,
                      bias_t=bias, beta=0.5, store=oracle.STORE_BETA_BIAS) == 0
    rel = ((out[M - 8:].float() - slow.float()).abs() /
           torch.maximum(slow.float().abs(), rms)).max().item()
    assert rel <= TOL, rel


@pytest.mark.parametrize("shape", [(70, 1024, 4100, "64x64"), (200, 4096, 4096, "64x64"),
                                   (64, 1152, 12288, "64x64"), (256, 11008, 4096, "64x64"),
                                   (120, 1024, 12200, "128x64"), (500, 11008, 4096, "128x64")])
def test_few_row_products_with_slices_of_128(shape):
    """At most one 64 x 64 (or 128 x 64) tile per CU and K % 128 == 0: the kernel with K slices
    of 128; exact on inputs whose sums are exact, ragged edges included."""
    M, K, N, tile = shape
    so, sl, sr = nt_strides(M, K, N)
    assert plan(1, M, K, N, so, sl, sr) == f"gemm_nt_mfma_dma_{tile}x128"
    gen = torch.Generator(device="cuda").manual_seed(M + K)
    a = (torch.randint(-8, 9, (M, K), generator=gen, device="cuda").float() / 64).half()
    w = (torch.randint(-8, 9, (N, K), generator=gen, device="cuda").float() / 64).half()
    out = torch.full((M, N), 9.0, dtype=torch.float16, device="cuda")
    assert raw_matmul("adr_matmul_f16", out, a, w, 1, M, K, N, so, sl, sr) == 0
    want = (a.double() @ w.double().t()).half()
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))


def test_full_size_attention_products():
    """benchmark config 4: 32 heads, head_dim 128, seq 2048.  QK^T scaled by 1/sqrt(128) with the
    causal mask; P.V with softmaxed scores.  Checked per head against an fp32 batched GEMM."""
    S, H, D = 2048, 32, 128
    HD = H * D
    gen = torch.Generator(device="cuda").manual_seed(43)
    q, k, v = (torch.randn(S, HD, generator=gen, device="cuda").half() for _ in range(3))
    qk = torch.zeros(H, S, S, dtype=torch.float16, device="cuda")
    so, sl, sr = (1, S, S * S), (1, HD, D), (HD, 1, D)
    scale = 1.0 / np.sqrt(D)
    assert raw_matmul("adr_matmul_f16", qk, q, k, H, S, D, S, so, sl, sr,
                      store=oracle.STORE_SCALE, scale=scale, mask=oracle.MASK_CAUSAL) == 0
    q3, k3, v3 = (t.view(S, H, D).permute(1, 0, 2).float() for t in (q, k, v))
    s16 = float(np.float16(np.float32(scale)))
    ref = torch.bmm(q3, k3.transpose(1, 2)) * s16
    tri = torch.ones(S, S, dtype=torch.bool, device="cuda").triu(1)
    assert torch.all(qk[:, tri].view(torch.int16) == -1024)  # 0xFC00
    keep = ~tri
    rms = ref[:, keep].pow(2).mean().sqrt()
    rel = ((qk.float() - ref).abs() / torch.maximum(ref.abs(), rms))[:, keep].max().item()
    assert rel <= TOL, rel
    p = torch.softmax(torch.where(tri, float("-inf"), qk.float()), dim=-1).half()
    o = torch.zeros(S, HD, dtype=torch.float16, device="cuda")
    so, sl, sr = (1, HD, D), (1, S, S * S), (1, HD, D)
    assert raw_matmul("adr_matmul_f16", o, p, v, H, S, S, D, so, sl, sr) == 0
    ref = torch.bmm(p.float(), v3).permute(1, 0, 2).reshape(S, HD)
    rms = ref.pow(2).mean().sqrt()
    rel = ((o.float() - ref).abs() / torch.maximum(ref.abs(), rms)).max().item()
    assert rel <= TOL, rel


def test_matmul_f16_raw_entry_point():
    """matmul_f16_raw (matmul.cu:515-517): the 16 common arguments, identity operators."""
    from adrastea_amd import _ffi
    g = rng(580)
    B, M, K, N = 2, 40, 64, 56
    l, r = dyadic(g, B * M * K), dyadic(g, B * K * N)
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, K * N)
    want = oracle_matmul(np.zeros(B * M * N, np.float16), l, r, B, M, K, N, so, sl, sr)
    o_t, l_t, r_t = to_dev(np.zeros(B * M * N, np.float16)), to_dev(l), to_dev(r)
    rc = _ffi.lib().adr_matmul_f16_raw(torch.cuda.current_stream().cuda_stream, o_t.data_ptr(),
                                       l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, *so, *sl, *sr)
    assert rc == 0
    assert np.array_equal(to_np(o_t).view(np.uint16), want.view(np.uint16))
