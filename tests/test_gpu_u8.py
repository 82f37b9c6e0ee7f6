"""GPU parity of the u8 absmax format kernels and the u8-weight GEMV / GEMM (through the C ABI).

Bars: the dequantised weight values are bit-exact against the oracle for EVERY (q, scale)
pair, both in the stand-alone dequantise kernel and inside the fused matmul kernels (extracted
with one-hot activations); quantise is bit-exact; matmul outputs are bit-exact where the sums
are exactly representable and within max relative error 1e-2 of an fp32/fp64 GEMM otherwise.
"""
import numpy as np
import pytest
import torch

import oracle
from helpers import rng, randn_f16, ulp_diff_f16, max_rel_err
from gpu_common import to_dev, to_np, nan_canon
from adrastea_amd import GpuKernels, _ffi

pytestmark = pytest.mark.gpu
TOL = 1e-2


@pytest.fixture(scope="module")
def kern():
    return GpuKernels()


@pytest.fixture(scope="module")
def ref():
    import refgpu
    if not refgpu.available():
        pytest.skip("oracle/_ref code objects not built")
    return refgpu.RefKernels()


def u8_plan(m, p, n, bs):
    import ctypes as C
    buf = C.create_string_buffer(64)
    assert _ffi.lib().adr_matmul_nt_fp16u8_plan(buf, 64, m, p, n, bs) == 0
    return buf.value.decode()


def test_dequantize_every_q_and_scale_bit_pattern(kern):
    """rows = all 65536 fp16 scale patterns, cols = all 256 quantised values."""
    q = np.tile(np.arange(256, dtype=np.uint8), (65536, 1))
    s = np.arange(65536, dtype=np.uint16).view(np.float16).reshape(65536, 1)
    out = torch.zeros(65536, 256, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(out, to_dev(s), to_dev(q))
    got = nan_canon(to_np(out).view(np.uint16))
    want = nan_canon(oracle.dequant_table().T.copy())
    assert np.array_equal(got, want)


def test_dequantize_matches_reference_kernel(kern, ref):
    g = rng(600)
    rows, cols, bs = 64, 512, 32
    q = g.integers(0, 256, size=(rows, cols), dtype=np.uint16).astype(np.uint8)
    s = g.integers(0, 0x7C00, size=(rows, cols // bs), dtype=np.uint32).astype(np.uint16).view(np.float16)
    q_t, s_t = to_dev(q), to_dev(s)
    o_ref = torch.zeros(rows, cols, dtype=torch.float16, device="cuda")
    ref.dequantize(o_ref, s_t, q_t)
    torch.cuda.synchronize()
    out = torch.zeros(rows, cols, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(out, s_t, q_t)
    assert np.array_equal(to_np(out).view(np.uint16), to_np(o_ref).view(np.uint16))
    assert np.array_equal(to_np(o_ref).view(np.uint16),
                          oracle.dequantize_absmax_u8(q, s, bs).view(np.uint16))


def test_quantize_matches_oracle_and_reference_kernel(kern, ref):
    g = rng(601)
    rows, cols, bs = 48, 384, 32
    x = randn_f16(g, (rows, cols), 0.05)
    x[0, :32] = 0.25           # all-equal block
    x[1, :32] = 0
    x[1, 7] = -3.0             # single negative spike
    x[2, :64] = np.float16(6.1e-5)  # smallest normal: subnormal scale
    q_want, s_want = oracle.quantize_absmax_u8(x, bs)
    x_t = to_dev(x)
    q_t = torch.zeros(rows, cols, dtype=torch.uint8, device="cuda")
    s_t = torch.zeros(rows, cols // bs, dtype=torch.float16, device="cuda")
    kern.quantize_absmax_uint8(q_t, s_t, x_t)
    assert np.array_equal(to_np(s_t).view(np.uint16), s_want.view(np.uint16))
    assert np.array_equal(to_np(q_t), q_want)
    q_r = torch.zeros_like(q_t)
    s_r = torch.zeros_like(s_t)
    ref.quantize(q_r, s_r, x_t)
    torch.cuda.synchronize()
    assert np.array_equal(to_np(s_r).view(np.uint16), s_want.view(np.uint16))
    assert np.array_equal(to_np(q_r), q_want)


@pytest.mark.parametrize("bs", [8, 16, 24, 32, 64, 96, 256, 512, 1024])
def test_quantize_block_sizes_vector_and_scalar_paths(kern, bs):
    """Block sizes 8 * 2^k <= 512 take the vectorised kernel, the others the one-wavefront-per-
    block kernel; both must agree with the oracle bit for bit, including all-zero blocks (scale 0:
    the value/0 quotients are NaN or infinite and map to 0 or saturate), and a ragged column
    count (cols not a multiple of the 2048 columns a workgroup covers)."""
    g = rng(670 + bs)
    rows, cols = 37, bs * 9
    x = randn_f16(g, (rows, cols), 0.3)
    x[3, :bs] = 0                      # all-zero block
    x[4, bs:2 * bs] = np.float16(65504.0)
    x[5, 0] = np.float16(-65504.0)
    q_want, s_want = oracle.quantize_absmax_u8(x, bs)
    q_t = torch.zeros(rows, cols, dtype=torch.uint8, device="cuda")
    s_t = torch.zeros(rows, cols // bs, dtype=torch.float16, device="cuda")
    kern.quantize_absmax_uint8(q_t, s_t, to_dev(x))
    assert np.array_equal(to_np(s_t).view(np.uint16), s_want.view(np.uint16))
    assert np.array_equal(to_np(q_t), q_want)


def _finite_scale_rows():
    # scale patterns whose 256 dequantised values are all finite (|s| <= 512): an infinite
    # weight times a zero activation would poison the row's sums.  Larger scales, inf and NaN
    # are covered by the stand-alone dequantise test above.
    s = np.arange(65536, dtype=np.uint16)
    return s[(s & 0x7FFF) <= 0x6000]


@pytest.mark.parametrize("m", [1, 4, 16])
@pytest.mark.parametrize("every", [1, 8], ids=["all_scales", "every_8th_scale"])
def test_fused_dequant_in_gemv_is_bit_exact_for_every_q_and_finite_scale(kern, m, every):
    """One-hot activations pick single weights out of the matmul: out[r, c] = w[c, k_r].
    All finite scales make a wide matrix (48-row workgroups), every 8th a narrower one (32)."""
    scales_bits = _finite_scale_rows()[::every]
    n, p, bs = scales_bits.size, 256, 32
    assert u8_plan(m, p, n, bs) == ("gemv_u8_dot2_stream" if m <= 2 else "gemv_u8_mfma16_regstream")
    q = np.tile(np.arange(256, dtype=np.uint8), (n, 1))
    s = np.repeat(scales_bits.view(np.float16).reshape(n, 1), p // bs, axis=1)
    table = oracle.dequant_table()  # [q][scale bits]
    q_t, s_t = to_dev(q), to_dev(s)
    for base in range(0, 256, m):
        ks = np.arange(base, base + m)
        lhs = np.zeros((m, p), np.float16)
        lhs[np.arange(m), ks] = 1.0
        out = torch.zeros(m, n, dtype=torch.float16, device="cuda")
        kern.matmul_nt_fp16u8(out, to_dev(lhs), q_t, s_t, bs)
        got = to_np(out).view(np.uint16)
        want = table[ks][:, scales_bits]
        # -0.0 + 0.0 products: a dequantised -0 sums to +0; compare values for zeros
        z = (want & 0x7FFF) == 0
        assert np.array_equal(got[~z], want[~z]), base
        assert np.all((got[z] & 0x7FFF) == 0)


# the tiles of the u8 kernel in the order of adr_debug_knob(1, 1 + i); "_k2" / "_k4": K split over
# two / four groups of wavefronts inside the workgroup
U8_TILES = ["256x192x64", "256x128x64", "128x128x64", "128x64x64", "64x64x64", "128x64x64_k2", "64x64x64_k4"]
U8_STAGED = len(U8_TILES) + 1   # knob value: the register-staged kernels


@pytest.fixture
def force_u8_tile():
    """force_u8_tile(name) makes the tiled u8 kernel run that tile until the test ends."""
    lib = _ffi.lib()

    def force(tile):
        assert lib.adr_debug_knob(1, U8_STAGED if tile == "staged" else U8_STAGED + 1 if tile == "passes" else
                                  1 + U8_TILES.index(tile)) == 0
    yield force
    assert lib.adr_debug_knob(1, 0) == 0


@pytest.mark.parametrize("tile", ["256x128x64", "256x192x64", "128x128x64", "128x64x64", "64x64x64", "128x64x64_k2",
                                  "64x64x64_k4"])
def test_fused_dequant_in_u8_gemm_is_bit_exact_for_every_q_and_finite_scale(kern, tile, force_u8_tile):
    """One-hot rows extract every weight of the tiled u8 kernel: all 49154 finite scales make 385
    tiles of 256 x 128; the first 49152 of them exactly 256 tiles of 256 x 192 (the two scales
    left out are covered by the other tile and by the stand-alone kernel).  The smaller tiles are
    forced on the same product."""
    scales_bits = _finite_scale_rows()
    if tile == "256x192x64":
        scales_bits = scales_bits[:192 * 256]
    n, p, bs, m = scales_bits.size, 256, 32, 256
    if tile in ("256x128x64", "256x192x64"):
        assert u8_plan(m, p, n, bs) == f"gemm_nt_u8_mfma_{tile}"   # what the dispatch runs here
    force_u8_tile(tile)
    assert u8_plan(m, p, n, bs) == f"gemm_nt_u8_mfma_{tile}"
    q = np.tile(np.arange(256, dtype=np.uint8), (n, 1))
    s = np.repeat(scales_bits.view(np.float16).reshape(n, 1), p // bs, axis=1)
    lhs = np.eye(m, dtype=np.float16)
    out = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    kern.matmul_nt_fp16u8(out, to_dev(lhs), to_dev(q), to_dev(s), bs)
    got = to_np(out).view(np.uint16)
    want = oracle.dequant_table()[:, scales_bits]
    z = (want & 0x7FFF) == 0
    assert np.array_equal(got[~z], want[~z])
    assert np.all((got[z] & 0x7FFF) == 0)


def _u8_case(g, m, p, n, bs, exact):
    q = g.integers(0, 256, size=(n, p), dtype=np.uint16).astype(np.uint8)
    if exact:
        # power-of-two scales and small dyadic activations: every product and sum is exact
        s = np.exp2(g.integers(-8, -4, size=(n, p // bs))).astype(np.float16)
        a = (g.integers(-8, 9, size=(m, p)) / 8.0).astype(np.float16)
    else:
        s = g.uniform(0.001, 0.02, size=(n, p // bs)).astype(np.float16)
        a = randn_f16(g, (m, p))
    return a, q, s


@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 7, 8, 9, 12, 13, 16])
@pytest.mark.parametrize("pn", [(256, 16), (512, 100), (1024, 33), (2816, 48), (4096, 52),
                                (5120, 40), (11008, 24),
                                # five to eight segments of 1 KiB (one per wavefront for one row), whole and ragged
                                (6656, 24), (8192, 20), (4128, 30), (7200, 18)])
def test_gemv_bit_exact_on_exact_inputs(kern, m, pn):
    p, n = pn
    g = rng(610 + m + n)
    a, q, s = _u8_case(g, m, p, n, 32, exact=True)
    prev = (g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)
    for beta in (0.0, 0.5):
        want = prev.copy()
        oracle.matmul_nt_fp16u8(want, a, q, s, 32, beta=beta)
        out = to_dev(prev)
        kern.matmul_nt_fp16u8(out, to_dev(a), to_dev(q), to_dev(s), 32, beta=beta)
        assert np.array_equal(to_np(out).view(np.uint16), want.view(np.uint16)), (m, p, n, beta)


@pytest.mark.parametrize("m", [3, 16])
def test_wide_dma_gemv_bit_exact_on_exact_inputs(kern, m):
    """K = 4096 on a wide matrix (48 rows per workgroup, two macro steps per wavefront); ragged
    last workgroup (12251 = 255 * 48 + 11 rows), beta path."""
    p, n = 4096, 12251
    g = rng(990 + m)
    assert u8_plan(m, p, n, 32) == "gemv_u8_mfma16_regstream"
    a, q, s = _u8_case(g, m, p, n, 32, exact=True)
    for beta in (0.0, 1.0):
        prev = (g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)
        want = prev.copy()
        oracle.matmul_nt_fp16u8(want, a, q, s, 32, beta=beta, threads=8)
        out = to_dev(prev)
        kern.matmul_nt_fp16u8(out, to_dev(a), to_dev(q), to_dev(s), 32, beta=beta)
        assert np.array_equal(to_np(out).view(np.uint16), want.view(np.uint16)), (m, beta)


@pytest.mark.parametrize("m", [3, 7, 16])
@pytest.mark.parametrize("pn", [(256, 8192), (768, 8200), (1024, 8251)])
def test_wide_gemv_bit_exact_on_exact_inputs(kern, m, pn):
    """32 rows per workgroup (n around 8192) with one to four macro steps, i.e. wavefronts
    without any step of their own: ragged last workgroup, beta path."""
    p, n = pn
    g = rng(660 + m + p)
    assert u8_plan(m, p, n, 32) == "gemv_u8_mfma16_regstream"
    a, q, s = _u8_case(g, m, p, n, 32, exact=True)
    for beta in (0.0, 1.0):
        prev = (g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)
        want = prev.copy()
        oracle.matmul_nt_fp16u8(want, a, q, s, 32, beta=beta, threads=8)
        out = to_dev(prev)
        kern.matmul_nt_fp16u8(out, to_dev(a), to_dev(q), to_dev(s), 32, beta=beta)
        assert np.array_equal(to_np(out).view(np.uint16), want.view(np.uint16)), (m, p, n, beta)


@pytest.mark.parametrize("m", [17, 31, 32, 33, 48, 50, 64, 70])
@pytest.mark.parametrize("pn", [(256, 16400), (768, 8200), (2304, 1900), (11008, 400), (4096, 1030)])
def test_blocks_kernel_bit_exact_on_exact_inputs(kern, m, pn, force_u8_tile):
    """Two to four blocks of sixteen activation rows per workgroup: one, two and three groups of
    weight rows, macro-step counts from one (wavefronts without a step) to 43, ragged rows of
    both operands, a second pass for rows 65 .. 70, beta path.  The passes are forced: from 33 rows
    on the dispatch sends wide matrices and short K to the tiled kernel."""
    p, n = pn
    g = rng(1700 + m + p)
    if m <= 32 or (n <= 1900 and (m <= 64 or p >= 4096)):   # what the dispatch runs in passes by itself
        assert u8_plan(m, p, n, 32) in ("gemv_u8_mfma16_blocks", "gemv_u8_mfma16_dma_32rows")
    force_u8_tile("passes")
    assert u8_plan(m, p, n, 32) in ("gemv_u8_mfma16_blocks", "gemv_u8_mfma16_dma_32rows")
    a, q, s = _u8_case(g, m, p, n, 32, exact=True)
    for beta in (0.0, 1.0):
        prev = (g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)
        want = prev.copy()
        oracle.matmul_nt_fp16u8(want, a, q, s, 32, beta=beta, threads=8)
        out = to_dev(prev)
        kern.matmul_nt_fp16u8(out, to_dev(a), to_dev(q), to_dev(s), 32, beta=beta)
        assert np.array_equal(to_np(out).view(np.uint16), want.view(np.uint16)), (m, p, n, beta)


@pytest.mark.parametrize("m", [1, 4, 16, 17, 100, 300])
def test_u8_matmul_random_matches_oracle_and_reference_kernel(kern, ref, m):
    g = rng(620 + m)
    p, n, bs = 512, 200, 32
    a, q, s = _u8_case(g, m, p, n, bs, exact=False)
    want = np.zeros((m, n), np.float16)
    oracle.matmul_nt_fp16u8(want, a, q, s, bs, threads=8)
    out = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    a_t, q_t, s_t = to_dev(a), to_dev(q), to_dev(s)
    kern.matmul_nt_fp16u8(out, a_t, q_t, s_t, bs)
    got = to_np(out)
    w = oracle.dequantize_absmax_u8(q, s, bs).astype(np.float64)
    ref64 = a.astype(np.float64) @ w.T
    assert max_rel_err(got, ref64) <= 2e-3
    assert np.max(ulp_diff_f16(got, want)) <= 1 or max_rel_err(got, want.astype(np.float64)) <= 2e-3
    # the reference's naive u8 kernel (double-precision product, unrounded weights)
    o_ref = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    ref.matmul_nt_fp16u8(o_ref, a_t, q_t, s_t, bs)
    torch.cuda.synchronize()
    assert max_rel_err(got, to_np(o_ref).astype(np.float64)) <= TOL
    naive = np.zeros((m, n), np.float16)
    oracle.matmul_nt_fp16u8(naive, a, q, s, bs, naive=True, threads=8)
    assert np.max(ulp_diff_f16(naive, to_np(o_ref))) <= 1


@pytest.mark.parametrize("case", [(300, 64, 1000, 32), (257, 128, 1030, 8), (512, 192, 520, 16),
                                  (260, 320, 1100, 64), (1024, 384, 300, 128), (1024, 448, 300, 64), (256, 832, 1024, 32),
                                  (700, 768, 400, 256)],
                         ids=lambda c: "M%d_K%d_N%d_bs%d" % c)
@pytest.mark.parametrize("route", ["staged", "dispatch"])
def test_u8_small_products_ragged_tiles_and_k_tails_bit_exact(kern, case, route, force_u8_tile):
    """Small u8 products on the register-staged kernels (dequantised while staging; what a K
    that is no multiple of 64 runs on, forced here) and on the tile the dispatch picks for them
    (the small tiles of the DMA kernel): partial tiles in M and N, K of one to thirteen slices,
    block sizes below, at and above the slice depth, and the beta path -- exact inputs, compared
    bit for bit.  (Every tile of the DMA kernel: test_u8_dma_kernel_* below.)"""
    m, p, n, bs = case
    if route == "staged":
        force_u8_tile("staged")
        assert u8_plan(m, p, n, bs).startswith("gemm_nt_u8_stage_")
    else:
        assert u8_plan(m, p, n, bs).startswith("gemm_nt_u8_mfma_")
    g = rng(640 + m + p)
    a, q, s = _u8_case(g, m, p, n, bs, exact=True)
    for beta in (0.0, 1.0):
        prev = (g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)
        want = prev.copy()
        oracle.matmul_nt_fp16u8(want, a, q, s, bs, beta=beta, threads=8)
        out = to_dev(prev)
        kern.matmul_nt_fp16u8(out, to_dev(a), to_dev(q), to_dev(s), bs, beta=beta)
        assert np.array_equal(to_np(out).view(np.uint16), want.view(np.uint16)), (case, beta)


_DMA_TILE_CASES = [("256x192x64", 520, 11000), ("256x128x64", 520, 2900), ("128x128x64", 520, 2900),
                   ("128x64x64", 520, 1900), ("64x64x64", 200, 1900), ("128x64x64_k2", 520, 1900),
                   ("64x64x64_k4", 200, 1900)]
# (K, tile): every tile on K of 5 .. 16 slices; the tiles that split K also on 20 .. 40
_DMA_TILE_K = [(t, p) for t in _DMA_TILE_CASES
               for p in [320, 384, 448, 512, 576, 640, 704, 768, 832, 896, 960, 1024] +
               ([1280, 1536, 1792, 2048, 2304, 2560] if t[0].endswith(("_k2", "_k4")) else [])]


@pytest.mark.parametrize("tile_mn,p", _DMA_TILE_K, ids=[f"{t[0]}-K{p}" for t, p in _DMA_TILE_K])
def test_u8_dma_kernel_ragged_tiles_and_every_k_remainder_bit_exact(kern, tile_mn, p, force_u8_tile):
    """Every tile of gemm_nt_u8_kernel, forced: a ragged last tile row (520 = 2 x 256 + 8,
    200 = 3 x 64 + 8) and tile column, K / 64 = 5 .. 16 slices and 20 .. 40 in steps of four, i.e.
    every remainder of the six-slice loop (twelve for the 256 x 128 tile with its four stages of the
    left operand), fewer slices than a period, and the same for the tiles that split K over two or
    four groups of wavefronts (which walk K / 128 or K / 256 steps; a K they do not divide runs
    the tile without groups), beta 0 and 1, block sizes 32 and 64 -- exact inputs, compared bit
    for bit.  Expected values: one rounding of the float64 product on the oracle's dequantised
    weights (every sum is exactly representable), cross-checked with the oracle's own matmul on
    the rows around the tile borders."""
    tile, m, n = tile_mn
    bs = 64 if p % 128 == 0 else 32
    force_u8_tile(tile)
    groups = 4 if tile.endswith("_k4") else 2 if tile.endswith("_k2") else 1
    assert u8_plan(m, p, n, bs) == "gemm_nt_u8_mfma_" + (tile if p % (64 * groups) == 0 else tile[:-3])
    g = rng(1640 + p + n)
    a, q, s = _u8_case(g, m, p, n, bs, exact=True)
    w64 = oracle.dequantize_absmax_u8(q, s, bs).astype(np.float64)
    prod = a.astype(np.float64) @ w64.T
    rows = np.array([r for r in (0, 1, 31, 32, 63, 64, 127, 128, 199, 255, 256, 257, 511, 512, 519) if r < m])
    a_t, q_t, s_t = to_dev(a), to_dev(q), to_dev(s)
    for beta in (0.0, 1.0):
        prev = (g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)
        want = (prod + beta * prev.astype(np.float64)).astype(np.float16)
        chk = prev[rows].copy()
        oracle.matmul_nt_fp16u8(chk, a[rows], q, s, bs, beta=beta, threads=8)
        assert np.array_equal(chk.view(np.uint16), want[rows].view(np.uint16))
        out = to_dev(prev)
        kern.matmul_nt_fp16u8(out, a_t, q_t, s_t, bs, beta=beta)
        got = to_np(out)
        bad = np.argwhere(got.view(np.uint16) != want.view(np.uint16))
        assert bad.size == 0, (tile, p, beta, bad[:5])


CFG5_U8 = [("qkv", 4096, 12288, "256x192"), ("o", 4096, 4096, "256x128"),
           ("gate_up", 4096, 11008, "256x192"), ("down", 11008, 4096, "256x128")]


@pytest.mark.parametrize("workspace_mode", ["pool_off", "shipped_default", "u8_dequantise_first"], indirect=True)
@pytest.mark.parametrize("case", CFG5_U8, ids=[c[0] for c in CFG5_U8])
def test_prefill_u8_gemm_layer_set_full_size(kern, case, workspace_mode):
    """benchmark config 5 (u8 half) at full size, M = 2048: every product of the layer set on the
    tile the benchmark measures (asserted through the plan), against an fp32 GEMM on the
    bit-exactly dequantised weights, both on the device; plus f(2a) = 2 f(a) exactly.  With the
    workspace pool off, as the library ships (the fused kernel either way), and on the route that
    adr_set_u8_dequantise_first(1) opens."""
    _, p, n, tile = case
    m = 2048
    assert u8_plan(m, p, n, 32) == ("dequantize_absmax_u8 + fp16 gemm" if workspace_mode == "u8_dequantise_first"
                                    else f"gemm_nt_u8_mfma_{tile}x64")
    gen = torch.Generator(device="cuda").manual_seed(45 + n)
    q = torch.randint(0, 256, (n, p), generator=gen, device="cuda", dtype=torch.uint8)
    s = (torch.rand(n, p // 32, generator=gen, device="cuda") * 0.019 + 0.001).half()
    a = torch.randn(m, p, generator=gen, device="cuda").half()
    out = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    kern.matmul_nt_fp16u8(out, a, q, s, 32)
    w = torch.zeros(n, p, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(w, s, q)
    ref32 = a.float() @ w.float().t()
    rms = ref32.pow(2).mean().sqrt()
    err = (out.float() - ref32).abs()
    rel = (err / torch.maximum(ref32.abs(), rms)).max().item()
    assert rel <= 2e-3, rel
    # the unfloored ratio on every element of at least typical magnitude
    big = ref32.abs() >= rms
    assert (err[big] / ref32.abs()[big]).max().item() <= TOL
    out2 = torch.zeros_like(out)
    kern.matmul_nt_fp16u8(out2, (a * 2).half(), q, s, 32)
    # (powers of two commute with the rounding of normal numbers; among 8 to 25 million outputs
    # a few dozen are subnormal, where they do not)
    normal = out.abs() >= 2.0 ** -13
    assert torch.equal(out2[normal], (out * 2).half()[normal])
    assert (out2[~normal].float() - 2 * out[~normal].float()).abs().max().item() <= 2.0 ** -23


def test_u8_other_block_sizes_and_fallbacks(kern):
    g = rng(630)
    for m, p, n, bs in [(4, 512, 40, 64), (4, 384, 40, 128), (3, 96, 20, 8), (2, 48, 10, 16),
                        (40, 320, 70, 64), (2, 4608, 40, 64), (2, 4608, 40, 32)]:
        a, q, s = _u8_case(g, m, p, n, bs, exact=True)
        want = np.zeros((m, n), np.float16)
        oracle.matmul_nt_fp16u8(want, a, q, s, bs)
        out = torch.zeros(m, n, dtype=torch.float16, device="cuda")
        kern.matmul_nt_fp16u8(out, to_dev(a), to_dev(q), to_dev(s), bs)
        assert np.array_equal(to_np(out).view(np.uint16), want.view(np.uint16)), (m, p, n, bs)
    lib = _ffi.lib()
    z = torch.zeros(64, dtype=torch.float16, device="cuda")
    assert lib.adr_matmul_nt_fp16u8(None, z.data_ptr(), z.data_ptr(), z.data_ptr(), z.data_ptr(),
                                    1, 40, 1, 32, 0.0) == -5   # p % block_size
    assert lib.adr_matmul_nt_fp16u8(None, None, z.data_ptr(), z.data_ptr(), z.data_ptr(),
                                    1, 32, 1, 32, 0.0) == -4
    # p == 0: an empty sum; the operands may be null, the output becomes beta * out for any m
    for m in (1, 4, 40):
        prev = torch.full((m, 24), 2.0, dtype=torch.float16, device="cuda")
        assert lib.adr_matmul_nt_fp16u8(torch.cuda.current_stream().cuda_stream, prev.data_ptr(),
                                        None, None, None, m, 0, 24, 32, 0.5) == 0
        assert torch.all(prev == 1.0)


DECODE = [(4096, 4096), (4096, 11008), (4096, 12288), (11008, 4096), (5120, 13824), (8192, 4100)]


@pytest.mark.parametrize("workspace_mode", ["pool_off", "shipped_default"], indirect=True)
@pytest.mark.parametrize("kn", DECODE, ids=[f"K{k}_N{n}" for k, n in DECODE])
@pytest.mark.parametrize("m", [1, 4, 16])
def test_decode_shapes_full_size(kern, kn, m, workspace_mode):
    """benchmark config 3 at full size against an fp32 GEMM on the (bit-exactly) dequantised
    weights, computed on the device; with the workspace pool off and as the library ships."""
    p, n = kn
    gen = torch.Generator(device="cuda").manual_seed(44)
    q = torch.randint(0, 256, (n, p), generator=gen, device="cuda", dtype=torch.uint8)
    s = (torch.rand(n, p // 32, generator=gen, device="cuda") * 0.019 + 0.001).half()
    a = torch.randn(m, p, generator=gen, device="cuda").half()
    assert u8_plan(m, p, n, 32) == ("gemv_u8_dot2_stream" if m <= 2 else "gemv_u8_mfma16_regstream")
    out = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    kern.matmul_nt_fp16u8(out, a, q, s, 32)
    w = torch.zeros(n, p, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(w, s, q)
    ref32 = a.float() @ w.float().t()
    rms = ref32.pow(2).mean().sqrt()
    rel = ((out.float() - ref32).abs() / torch.maximum(ref32.abs(), rms)).max().item()
    assert rel <= 2e-3, rel
    # the plain ratio |got - ref| / |ref| wherever the reference is at least of typical size
    big = ref32.abs() >= rms
    assert ((out.float() - ref32).abs()[big] / ref32.abs()[big]).max().item() <= 2e-3
    # linearity in the activations: f(2a) == 2 f(a) exactly (powers of two commute with rounding)
    out2 = torch.zeros_like(out)
    kern.matmul_nt_fp16u8(out2, (a * 2).half(), q, s, 32)
    assert torch.equal(out2, (out * 2).half())


@pytest.mark.parametrize("m", [10, 13, 16])
@pytest.mark.parametrize("kn", [(11008, 1000), (9472, 530), (12288, 700)])
def test_decode_ten_rows_and_more_long_k(kern, kn, m):
    """K 9472 .. 12288 with ten to sixteen rows: five and six macro steps per wavefront with
    uneven counts over the wavefronts (37, 43 and 48 steps over eight), ragged N, previous output
    added."""
    p, n = kn
    gen = torch.Generator(device="cuda").manual_seed(46 + m + p)
    q = torch.randint(0, 256, (n, p), generator=gen, device="cuda", dtype=torch.uint8)
    s = (torch.rand(n, p // 32, generator=gen, device="cuda") * 0.019 + 0.001).half()
    a = torch.randn(m, p, generator=gen, device="cuda").half()
    prev = torch.randn(m, n, generator=gen, device="cuda").half()
    assert u8_plan(m, p, n, 32) == "gemv_u8_mfma16_regstream"
    out = prev.clone()
    assert _ffi.lib().adr_matmul_nt_fp16u8(torch.cuda.current_stream().cuda_stream, out.data_ptr(),
                                           a.data_ptr(), q.data_ptr(), s.data_ptr(), m, p, n, 32, 0.5) == 0
    w = torch.zeros(n, p, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(w, s, q)
    ref32 = a.float() @ w.float().t() + 0.5 * prev.float()
    rms = ref32.pow(2).mean().sqrt()
    rel = ((out.float() - ref32).abs() / torch.maximum(ref32.abs(), rms)).max().item()
    assert rel <= 2e-3, rel


@pytest.mark.parametrize("m", [17, 32, 33, 50, 64, 65, 100, 128, 200, 256])
@pytest.mark.parametrize("kn", [(4096, 4100), (4096, 8200), (11008, 1000), (2048, 2100)])
def test_seventeen_and_more_rows_in_passes(kern, kn, m):
    """17 rows and more on matrices of 4 MiB and more run in passes of up to 64 rows, each
    reading the weights once for two to four blocks of sixteen rows (K = 4096 up to 32 rows: the
    DMA-ring kernel; a last pass of up to sixteen rows: the blocks kernel with one block); above
    32 rows only where that is estimated to beat the tiled GEMM.  Previous output added, ragged N."""
    p, n = kn
    name = u8_plan(m, p, n, 32)
    if m <= 32:
        assert name == ("gemv_u8_mfma16_dma_32rows" if p == 4096 else "gemv_u8_mfma16_blocks")
    else:
        assert name == "gemv_u8_mfma16_blocks" or name.startswith("gemm_nt_u8_")
    # decisions the estimate must make: to 128 rows against a narrow matrix the passes stay,
    # more rows or a matrix of several rounds of workgroups go to the tiled kernel
    assert u8_plan(64, 11008, 4096, 32) == "gemv_u8_mfma16_blocks"
    assert u8_plan(128, 11008, 4096, 32) == "gemv_u8_mfma16_blocks"
    assert u8_plan(160, 11008, 4096, 32).startswith("gemm_nt_u8_mfma_64x64")
    assert u8_plan(48, 4096, 12288, 32).startswith("gemm_nt_u8_mfma_64x64")
    assert u8_plan(100, 4096, 8200, 32).startswith("gemm_nt_u8_")
    assert u8_plan(257, 11008, 1000, 32).startswith("gemm_nt_u8_")
    # one pass against a matrix whose 64 x 64 tiles would need a second round (LLaMA-30B's and
    # 65B's gate / up projections): the pass
    assert u8_plan(40, 6656, 17920, 32) == "gemv_u8_mfma16_blocks"
    assert u8_plan(48, 8192, 22016, 32) == "gemv_u8_mfma16_blocks"
    assert u8_plan(64, 8192, 22016, 32).startswith("gemm_nt_u8_")
    gen = torch.Generator(device="cuda").manual_seed(47 + m + p)
    q = torch.randint(0, 256, (n, p), generator=gen, device="cuda", dtype=torch.uint8)
    s = (torch.rand(n, p // 32, generator=gen, device="cuda") * 0.019 + 0.001).half()
    a = torch.randn(m, p, generator=gen, device="cuda").half()
    prev = torch.randn(m, n, generator=gen, device="cuda").half()
    out = prev.clone()
    assert _ffi.lib().adr_matmul_nt_fp16u8(torch.cuda.current_stream().cuda_stream, out.data_ptr(),
                                           a.data_ptr(), q.data_ptr(), s.data_ptr(), m, p, n, 32, 0.5) == 0
    w = torch.zeros(n, p, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(w, s, q)
    ref32 = a.float() @ w.float().t() + 0.5 * prev.float()
    rms = ref32.pow(2).mean().sqrt()
    rel = ((out.float() - ref32).abs() / torch.maximum(ref32.abs(), rms)).max().item()
    assert rel <= 2e-3, rel


@pytest.mark.parametrize("mpn", [(256, 11008, 4096), (500, 4096, 4090)])
def test_tiles_that_split_k_over_wavefront_groups_give_the_same_bits_every_launch(kern, mpn):
    """The groups' partial sums meet in LDS in group order, whichever group finishes first: twenty
    launches (and one on another stream) of the 64 x 64 tile with four groups and of the 128 x 64
    tile with two give one result, equal to the same tile without groups up to fp32 summation
    order."""
    m, p, n = mpn
    name = u8_plan(m, p, n, 32)
    assert name in ("gemm_nt_u8_mfma_64x64x64_k4", "gemm_nt_u8_mfma_128x64x64_k2")
    gen = torch.Generator(device="cuda").manual_seed(49 + m)
    q = torch.randint(0, 256, (n, p), generator=gen, device="cuda", dtype=torch.uint8)
    s = (torch.rand(n, p // 32, generator=gen, device="cuda") * 0.019 + 0.001).half()
    a = torch.randn(m, p, generator=gen, device="cuda").half()
    lib = _ffi.lib()

    def run(stream):
        out = torch.zeros(m, n, dtype=torch.float16, device="cuda")
        assert lib.adr_matmul_nt_fp16u8(stream, out.data_ptr(), a.data_ptr(), q.data_ptr(), s.data_ptr(),
                                        m, p, n, 32, 0.0) == 0
        return out
    first = run(torch.cuda.current_stream().cuda_stream)
    for _ in range(19):
        assert torch.equal(run(torch.cuda.current_stream().cuda_stream), first)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        other = run(side.cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(other, first)
    w = torch.zeros(n, p, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(w, s, q)
    ref32 = a.float() @ w.float().t()
    rms = ref32.pow(2).mean().sqrt()
    assert ((first.float() - ref32).abs() / torch.maximum(ref32.abs(), rms)).max().item() <= 2e-3


@pytest.mark.parametrize("mpn", [(300, 4096, 4096), (512, 2048, 4090), (260, 11008, 1000)])
def test_mid_row_counts_take_the_smaller_tiles(kern, mpn):
    """A few hundred rows against a narrow matrix are too few 256-row tiles for the compute units:
    the u8 kernel's 128 x 64 and 64 x 64 tiles take them, K split over groups of wavefronts where
    there is at most one tile per compute unit; same arithmetic bar as the large tiles."""
    m, p, n = mpn
    assert (m + 255) // 256 * ((n + 127) // 128) <= 64
    assert u8_plan(m, p, n, 32) in ("gemm_nt_u8_mfma_128x64x64_k2", "gemm_nt_u8_mfma_64x64x64_k4",
                                    "gemm_nt_u8_mfma_128x64x64", "gemm_nt_u8_mfma_64x64x64")
    gen = torch.Generator(device="cuda").manual_seed(48 + m)
    q = torch.randint(0, 256, (n, p), generator=gen, device="cuda", dtype=torch.uint8)
    s = (torch.rand(n, p // 32, generator=gen, device="cuda") * 0.019 + 0.001).half()
    a = torch.randn(m, p, generator=gen, device="cuda").half()
    prev = torch.randn(m, n, generator=gen, device="cuda").half()
    out = prev.clone()
    assert _ffi.lib().adr_matmul_nt_fp16u8(torch.cuda.current_stream().cuda_stream, out.data_ptr(),
                                           a.data_ptr(), q.data_ptr(), s.data_ptr(), m, p, n, 32, 0.5) == 0
    w = torch.zeros(n, p, dtype=torch.float16, device="cuda")
    kern.dequantize_absmax_uint8(w, s, q)
    ref32 = a.float() @ w.float().t() + 0.5 * prev.float()
    rms = ref32.pow(2).mean().sqrt()
    rel = ((out.float() - ref32).abs() / torch.maximum(ref32.abs(), rms)).max().item()
    assert rel <= 2e-3, rel


def test_descriptor_forms_on_strided_views(kern):
    """adr_dequantize_absmax_uint8 / adr_quantize_absmax_uint8 take the reference's by-value
    TensorGpuDescriptor (index 0 = innermost dim, kernels.rs:28-61); views with row padding."""
    from adrastea_amd import TensorView, TensorLayout
    from adrastea_amd.kernels import descriptor
    g = rng(640)
    rows, cols, bs, pad = 7, 96, 32, 40
    x = randn_f16(g, (rows, cols), 0.05)
    xb = torch.zeros(rows, cols + pad, dtype=torch.float16, device="cuda")
    xb[:, :cols] = to_dev(x)
    qb = torch.zeros(rows, cols + pad, dtype=torch.uint8, device="cuda")
    sb = torch.zeros(rows, cols // bs + 3, dtype=torch.float16, device="cuda")
    xv = TensorView(xb, TensorLayout((rows, cols), (cols + pad, 1)))
    qv = TensorView(qb, TensorLayout((rows, cols), (cols + pad, 1)))
    sv = TensorView(sb, TensorLayout((rows, cols // bs), (cols // bs + 3, 1)))
    lib = _ffi.lib()
    assert lib.adr_quantize_absmax_uint8(None, descriptor(qv), descriptor(sv), descriptor(xv)) == 0
    q_want, s_want = oracle.quantize_absmax_u8(x, bs)
    assert np.array_equal(to_np(qb)[:, :cols], q_want)
    assert np.all(to_np(qb)[:, cols:] == 0)
    assert np.array_equal(to_np(sb)[:, :cols // bs].view(np.uint16), s_want.view(np.uint16))
    ob = torch.full((rows, cols + pad), 9.0, dtype=torch.float16, device="cuda")
    ov = TensorView(ob, TensorLayout((rows, cols), (cols + pad, 1)))
    assert lib.adr_dequantize_absmax_uint8(None, descriptor(ov), descriptor(sv), descriptor(qv)) == 0
    want = oracle.dequantize_absmax_u8(q_want, s_want, bs)
    assert np.array_equal(to_np(ob)[:, :cols].view(np.uint16), want.view(np.uint16))
    assert np.all(to_np(ob)[:, cols:] == 9.0)
    # shape errors
    bad = TensorView(sb, TensorLayout((rows + 1, cols // bs), (cols // bs + 3, 1)))
    assert lib.adr_dequantize_absmax_uint8(None, descriptor(ov), descriptor(bad), descriptor(qv)) == -1


@pytest.mark.parametrize("shape", [(129, 4096, 4096), (300, 1024, 8200), (512, 11008, 4096), (1024, 4096, 4096),
                                   (1100, 448, 12288), (2048, 4096, 12288), (1700, 640, 9000), (96, 4096, 4096),
                                   (65, 11008, 4096), (128, 4096, 4096), (80, 4096, 8200),
                                   # the fused call in passes of 64 rows, the workspace used
                                   (200, 11008, 1000), (100, 2048, 8200), (256, 4096, 4100)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_workspace_variant_gives_the_bits_of_the_fused_call(shape, beta):
    """adr_matmul_nt_fp16u8_ws (weights dequantised once into the workspace, then the fp16
    kernels) against adr_matmul_nt_fp16u8 on the same operands.  Both round every weight to fp16
    with the reference's dequantisation; where the fused call runs its tiled kernels (always from
    257 rows on) both also sum slices of K in the same order and the outputs are compared bit for
    bit, as they are where the workspace is not used.  Where the fused call runs its passes of 64
    rows (wavefronts split K) both are held to the fp32 product.  With the previous output added
    and without."""
    m, p, n = shape
    lib = _ffi.lib()
    gen = torch.Generator(device="cuda").manual_seed(m + p + n)
    q = torch.randint(0, 256, (n, p), generator=gen, device="cuda", dtype=torch.uint8)
    s = (torch.rand(n, p // 32, generator=gen, device="cuda") * 0.019 + 0.001).half()
    a = torch.randn(m, p, generator=gen, device="cuda").half()
    prev = torch.randn(m, n, generator=gen, device="cuda").half()
    need = lib.adr_matmul_nt_fp16u8_workspace_bytes(m, p, n, 32)
    assert need in (0, n * p * 2)
    ws = torch.full((max(need, 16),), 0x7f, dtype=torch.uint8, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    want, got = prev.clone(), prev.clone()
    assert lib.adr_matmul_nt_fp16u8(st, want.data_ptr(), a.data_ptr(), q.data_ptr(), s.data_ptr(), m, p, n, 32, beta) == 0
    assert lib.adr_matmul_nt_fp16u8_ws(st, got.data_ptr(), a.data_ptr(), q.data_ptr(), s.data_ptr(), m, p, n, 32,
                                       beta, ws.data_ptr(), ws.numel()) == 0
    torch.cuda.synchronize()
    if not need or u8_plan(m, p, n, 32).startswith("gemm_nt_u8_"):
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    else:
        # the fused call's wavefronts split K, the workspace path's do not: same weights, another
        # order of the fp32 sums
        assert m <= 256
        w = torch.empty(n, p, dtype=torch.float16, device="cuda")
        assert lib.adr_dequantize_absmax_u8(st, w.data_ptr(), q.data_ptr(), s.data_ptr(), n, p, 32) == 0
        ref = a.float() @ w.float().t() + beta * prev.float()
        rms = ref.pow(2).mean().sqrt()
        for t in (got, want):
            assert ((t.float() - ref).abs() / torch.maximum(ref.abs(), rms)).max().item() <= 2e-3
    if need:
        # the workspace held the dequantised matrix, bit-identical to the stand-alone kernel
        w = torch.empty(n, p, dtype=torch.float16, device="cuda")
        assert lib.adr_dequantize_absmax_u8(st, w.data_ptr(), q.data_ptr(), s.data_ptr(), n, p, 32) == 0
        assert torch.equal(ws[:need].view(torch.float16).view(n, p), w)
        # too small a workspace: the fused call, same bits again
        again = prev.clone()
        assert lib.adr_matmul_nt_fp16u8_ws(st, again.data_ptr(), a.data_ptr(), q.data_ptr(), s.data_ptr(), m, p, n,
                                           32, beta, ws.data_ptr(), need - 16) == 0
        assert torch.equal(again.view(torch.int16), want.view(torch.int16))   # (the fused call itself)
    else:
        assert torch.all(ws == 0x7f)   # untouched
