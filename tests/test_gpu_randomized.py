"""Randomised differential tests of the dispatch: seeded random shapes, strides, offsets and
operators through adr_matmul_f16 against adr_matmul_f16_slow (the step-for-step kernel of
matmul.cu:195-222, itself held bit for bit to the CPU oracle in test_gpu_matmul.py), and random
u8 products through adr_matmul_nt_fp16u8 against a float64 evaluation of matmul_nt_fp16u8.cu:17-21.

The data make the arithmetic exact, so the bar is bit identity of the WHOLE output buffer,
padding included: operands are small integers (every product and every partial sum is an integer
below 2^24, exact in fp32 in any summation order), scales are powers of two, previous outputs and
biases multiples of 1/4.  The two GELU operators are the exception: the tiled kernels evaluate
them with the hardware's exp2 and reciprocal, the slow kernel with expf / tanhf as the reference
does (matmul.cu:109-144); there the bar is 2 fp16 steps, the sign of a zero left free.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from adrastea_amd import _ffi

pytestmark = pytest.mark.gpu

GELU_STORES = (oracle.STORE_BETA_GELU_BIAS, oracle.STORE_QUICK_GELU_BIAS)
# (STORE_GELU_BIAS is not drawn: it has no device case in the reference and is refused)
STORES = [oracle.STORE_IDENTITY, oracle.STORE_IDENTITY, oracle.STORE_BETA_GELU_BIAS, oracle.STORE_BETA_BIAS,
          oracle.STORE_SCALE, oracle.STORE_ADD, oracle.STORE_QUICK_GELU_BIAS]


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _layout(g, rows, cols, contiguous, pads):
    """(stride along a row, stride between rows, elements spanned) of a rows x cols matrix."""
    pad = int(g.choice(pads))
    if contiguous:
        return 1, cols + pad, rows * (cols + pad)
    return rows + pad, 1, cols * (rows + pad)


def _f16_case(g, long_k=False):
    pick = lambda xs: xs[int(g.integers(0, len(xs)))]
    aligned = g.random() < 0.85
    B = int(pick([1, 1, 1, 1, 2, 3, 5]))
    r = g.random()
    M = int(g.integers(1, 65)) if r < 0.25 else int(g.integers(65, 700)) if r < 0.55 else \
        int(pick([1024, 1280, 1536, 2048, 2056, 2304, 4096])) + int(pick([0, 0, 0, 1, -1, 8, -8, 3, 24, 40, -100]))
    r = g.random()
    N = int(g.integers(1, 600)) if r < 0.25 else \
        int(pick([1024, 2304, 4096, 5120, 8192, 11008, 12288])) + int(pick([0, 0, 0, 0, 1, -1, 8, -8, 3, 24, 40, -200]))
    km = g.random()
    if aligned:
        K = int(pick([64, 128, 192, 256, 320, 512, 768, 1024, 2048, 4096, 5120, 11008])) if km < 0.7 \
            else 8 * int(g.integers(1, 300))
    else:
        K = 8 * int(g.integers(1, 200)) if km < 0.5 else int(g.integers(1, 700))
    if long_k and g.random() < 0.6:   # few tiles, long K: what a workspace splits
        M = int(g.integers(1, 400))
        N = int(pick([256, 512, 1024, 2048, 4096, 5120])) + int(pick([0, 0, 8, -8, 1]))
        K = int(pick([1024, 2048, 4096, 5120, 8192, 11008, 13824]))
    if M * N * B > 40e6 or M * N * K * B > 1.2e11:
        return None
    pads = [0, 0, 0, 8, 16, 64] if aligned else [0, 0, 8, 1, 3]
    lx, ly, lsz = _layout(g, M, K, aligned or g.random() < 0.7, pads)
    if g.random() < 0.75:   # W[N, K].permute([1, 0]): k contiguous
        ry, rx, rsz = _layout(g, N, K, True, pads)
    else:                   # [K, N] row major
        rx, ry, rsz = _layout(g, K, N, True, pads)
    ox, oy, osz = _layout(g, M, N, g.random() < 0.93, pads if g.random() < 0.8 else [1, 3])
    lz, rz, oz = lsz, rsz, osz
    bm = g.random()
    if B > 1 and bm < 0.2:
        lz = 0
    elif B > 1 and bm < 0.4:
        rz = 0
    elif B > 1 and bm < 0.55 and lx == 1:
        ly, lz = B * ly, ly   # head views: the batches interleaved inside a row (llama.rs:534-540)
    offs = [int(pick([0, 0, 0, 8, 16] if aligned else [0, 8, 1, 5])) for _ in range(3)]
    return dict(B=B, M=M, K=K, N=N, so=(ox, oy, oz), sl=(lx, ly, lz), sr=(rx, ry, rz), offs=offs,
                boff=int(pick([0, 0, 8, 1])), store=int(pick(STORES)),
                load=int(pick([0, 0, 0, 1])), mask=int(pick([0, 0, 0, 1])),
                beta=float(pick([0.0, 1.0, 0.5, -2.0])), scale=float(pick([1.0, 0.5, 0.25, 2.0])))


def _plan(c):
    buf = C.create_string_buffer(64)
    assert _ffi.lib().adr_matmul_f16_plan(buf, 64, c["B"], c["M"], c["K"], c["N"], *c["so"], *c["sl"], *c["sr"],
                                          c["store"], c["load"], c["mask"]) == 0
    return buf.value.decode()


@pytest.fixture
def held(request):
    """The library's own workspace cache switched on (default size) or left off for the test."""
    L = _ffi.lib()
    L.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES if request.param else 0)
    L.adr_set_u8_dequantise_first(1 if request.param else 0)
    yield request.param
    L.adr_set_held_workspace_limit(0)
    L.adr_set_u8_dequantise_first(0)


@pytest.mark.parametrize("seed,held", [(11, False), (12, False), (13, False), (14, True), (15, True)],
                         indirect=["held"])
def test_random_products_match_the_slow_kernel(seed, held):
    g = np.random.default_rng(seed)
    L = _ffi.lib()
    plans, failures = {}, []
    for it in range(110):
        c = _f16_case(g, long_k=held)
        if c is None:
            continue
        B, M, K, N = c["B"], c["M"], c["K"], c["N"]
        (ox, oy, oz), (lx, ly, lz), (rx, ry, rz), offs = c["so"], c["sl"], c["sr"], c["offs"]
        # every address the product may touch lies inside its buffer
        l_len = offs[1] + (M - 1) * ly + (K - 1) * lx + (B - 1) * lz + 1 + 8
        r_len = offs[2] + (K - 1) * ry + (N - 1) * rx + (B - 1) * rz + 1 + 8
        o_len = offs[0] + (M - 1) * oy + (N - 1) * ox + (B - 1) * oz + 1 + 8
        l_t = torch.from_numpy(g.integers(-3, 4, size=l_len).astype(np.float16)).cuda()
        r_t = torch.from_numpy(g.integers(-2, 3, size=r_len).astype(np.float16)).cuda()
        b_t = torch.from_numpy((g.integers(-8, 9, size=N + 8) / 4.0).astype(np.float16)).cuda()
        o1 = torch.from_numpy((g.integers(-8, 9, size=o_len) / 4.0).astype(np.float16)).cuda()
        o2 = o1.clone()
        name = _plan(c)
        plans[name] = plans.get(name, 0) + 1
        print(f"seed {seed} case {it}: {c} -> {name}", flush=True)
        rcs = [fn(_stream(), o.data_ptr() + 2 * offs[0], l_t.data_ptr() + 2 * offs[1], r_t.data_ptr() + 2 * offs[2],
                  B, M, K, N, ox, oy, oz, lx, ly, lz, rx, ry, rz, b_t.data_ptr() + 2 * c["boff"],
                  c["beta"], c["scale"], c["store"], c["load"], c["mask"])
               for fn, o in ((L.adr_matmul_f16, o1), (L.adr_matmul_f16_slow, o2))]
        torch.cuda.synchronize()
        assert rcs == [0, 0], (c, rcs)
        a, b = o1.view(torch.int16), o2.view(torch.int16)
        if torch.equal(a, b):
            continue
        diff = (a != b) & ~(torch.isnan(o1) & torch.isnan(o2))
        if c["store"] in GELU_STORES:
            ka = torch.where(a < 0, -(a.int() & 0x7FFF), a.int())
            kb = torch.where(b < 0, -(b.int() & 0x7FFF), b.int())
            diff &= (ka - kb).abs() > 2
        if bool(diff.any()):
            failures.append((c, name, int(diff.sum())))
    assert not failures, failures
    # the draw reaches the tiled kernels, not only the general one
    assert sum(v for k, v in plans.items() if k != "matmul_general") >= 40, plans


def _pv_case(g):
    """P.V on head views (llama.rs:552-554, whisper.rs:433-436): probabilities [H, S, T] with rows
    of any pitch from any element, values [T, H * D] and the output [S, H * D] interleaved by head."""
    pick = lambda xs: xs[int(g.integers(0, len(xs)))]
    H = int(pick([1, 2, 3, 8, 12, 20, 32]))
    D = int(pick([64, 64, 128, 128, 72, 200, 8, 136]))
    r = g.random()
    S = int(g.integers(1, 40)) if r < 0.35 else int(g.integers(40, 500)) if r < 0.8 else int(g.integers(500, 1600))
    r = g.random()
    T = int(g.integers(1, 200)) if r < 0.2 else int(g.integers(193, 1100)) if r < 0.6 else int(g.integers(1024, 2600))
    if g.random() < 0.15:
        T = 64 * int(g.integers(1, 40))
    if H * S * T > 30e6:
        return None
    pitch = T + int(pick([0, 0, 0, 1, 5, 8]))
    HD = H * D + int(pick([0, 0, 8, 64]))
    offs = [int(pick([0, 8])), int(pick([0, 0, 1, 8, 3])), int(pick([0, 8]))]
    return dict(B=H, M=S, K=T, N=D, so=(1, HD, D), sl=(1, pitch, S * pitch), sr=(1, HD, D), offs=offs,
                boff=int(pick([0, 0, 8, 1])), store=int(pick(STORES)), load=0, mask=int(pick([0, 0, 0, 1])),
                beta=float(pick([0.0, 1.0, 0.5, -2.0])), scale=float(pick([1.0, 0.5, 0.25, 2.0])))


@pytest.mark.parametrize("seed", [41, 42, 43])
def test_random_pv_products_match_the_slow_kernel(seed):
    """Every tile of the kernel for left rows of any alignment (and the direct-to-LDS kernels where
    the draw is aligned), every store operator and the causal mask on them."""
    g = np.random.default_rng(seed)
    L = _ffi.lib()
    plans, failures = {}, []
    for it in range(70):
        c = _pv_case(g)
        if c is None:
            continue
        B, M, K, N = c["B"], c["M"], c["K"], c["N"]
        (ox, oy, oz), (lx, ly, lz), (rx, ry, rz), offs = c["so"], c["sl"], c["sr"], c["offs"]
        l_len = offs[1] + (M - 1) * ly + (K - 1) * lx + (B - 1) * lz + 1   # the last probability ends the buffer
        r_len = offs[2] + (K - 1) * ry + (N - 1) * rx + (B - 1) * rz + 1 + 8
        o_len = offs[0] + (M - 1) * oy + (N - 1) * ox + (B - 1) * oz + 1 + 8
        l_t = torch.from_numpy(g.integers(-3, 4, size=l_len).astype(np.float16)).cuda()
        r_t = torch.from_numpy(g.integers(-2, 3, size=r_len).astype(np.float16)).cuda()
        b_t = torch.from_numpy((g.integers(-8, 9, size=N + 8) / 4.0).astype(np.float16)).cuda()
        o1 = torch.from_numpy((g.integers(-8, 9, size=o_len) / 4.0).astype(np.float16)).cuda()
        o2 = o1.clone()
        name = _plan(c)
        plans[name] = plans.get(name, 0) + 1
        print(f"seed {seed} case {it}: {c} -> {name}", flush=True)
        rcs = [fn(_stream(), o.data_ptr() + 2 * offs[0], l_t.data_ptr() + 2 * offs[1], r_t.data_ptr() + 2 * offs[2],
                  B, M, K, N, ox, oy, oz, lx, ly, lz, rx, ry, rz, b_t.data_ptr() + 2 * c["boff"],
                  c["beta"], c["scale"], c["store"], c["load"], c["mask"])
               for fn, o in ((L.adr_matmul_f16, o1), (L.adr_matmul_f16_slow, o2))]
        torch.cuda.synchronize()
        assert rcs == [0, 0], (c, rcs)
        a, b = o1.view(torch.int16), o2.view(torch.int16)
        if torch.equal(a, b):
            continue
        diff = (a != b) & ~(torch.isnan(o1) & torch.isnan(o2))
        if c["store"] in GELU_STORES:
            ka = torch.where(a < 0, -(a.int() & 0x7FFF), a.int())
            kb = torch.where(b < 0, -(b.int() & 0x7FFF), b.int())
            diff &= (ka - kb).abs() > 2
        if bool(diff.any()):
            failures.append((c, name, int(diff.sum())))
    assert not failures, failures
    for tile in ("128x128x64", "128x64x64", "64x64x64_k4", "32x64x64_k4"):
        assert any(k == "gemm_nn_mfma_anyrow_" + tile for k in plans) or seed != 41, (tile, plans)


def _u8_case(g):
    pick = lambda xs: xs[int(g.integers(0, len(xs)))]
    bs = int(pick([32, 32, 32, 64, 128, 8, 16]))
    r = g.random()
    m = int(g.integers(1, 65)) if r < 0.4 else int(g.integers(65, 257)) if r < 0.6 else \
        int(pick([300, 512, 1024, 1100, 2048])) + int(pick([0, 0, 1, -1, 17]))
    r = g.random()
    n = int(g.integers(1, 700)) if r < 0.2 else \
        int(pick([1000, 1024, 4096, 5120, 8200, 11008, 12288])) + int(pick([0, 0, 0, 1, -1, 5, 16]))
    p = int(pick([256, 512, 1024, 2048, 4096, 11008, 5120, 320, 640])) if g.random() < 0.75 else \
        bs * int(g.integers(1, max(2, 4096 // bs)))
    p = (p + bs - 1) // bs * bs
    if m * n > 30e6 or m * n * p > 1.2e11 or n * p > 140e6:
        return None
    return dict(m=m, p=p, n=n, bs=bs, beta=float(pick([0.0, 0.0, 1.0, 0.5])))


@pytest.mark.parametrize("seed,held", [(21, False), (22, False), (23, True)], indirect=["held"])
def test_random_u8_products_match_float64(seed, held):
    g = np.random.default_rng(seed)
    L = _ffi.lib()
    plans, failures = {}, []
    for it in range(90):
        c = _u8_case(g)
        if c is None:
            continue
        m, p, n, bs, beta = c["m"], c["p"], c["n"], c["bs"], c["beta"]
        q_t = torch.from_numpy(g.integers(0, 256, size=(n, p), dtype=np.uint8)).cuda()
        s_t = torch.from_numpy((2.0 ** g.integers(-6, -2, size=(n, p // bs))).astype(np.float16)).cuda()
        x_t = torch.from_numpy(g.integers(-3, 4, size=(m, p)).astype(np.float16)).cuda()
        o_t = torch.from_numpy((g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)).cuda()
        prev = o_t.double()
        buf = C.create_string_buffer(64)
        assert L.adr_matmul_nt_fp16u8_plan(buf, 64, m, p, n, bs) == 0
        name = buf.value.decode()
        plans[name] = plans.get(name, 0) + 1
        print(f"seed {seed} case {it}: {c} -> {name}", flush=True)
        rc = L.adr_matmul_nt_fp16u8(_stream(), o_t.data_ptr(), x_t.data_ptr(), q_t.data_ptr(), s_t.data_ptr(),
                                    m, p, n, bs, beta)
        torch.cuda.synchronize()
        assert rc == 0, c
        # (q - 127.5) s: nine significant bits times a power of two; the sums stay below 2^53
        w = (q_t.double() - 127.5) * s_t.double().repeat_interleave(bs, dim=1)
        want = (x_t.double() @ w.t() + beta * prev).half()
        if not torch.equal(want.view(torch.int16), o_t.view(torch.int16)):
            failures.append((c, name, int((want.view(torch.int16) != o_t.view(torch.int16)).sum())))
    assert not failures, failures
    assert len(plans) >= 4, plans


@pytest.mark.parametrize("seed,held", [(31, False), (32, True)], indirect=["held"])
def test_random_nt_f16_products_match_float64(seed, held):
    """adr_matmul_nt_f16 (matmul_nt_wmma_16x128x256.cu:8-68: O = A B^T + beta O on the fp32 sum,
    rounded once) on random sizes; exact data, so every kernel and epilogue it may take -- streaming
    kernels, tiles with rows or columns past the matrix, aligned and unaligned rows -- has to give
    the bits of a float64 evaluation."""
    g = np.random.default_rng(seed)
    L = _ffi.lib()
    pick = lambda xs: xs[int(g.integers(0, len(xs)))]
    failures = []
    for it in range(70):
        r = g.random()
        m = int(g.integers(1, 65)) if r < 0.3 else int(g.integers(65, 700)) if r < 0.6 else \
            int(pick([1024, 2048, 2056, 4096])) + int(pick([0, 0, 1, -1, 8, -100]))
        n = int(g.integers(1, 600)) if g.random() < 0.25 else \
            int(pick([1024, 4096, 8192, 11008, 12288])) + int(pick([0, 0, 0, 1, -1, 8, -8, 24, -200]))
        p = int(pick([64, 128, 256, 320, 512, 1024, 2048, 4096, 11008])) if g.random() < 0.8 else 8 * int(g.integers(1, 300))
        if m * n > 40e6 or m * n * p > 1.2e11:
            continue
        beta = float(pick([0.0, 1.0, 1.0, 0.5, -2.0]))
        a = torch.from_numpy(g.integers(-3, 4, size=(m, p)).astype(np.float16)).cuda()
        w = torch.from_numpy(g.integers(-2, 3, size=(n, p)).astype(np.float16)).cuda()
        prev = torch.from_numpy((g.integers(-8, 9, size=(m, n)) / 4.0).astype(np.float16)).cuda()
        out = prev.clone()
        print(f"seed {seed} case {it}: m={m} p={p} n={n} beta={beta}", flush=True)
        rc = L.adr_matmul_nt_f16(_stream(), out.data_ptr(), a.data_ptr(), w.data_ptr(), m, p, n, beta)
        torch.cuda.synchronize()
        assert rc == 0
        want = (a.double() @ w.double().t() + beta * prev.double()).half()
        if not torch.equal(want.view(torch.int16), out.view(torch.int16)):
            failures.append((m, p, n, beta, int((want.view(torch.int16) != out.view(torch.int16)).sum())))
    assert not failures, failures
