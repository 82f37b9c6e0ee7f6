"""GPU parity of the split-K form of the fp16 NT GEMM (adr_matmul_f16_ws, through the C ABI):
products with few output tiles and a long K run as several workgroups per tile plus a reduction
launch.  Bars as for the unsplit kernels: bit-exact against the oracle where every sum is exactly
representable (every store operator, the causal mask, ragged M / N, pieces of unequal length,
batches); max relative error 1e-2 against an fp32 GEMM on random inputs at the sizes the split is
meant for; and the workspace contract (too small -> the unsplit kernel, same result)."""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from helpers import rng, ulp_diff_f16
from gpu_common import to_dev, to_np, oracle_matmul
from adrastea_amd import _ffi

pytestmark = pytest.mark.gpu
TOL = 1e-2


def ws_plan(B, M, K, N, so, sl, sr, store=0, load=0, mask=0, ws_bytes=0):
    buf = C.create_string_buffer(96)
    rc = _ffi.lib().adr_matmul_f16_ws_plan(buf, 96, B, M, K, N, *so, *sl, *sr, store, load, mask, ws_bytes)
    assert rc == 0
    return buf.value.decode()


def ws_bytes_needed(B, M, K, N, so, sl, sr, store=0, load=0, mask=0):
    return _ffi.lib().adr_matmul_f16_workspace_bytes(B, M, K, N, *so, *sl, *sr, store, load, mask)


def call_ws(out_t, l_t, r_t, B, M, K, N, so, sl, sr, ws_t, ws_bytes=None, bias_t=None, beta=0.0, scale=1.0,
            store=0, load=0, mask=0):
    stream = torch.cuda.current_stream().cuda_stream
    return _ffi.lib().adr_matmul_f16_ws(
        stream, out_t.data_ptr(), l_t.data_ptr(), r_t.data_ptr(), B, M, K, N, *so, *sl, *sr,
        bias_t.data_ptr() if bias_t is not None else None, float(beta), float(scale), store, load, mask,
        ws_t.data_ptr() if ws_t is not None else None,
        (ws_t.numel() if ws_t is not None else 0) if ws_bytes is None else ws_bytes)


@pytest.fixture(scope="module")
def ws():
    return torch.empty(64 << 20, dtype=torch.uint8, device="cuda")


def nt(M, K, N):
    return (1, N, 0), (1, K, 0), (K, 1, 0)


STORES = [(0, "identity"), (4, "scale"), (5, "add"), (3, "beta_bias"), (6, "quick_gelu_bias"),
          (2, "beta_gelu_bias")]


@pytest.mark.parametrize("store", STORES, ids=[s[1] for s in STORES])
@pytest.mark.parametrize("shape", [(100, 1472, 1000), (130, 3008, 520), (250, 11008, 300)],
                         ids=lambda s: "M%d_K%d_N%d" % s)
def test_split_k_bit_exact_on_exact_inputs(ws, store, shape):
    """Dyadic inputs: every partial sum is exact in fp32, so the split result must equal the
    oracle bit for bit whatever the number of pieces (here 5, 8 and 16 of 23, 47 and 172 slices:
    pieces of unequal length); ragged last tile row and column."""
    op, _ = store
    M, K, N = shape
    so, sl, sr = nt(M, K, N)
    need = ws_bytes_needed(1, M, K, N, so, sl, sr, store=op)
    assert need > 0 and "_splitk" in ws_plan(1, M, K, N, so, sl, sr, store=op, ws_bytes=ws.numel())
    g = rng(4200 + M + op)
    a = (g.integers(-4, 5, size=(M, K)) / 8.0).astype(np.float16)
    w = (g.integers(-4, 5, size=(N, K)) / 8.0).astype(np.float16)
    prev = (g.integers(-8, 9, size=(M, N)) / 4.0).astype(np.float16)
    bias = (g.integers(-8, 9, size=N) / 4.0).astype(np.float16)
    beta, scale = 0.5, 0.25
    want = oracle_matmul(prev.reshape(-1), a, w, 1, M, K, N, so, sl, sr, bias=bias, beta=beta,
                         scale=scale if op == 4 else 1.0, store=op, mode=oracle.EXACT)
    out = to_dev(prev)
    rc = call_ws(out, to_dev(a), to_dev(w), 1, M, K, N, so, sl, sr, ws, bias_t=to_dev(bias), beta=beta,
                 scale=scale if op == 4 else 1.0, store=op)
    assert rc == 0
    got = to_np(out).reshape(-1)
    if op in (6, 2):   # exp / tanh in the epilogue: device intrinsics against libm
        assert np.max(ulp_diff_f16(got, want)) <= 2
    else:
        assert np.array_equal(got.view(np.uint16), want.view(np.uint16))


def test_split_k_causal_mask_and_batches(ws):
    """Batched product with the causal mask: tiles above the diagonal are filled by the reduction
    launch without any piece having been written for them; batch strides on all three tensors."""
    B, M, K, N = 3, 200, 4096, 260
    so, sl, sr = (1, N, M * N), (1, K, M * K), (K, 1, N * K)
    assert "_splitk" in ws_plan(B, M, K, N, so, sl, sr, store=4, mask=1, ws_bytes=ws.numel())
    g = rng(4300)
    a = (g.integers(-4, 5, size=(B, M, K)) / 8.0).astype(np.float16)
    w = (g.integers(-4, 5, size=(B, N, K)) / 8.0).astype(np.float16)
    want = oracle_matmul(np.zeros(B * M * N, np.float16), a, w, B, M, K, N, so, sl, sr, scale=0.125,
                         store=4, mask=1, mode=oracle.EXACT)
    out = torch.full((B, M, N), 7.0, dtype=torch.float16, device="cuda")
    assert call_ws(out, to_dev(a), to_dev(w), B, M, K, N, so, sl, sr, ws, scale=0.125, store=4, mask=1) == 0
    got = to_np(out).reshape(-1)
    assert np.array_equal(got.view(np.uint16), want.view(np.uint16))
    assert np.all(got.reshape(B, M, N)[:, 0, 1:].view(np.uint16) == 0xFC00)


@pytest.mark.parametrize("case", [(200, 4160, 3000, "128x64x64"), (128, 11008, 4096, "128x128x64"),
                                  (70, 6080, 2048, "64x64x64")], ids=lambda c: c[3])
def test_split_k_every_tile_bit_exact_against_float64(ws, case):
    """The three tile shapes of the split kernel at sizes the oracle would take minutes for:
    dyadic inputs, expected value = one rounding of the float64 product (every partial sum is
    exactly representable, so any summation order gives it)."""
    M, K, N, tile = case
    so, sl, sr = nt(M, K, N)
    assert ("_dma_" + tile + "_splitk") in ws_plan(1, M, K, N, so, sl, sr, ws_bytes=ws.numel())
    gen = torch.Generator(device="cuda").manual_seed(4400 + M)
    a = (torch.randint(-4, 5, (M, K), generator=gen, device="cuda") / 8.0).half()
    w = (torch.randint(-4, 5, (N, K), generator=gen, device="cuda") / 8.0).half()
    out = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    assert call_ws(out, a, w, 1, M, K, N, so, sl, sr, ws) == 0
    want = (a.double() @ w.double().t()).half()
    assert torch.equal(out, want)


@pytest.mark.parametrize("m", [96, 128, 256])
def test_split_k_down_projection_random_inputs(ws, m):
    """The shape the split is for: a few dozen to a few hundred rows against the LLaMA-7B down
    projection (K 11008 -> N 4096), random inputs, against an fp32 GEMM on the device and against
    the unsplit kernel."""
    K, N = 11008, 4096
    so, sl, sr = nt(m, K, N)
    assert "_splitk" in ws_plan(1, m, K, N, so, sl, sr, ws_bytes=ws.numel())
    assert "_splitk" not in ws_plan(1, m, K, N, so, sl, sr, ws_bytes=0)
    gen = torch.Generator(device="cuda").manual_seed(77 + m)
    a = torch.randn(m, K, generator=gen, device="cuda").half()
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    out = torch.zeros(m, N, dtype=torch.float16, device="cuda")
    assert call_ws(out, a, w, 1, m, K, N, so, sl, sr, ws) == 0
    ref = a.float() @ w.float().t()
    rms = ref.pow(2).mean().sqrt()
    err = (out.float() - ref).abs()
    assert (err / torch.maximum(ref.abs(), rms)).max().item() <= 2e-3
    big = ref.abs() >= rms
    assert (err[big] / ref.abs()[big]).max().item() <= TOL
    plain = torch.zeros_like(out)
    assert call_ws(plain, a, w, 1, m, K, N, so, sl, sr, None) == 0
    # different summation order only: the two agree to a fraction of an fp16 step of the typical
    # output magnitude
    assert (out.float() - plain.float()).abs().max().item() <= 2e-3 * rms.item()


def test_workspace_contract(ws):
    """With no workspace, or one smaller than adr_matmul_f16_workspace_bytes says, the call is
    adr_matmul_f16 bit for bit; a misaligned or missing buffer is an argument error; the second
    call on the same workspace with a smaller problem is unaffected by the first."""
    lib = _ffi.lib()
    M, K, N = 128, 11008, 4096
    so, sl, sr = nt(M, K, N)
    need = ws_bytes_needed(1, M, K, N, so, sl, sr)
    assert need > 0 and need % 16 == 0
    assert "_splitk" in ws_plan(1, M, K, N, so, sl, sr, ws_bytes=need)
    assert "_splitk" not in ws_plan(1, M, K, N, so, sl, sr, ws_bytes=need // 8)
    gen = torch.Generator(device="cuda").manual_seed(78)
    a = torch.randn(M, K, generator=gen, device="cuda").half()
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    base = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.adr_matmul_f16(stream, base.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N, *so, *sl,
                              *sr, None, 0.0, 1.0, 0, 0, 0) == 0
    small = torch.zeros_like(base)
    assert call_ws(small, a, w, 1, M, K, N, so, sl, sr, ws, ws_bytes=1024) == 0
    assert torch.equal(small, base)
    none = torch.zeros_like(base)
    assert call_ws(none, a, w, 1, M, K, N, so, sl, sr, None) == 0
    assert torch.equal(none, base)
    # argument errors
    assert lib.adr_matmul_f16_ws(stream, base.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N, *so,
                                 *sl, *sr, None, 0.0, 1.0, 0, 0, 0, None, 4096) == _ffi.ADR_ENULL
    assert lib.adr_matmul_f16_ws(stream, base.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N, *so,
                                 *sl, *sr, None, 0.0, 1.0, 0, 0, 0, ws.data_ptr() + 4, 4096) == _ffi.ADR_EINVAL_SHAPE
    assert lib.adr_matmul_f16_ws(stream, base.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N, *so,
                                 *sl, *sr, None, 0.0, 1.0, 0, 0, 0, ws.data_ptr(), -1) == _ffi.ADR_ENULL
    # two calls in a row on one workspace, the second smaller: nothing carries over
    first = torch.zeros_like(base)
    assert call_ws(first, a, w, 1, M, K, N, so, sl, sr, ws) == 0
    m2 = 70
    so2, sl2, sr2 = nt(m2, K, N)
    second = torch.zeros(m2, N, dtype=torch.float16, device="cuda")
    assert call_ws(second, a[:m2], w, 1, m2, K, N, so2, sl2, sr2, ws) == 0
    fresh = torch.zeros_like(second)
    ws2 = torch.zeros(ws.numel(), dtype=torch.uint8, device="cuda")
    assert call_ws(fresh, a[:m2], w, 1, m2, K, N, so2, sl2, sr2, ws2) == 0
    assert torch.equal(second, fresh)
