"""adr_matmul_f16_noalloc (the entry point that allocates nothing: its scratch is a fixed array
inside the library's device code) against adr_matmul_f16_ws (the same kernels with a
caller-provided workspace), through the C ABI: bit-identical results on two calls in a row, the
second with a smaller input; a product that would like more than the scratch holds; products
that need no scratch."""
import ctypes as C

import pytest
import torch

from adrastea_amd import _ffi

pytestmark = pytest.mark.gpu


def nt(M, K, N):
    return (1, N, 0), (1, K, 0), (K, 1, 0)


def call(fn_name, out, a, w, M, K, N, bias=None, beta=0.0, store=0, ws=None):
    lib = _ffi.lib()
    so, sl, sr = nt(M, K, N)
    args = [torch.cuda.current_stream().cuda_stream, out.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N,
            *so, *sl, *sr, bias.data_ptr() if bias is not None else None, beta, 1.0, store, 0, 0]
    if ws is not None:
        args += [ws.data_ptr(), ws.numel()]
    return getattr(lib, fn_name)(*args)


def test_noalloc_matches_workspace_entry_point_on_two_calls_in_a_row():
    lib = _ffi.lib()
    K, N = 11008, 4096
    gen = torch.Generator(device="cuda").manual_seed(91)
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    bias = torch.randn(N, generator=gen, device="cuda").half()
    ws = torch.empty(_ffi.NOALLOC_SCRATCH_BYTES, dtype=torch.uint8, device="cuda")
    results = []
    for M in (256, 100):   # the second call is smaller and must not see the first one's partials
        so, sl, sr = nt(M, K, N)
        need = lib.adr_matmul_f16_workspace_bytes(1, M, K, N, *so, *sl, *sr, 3, 0, 0)
        assert 0 < need <= _ffi.NOALLOC_SCRATCH_BYTES   # the scratch is really used
        a = torch.randn(M, K, generator=gen, device="cuda").half()
        prev = torch.randn(M, N, generator=gen, device="cuda").half()
        want = prev.clone()
        assert call("adr_matmul_f16_ws", want, a, w, M, K, N, bias=bias, beta=0.5, store=3, ws=ws) == 0
        got = prev.clone()
        assert call("adr_matmul_f16_noalloc", got, a, w, M, K, N, bias=bias, beta=0.5, store=3) == 0
        torch.cuda.synchronize()
        assert torch.equal(got, want), M
        ref = a.float() @ w.float().t() + bias.float() + 0.5 * prev.float()
        rms = ref.pow(2).mean().sqrt()
        assert ((got.float() - ref).abs() / torch.maximum(ref.abs(), rms)).max().item() <= 2e-3
        results.append(got)
    # the first problem again: same bits as before the smaller call used the scratch
    M = 256
    gen = torch.Generator(device="cuda").manual_seed(91)
    w2 = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    bias2 = torch.randn(N, generator=gen, device="cuda").half()
    a = torch.randn(M, K, generator=gen, device="cuda").half()
    prev = torch.randn(M, N, generator=gen, device="cuda").half()
    again = prev.clone()
    assert call("adr_matmul_f16_noalloc", again, a, w2, M, K, N, bias=bias2, beta=0.5, store=3) == 0
    assert torch.equal(again, results[0])


def test_noalloc_size_limit_and_products_without_scratch():
    lib = _ffi.lib()
    # a product whose best split would need more than the built-in scratch is cut into as many
    # pieces as fit: the result of adr_matmul_f16_ws given a workspace of exactly that size
    M, K, N = 300, 22016, 4096
    so, sl, sr = nt(M, K, N)
    assert lib.adr_matmul_f16_workspace_bytes(1, M, K, N, *so, *sl, *sr, 0, 0, 0) > _ffi.NOALLOC_SCRATCH_BYTES
    name = C.create_string_buffer(96)
    assert lib.adr_matmul_f16_ws_plan(name, 96, 1, M, K, N, *so, *sl, *sr, 0, 0, 0, _ffi.NOALLOC_SCRATCH_BYTES) == 0
    gen = torch.Generator(device="cuda").manual_seed(94)
    a = torch.randn(M, K, generator=gen, device="cuda").half()
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    ws = torch.empty(_ffi.NOALLOC_SCRATCH_BYTES, dtype=torch.uint8, device="cuda")
    want = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    got = torch.zeros_like(want)
    assert call("adr_matmul_f16_ws", want, a, w, M, K, N, ws=ws) == 0
    assert call("adr_matmul_f16_noalloc", got, a, w, M, K, N) == 0
    torch.cuda.synchronize()
    assert torch.equal(got, want), name.value
    ref = a.float() @ w.float().t()
    rms = ref.pow(2).mean().sqrt()
    assert ((got.float() - ref).abs() / torch.maximum(ref.abs(), rms)).max().item() <= 2e-3
    # products that are not split run as adr_matmul_f16 does: prefill, decode, empty
    gen = torch.Generator(device="cuda").manual_seed(92)
    for M, K, N in ((512, 1024, 768), (4, 4096, 4096), (0, 64, 64)):
        a = torch.randn(max(M, 1), K, generator=gen, device="cuda").half()
        w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
        got = torch.zeros(max(M, 1), N, dtype=torch.float16, device="cuda")
        want = torch.zeros_like(got)
        assert call("adr_matmul_f16_noalloc", got, a, w, M, K, N) == 0
        assert call("adr_matmul_f16", want, a, w, M, K, N) == 0
        assert torch.equal(got, want)
    # same validation as the other entry points
    assert lib.adr_matmul_f16_noalloc(None, None, a.data_ptr(), w.data_ptr(), 1, 4, 64, 64, 1, 64, 0, 1, 64, 0,
                                      64, 1, 0, None, 0.0, 1.0, 0, 0, 0) == _ffi.ADR_ENULL
    assert lib.adr_matmul_f16_noalloc(None, got.data_ptr(), a.data_ptr(), w.data_ptr(), 1, 4, 64, 64, 1, 64, 0,
                                      1, 64, 0, 64, 1, 0, None, 0.0, 1.0, 1, 0, 0) == _ffi.ADR_ENOTIMPL


def test_noalloc_in_a_captured_graph():
    """What the entry point is for: a split product (partial tiles in the built-in scratch, then
    the reduction launch) recorded into a HIP graph and replayed, with eager calls that use the
    same scratch for another product and synchronisations between the replays; every replay
    reproduces the eager result bit for bit.  (The first call on a device, which looks the
    scratch address up, is made before the capture.)"""
    K, N, M = 11008, 4096, 200
    gen = torch.Generator(device="cuda").manual_seed(93)
    w = (torch.randn(N, K, generator=gen, device="cuda") * K ** -0.5).half()
    a = torch.randn(M, K, generator=gen, device="cuda").half()
    a2 = torch.randn(96, K, generator=gen, device="cuda").half()
    out = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    other = torch.zeros(96, N, dtype=torch.float16, device="cuda")
    so, sl, sr = nt(M, K, N)
    assert _ffi.lib().adr_matmul_f16_workspace_bytes(1, M, K, N, *so, *sl, *sr, 0, 0, 0) > 0
    assert call("adr_matmul_f16_noalloc", out, a, w, M, K, N) == 0
    torch.cuda.synchronize()
    want = out.clone()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            assert call("adr_matmul_f16_noalloc", out, a, w, M, K, N) == 0
    torch.cuda.current_stream().wait_stream(side)
    for _ in range(3):
        out.zero_()
        assert call("adr_matmul_f16_noalloc", other, a2, w, 96, K, N) == 0   # dirties the scratch
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want)
