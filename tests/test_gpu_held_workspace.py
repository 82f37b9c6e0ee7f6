"""The workspaces the plain entry points hold themselves (adr_set_held_workspace_limit): products
that adr_matmul_f16_ws splits along K -- and, after adr_set_u8_dequantise_first(1), u8 products that
adr_matmul_nt_fp16u8_ws runs on a matrix dequantised once -- take their buffer from a pool inside
the library when they come through adr_matmul_f16 / adr_matmul_nt_f16 / adr_matmul_nt_fp16u8.
Bars: the same bits as the _ws entry point given a buffer of the same size; one allocation per
(device, stream), growing on demand, none under stream capture, none with the limit at 0; buffers
given back by adr_release_held_workspace*, a bounded pool however many streams come and go."""
import ctypes as C

import numpy as np
import pytest
import torch

from adrastea_amd import _ffi
from helpers import rng, randn_f16

pytestmark = pytest.mark.gpu

MIB = 1 << 20


@pytest.fixture
def held_on():
    lib = _ffi.lib()
    torch.cuda.synchronize()
    assert lib.adr_release_held_workspace_all() == 0   # every test starts from an empty pool
    lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
    yield lib
    lib.adr_set_held_workspace_limit(0)
    lib.adr_set_u8_dequantise_first(0)
    torch.cuda.synchronize()
    assert lib.adr_release_held_workspace_all() == 0
    assert lib.adr_held_workspace_bytes() == 0


def _nt_args(o, a, w, M, K, N, store=0, bias=None, beta=0.0):
    return (o.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N, 1, N, 0, 1, K, 0, K, 1, 0,
            bias.data_ptr() if bias is not None else None, beta, 1.0, store, 0, 0)


def _plain(lib, stream, *args):
    rc = lib.adr_matmul_f16(stream, *args)
    assert rc == 0, _ffi.strerror(rc)


def _need(lib, M, K, N):
    return lib.adr_matmul_f16_workspace_bytes(1, M, K, N, 1, N, 0, 1, K, 0, K, 1, 0, 0, 0, 0)


def test_split_products_through_the_plain_entry_point(held_on):
    lib = held_on
    g = rng(7)
    main = torch.cuda.current_stream().cuda_stream
    for M, K, N in [(128, 11008, 4096), (70, 6080, 1000), (640, 22016, 4096), (200, 8192, 2048)]:
        need = _need(lib, M, K, N)
        assert need > 0, (M, K, N)
        a = torch.from_numpy(randn_f16(g, (M, K))).cuda()
        w = torch.from_numpy(randn_f16(g, (N, K), K ** -0.5)).cuda()
        o_plain = torch.zeros(M, N, dtype=torch.float16, device="cuda")
        o_ws = torch.zeros_like(o_plain)
        o_off = torch.zeros_like(o_plain)
        before = lib.adr_held_workspace_bytes()
        _plain(lib, main, *_nt_args(o_plain, a, w, M, K, N))
        grown = lib.adr_held_workspace_bytes() - before
        # the same call with a caller's buffer of the size the cache holds
        size = max(16 * MIB, 1 << (need - 1).bit_length())
        ws = torch.empty(size, dtype=torch.uint8, device="cuda")
        rc = lib.adr_matmul_f16_ws(main, *_nt_args(o_ws, a, w, M, K, N), ws.data_ptr(), size)
        assert rc == 0
        lib.adr_set_held_workspace_limit(0)
        _plain(lib, main, *_nt_args(o_off, a, w, M, K, N))
        lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
        torch.cuda.synchronize()
        assert grown in (0, 16 * MIB, 32 * MIB, 64 * MIB, 128 * MIB)
        assert torch.equal(o_plain.view(torch.int16), o_ws.view(torch.int16)), (M, K, N)
        ref = a.double() @ w.double().t()
        scale = ref.pow(2).mean().sqrt()
        assert float((o_plain.double() - ref).abs().max() / scale) < 1e-2
        assert float((o_off.double() - ref).abs().max() / scale) < 1e-2
    # exact inputs, in-place operators: bit for bit whatever the split
    M, K, N = 96, 11008, 4096
    a = torch.from_numpy(g.integers(-3, 4, size=(M, K)).astype(np.float16)).cuda()
    w = torch.from_numpy(g.integers(-2, 3, size=(N, K)).astype(np.float16)).cuda()
    bias = torch.from_numpy((g.integers(-8, 9, size=N) / 4.0).astype(np.float16)).cuda()
    prev = torch.from_numpy((g.integers(-8, 9, size=(M, N)) / 4.0).astype(np.float16)).cuda()
    for store, beta in ((5, 0.0), (3, 0.5), (4, 0.0)):   # Add, BetaBias, Scale
        o_on, o_off = prev.clone(), prev.clone()
        _plain(lib, main, *_nt_args(o_on, a, w, M, K, N, store=store, bias=bias, beta=beta))
        lib.adr_set_held_workspace_limit(0)
        _plain(lib, main, *_nt_args(o_off, a, w, M, K, N, store=store, bias=bias, beta=beta))
        lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
        torch.cuda.synchronize()
        assert torch.equal(o_on.view(torch.int16), o_off.view(torch.int16)), store


def test_one_buffer_per_stream_growing_on_demand(held_on):
    lib = held_on
    g = rng(8)
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    small, large = (70, 6080, 1000), (640, 22016, 4096)
    assert 0 < _need(lib, *small) <= 16 * MIB < _need(lib, *large)
    ops = {}
    for M, K, N in (small, large):
        ops[(M, K, N)] = (torch.from_numpy(randn_f16(g, (M, K))).cuda(),
                          torch.from_numpy(randn_f16(g, (N, K), K ** -0.5)).cuda(),
                          torch.zeros(M, N, dtype=torch.float16, device="cuda"))
    torch.cuda.synchronize()

    def call(stream, shape):
        a, w, o = ops[shape]
        _plain(lib, stream.cuda_stream, *_nt_args(o, a, w, *shape))

    base = lib.adr_held_workspace_bytes()
    call(s1, small)
    assert lib.adr_held_workspace_bytes() == base + 16 * MIB      # first use on s1
    call(s1, small)
    assert lib.adr_held_workspace_bytes() == base + 16 * MIB      # reused
    call(s2, small)
    assert lib.adr_held_workspace_bytes() == base + 32 * MIB      # s2 has its own
    call(s1, large)
    grown = lib.adr_held_workspace_bytes() - base - 32 * MIB
    assert grown in (32 * MIB, 64 * MIB, 128 * MIB)               # replaced by a larger one
    call(s1, small)
    call(s1, large)
    assert lib.adr_held_workspace_bytes() == base + 32 * MIB + grown
    torch.cuda.synchronize()
    for shape in (small, large):
        a, w, o = ops[shape]
        ref = a.double() @ w.double().t()
        assert float((o.double() - ref).abs().max() / ref.pow(2).mean().sqrt()) < 1e-2
    # a limit below what the product asks for: fewer pieces or none, no buffer above the limit
    for limit in (20 * MIB, 4 * MIB):
        lib.adr_set_held_workspace_limit(limit)
        s3 = torch.cuda.Stream()
        before = lib.adr_held_workspace_bytes()
        call(s3, large)
        assert lib.adr_held_workspace_bytes() - before <= limit
        torch.cuda.synchronize()
    # off: nothing is allocated
    lib.adr_set_held_workspace_limit(0)
    s4 = torch.cuda.Stream()
    before = lib.adr_held_workspace_bytes()
    call(s4, large)
    torch.cuda.synchronize()
    assert lib.adr_held_workspace_bytes() == before


def test_nothing_is_held_under_capture(held_on):
    lib = held_on
    g = rng(9)
    M, K, N = 128, 11008, 4096
    a = torch.from_numpy(randn_f16(g, (M, K))).cuda()
    w = torch.from_numpy(randn_f16(g, (N, K), K ** -0.5)).cuda()
    o_graph = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    o_off = torch.zeros_like(o_graph)
    lib.adr_set_held_workspace_limit(0)
    _plain(lib, torch.cuda.current_stream().cuda_stream, *_nt_args(o_off, a, w, M, K, N))
    lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
    torch.cuda.synchronize()
    before = lib.adr_held_workspace_bytes()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _plain(lib, torch.cuda.current_stream().cuda_stream, *_nt_args(o_graph, a, w, M, K, N))
    assert lib.adr_held_workspace_bytes() == before
    for _ in range(3):
        o_graph.zero_()
        graph.replay()
        torch.cuda.synchronize()
        # the captured launch is the unsplit one
        assert torch.equal(o_graph.view(torch.int16), o_off.view(torch.int16))


def test_u8_products_by_way_of_the_held_workspace(held_on):
    lib = held_on
    g = rng(10)
    main = torch.cuda.current_stream().cuda_stream
    # the default: the fused kernels whatever the pool would allow, nothing allocated
    m, p, n, bs = 800, 4096, 4096, 32
    q = torch.from_numpy(g.integers(0, 256, size=(n, p), dtype=np.uint8)).cuda()
    sc = torch.from_numpy((g.random((n, p // bs)) * 0.019 + 0.001).astype(np.float16)).cuda()
    x = torch.from_numpy(randn_f16(g, (m, p))).cuda()
    o_default = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    o_fused = torch.zeros_like(o_default)
    assert lib.adr_u8_dequantise_first() == 0
    name = C.create_string_buffer(96)
    assert lib.adr_matmul_nt_fp16u8_plan(name, 96, m, p, n, bs) == 0 and name.value.startswith(b"gemm_nt_u8")
    assert lib.adr_matmul_nt_fp16u8(main, o_default.data_ptr(), x.data_ptr(), q.data_ptr(), sc.data_ptr(), m, p, n, bs, 0.0) == 0
    lib.adr_set_held_workspace_limit(0)
    assert lib.adr_matmul_nt_fp16u8(main, o_fused.data_ptr(), x.data_ptr(), q.data_ptr(), sc.data_ptr(), m, p, n, bs, 0.0) == 0
    lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
    torch.cuda.synchronize()
    assert torch.equal(o_default.view(torch.int16), o_fused.view(torch.int16))
    assert lib.adr_held_workspace_bytes() == 0
    # on request: the matrix dequantised once into a buffer of the pool
    assert lib.adr_set_u8_dequantise_first(1) == 0 and lib.adr_u8_dequantise_first() == 1
    assert lib.adr_matmul_nt_fp16u8_plan(name, 96, m, p, n, bs) == 0 and name.value == b"dequantize_absmax_u8 + fp16 gemm"
    for m, p, n, bs in [(800, 4096, 4096, 32), (2048, 4096, 4096, 32), (768, 4096, 8192, 32), (1100, 1024, 5120, 64),
                        (1000, 11008, 4096, 32)]:
        need = lib.adr_matmul_nt_fp16u8_workspace_bytes(m, p, n, bs)
        assert need == n * p * 2
        q = torch.from_numpy(g.integers(0, 256, size=(n, p), dtype=np.uint8)).cuda()
        sc = torch.from_numpy((g.random((n, p // bs)) * 0.019 + 0.001).astype(np.float16)).cuda()
        x = torch.from_numpy(randn_f16(g, (m, p))).cuda()
        o_held = torch.zeros(m, n, dtype=torch.float16, device="cuda")
        o_ws = torch.zeros_like(o_held)
        o_fused = torch.zeros_like(o_held)
        rc = lib.adr_matmul_nt_fp16u8(main, o_held.data_ptr(), x.data_ptr(), q.data_ptr(), sc.data_ptr(), m, p, n, bs, 0.0)
        assert rc == 0
        # (a caller's buffer of the cache's limit; only the matrix's n * p * 2 bytes are used)
        ws = torch.empty(_ffi.HELD_WORKSPACE_DEFAULT_BYTES, dtype=torch.uint8, device="cuda")
        rc = lib.adr_matmul_nt_fp16u8_ws(main, o_ws.data_ptr(), x.data_ptr(), q.data_ptr(), sc.data_ptr(), m, p, n, bs, 0.0,
                                         ws.data_ptr(), ws.numel())
        assert rc == 0
        lib.adr_set_held_workspace_limit(0)
        rc = lib.adr_matmul_nt_fp16u8(main, o_fused.data_ptr(), x.data_ptr(), q.data_ptr(), sc.data_ptr(), m, p, n, bs, 0.0)
        assert rc == 0
        lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
        torch.cuda.synchronize()
        assert torch.equal(o_held.view(torch.int16), o_ws.view(torch.int16)), (m, p, n)
        wd = torch.empty(n, p, dtype=torch.float16, device="cuda")
        assert lib.adr_dequantize_absmax_u8(main, wd.data_ptr(), q.data_ptr(), sc.data_ptr(), n, p, bs) == 0
        ref = x.double() @ wd.double().t()
        scale = ref.pow(2).mean().sqrt()
        assert float((o_held.double() - ref).abs().max() / scale) < 1e-2  # (fp16 output: half a step at 4 x RMS is 2e-3)
        assert float((o_fused.double() - ref).abs().max() / scale) < 1e-2
    # a matrix that needs more than the limit stays on the fused kernels and allocates nothing
    lib.adr_set_held_workspace_limit(8 * MIB)
    before = lib.adr_held_workspace_bytes()
    s = torch.cuda.Stream()
    m, p, n, bs = 800, 4096, 4096, 32
    q = torch.from_numpy(g.integers(0, 256, size=(n, p), dtype=np.uint8)).cuda()
    sc = torch.from_numpy((g.random((n, p // bs)) * 0.019 + 0.001).astype(np.float16)).cuda()
    x = torch.from_numpy(randn_f16(g, (m, p))).cuda()
    o = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    assert lib.adr_matmul_nt_fp16u8(s.cuda_stream, o.data_ptr(), x.data_ptr(), q.data_ptr(), sc.data_ptr(), m, p, n, bs, 0.0) == 0
    torch.cuda.synchronize()
    assert lib.adr_held_workspace_bytes() == before


def test_threads_on_their_own_streams(held_on):
    import threading
    lib = held_on
    g = rng(11)
    M, K, N = 128, 11008, 4096
    a = torch.from_numpy(randn_f16(g, (M, K))).cuda()
    w = torch.from_numpy(randn_f16(g, (N, K), K ** -0.5)).cuda()
    streams = [torch.cuda.Stream() for _ in range(4)]
    outs = [torch.zeros(M, N, dtype=torch.float16, device="cuda") for _ in streams]
    torch.cuda.synchronize()
    errors = []

    def work(i):
        try:
            for _ in range(20):
                _plain(lib, streams[i].cuda_stream, *_nt_args(outs[i], a, w, M, K, N))
        except Exception as e:  # noqa: BLE001
            errors.append(e)
    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(streams))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors
    for o in outs[1:]:
        assert torch.equal(o.view(torch.int16), outs[0].view(torch.int16))
    ref = a.double() @ w.double().t()
    assert float((outs[0].double() - ref).abs().max() / ref.pow(2).mean().sqrt()) < 1e-2


def test_release_gives_the_memory_back_and_later_calls_allocate_afresh(held_on):
    lib = held_on
    g = rng(12)
    M, K, N = 128, 11008, 4096
    a = torch.from_numpy(randn_f16(g, (M, K))).cuda()
    w = torch.from_numpy(randn_f16(g, (N, K), K ** -0.5)).cuda()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    o1 = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    o2, o3 = torch.zeros_like(o1), torch.zeros_like(o1)
    torch.cuda.synchronize()
    _plain(lib, s1.cuda_stream, *_nt_args(o1, a, w, M, K, N))
    _plain(lib, s2.cuda_stream, *_nt_args(o2, a, w, M, K, N))
    assert lib.adr_held_workspace_bytes() == 32 * MIB
    # released right behind the launch: the call waits for the buffer's last use, not for the caller
    assert lib.adr_release_held_workspace(s1.cuda_stream) == 0
    assert lib.adr_held_workspace_bytes() == 16 * MIB          # s2 keeps its own
    assert lib.adr_release_held_workspace(s1.cuda_stream) == 0  # nothing left to release: fine
    _plain(lib, s1.cuda_stream, *_nt_args(o3, a, w, M, K, N))   # allocates afresh
    assert lib.adr_held_workspace_bytes() == 32 * MIB
    torch.cuda.synchronize()
    assert torch.equal(o1.view(torch.int16), o2.view(torch.int16))
    assert torch.equal(o1.view(torch.int16), o3.view(torch.int16))
    assert lib.adr_release_held_workspace_all() == 0
    assert lib.adr_held_workspace_bytes() == 0


def test_streams_that_come_and_go_leave_a_bounded_pool(held_on):
    lib = held_on
    g = rng(13)
    M, K, N = 128, 11008, 4096
    a = torch.from_numpy(randn_f16(g, (M, K))).cuda()
    w = torch.from_numpy(randn_f16(g, (N, K), K ** -0.5)).cuda()
    want = torch.zeros(M, N, dtype=torch.float16, device="cuda")
    _plain(lib, torch.cuda.current_stream().cuda_stream, *_nt_args(want, a, w, M, K, N))
    torch.cuda.synchronize()
    declined = lib.adr_held_workspace_declined()
    # a host that releases before it destroys a stream holds nothing afterwards
    base = lib.adr_held_workspace_bytes()
    for _ in range(20):
        s = torch.cuda.Stream()
        o = torch.zeros_like(want)
        _plain(lib, s.cuda_stream, *_nt_args(o, a, w, M, K, N))
        assert lib.adr_release_held_workspace(s.cuda_stream) == 0
        assert lib.adr_held_workspace_bytes() == base
        assert torch.equal(o.view(torch.int16), want.view(torch.int16))
        del s
    # a host that does not: the pool stops at 16 buffers and hands the least recently used one on
    streams, outs = [], []
    for i in range(100):
        s = torch.cuda.Stream()
        o = torch.zeros_like(want) if i % 10 == 0 else outs[-1]
        _plain(lib, s.cuda_stream, *_nt_args(o, a, w, M, K, N))
        streams.append(s)
        outs.append(o)
        assert lib.adr_held_workspace_bytes() <= 16 * 16 * MIB
    torch.cuda.synchronize()
    assert lib.adr_held_workspace_bytes() == 16 * 16 * MIB
    assert lib.adr_held_workspace_declined() == declined       # every call found a buffer
    for o in outs[::10]:
        assert torch.equal(o.view(torch.int16), want.view(torch.int16))
    # the pool is full of 16 MiB buffers: a product that wants more runs without one, and is counted
    big = (640, 22016, 4096)
    assert _need(lib, *big) > 16 * MIB
    ab = torch.from_numpy(randn_f16(g, big[:2])).cuda()
    wb = torch.from_numpy(randn_f16(g, (big[2], big[1]), big[1] ** -0.5)).cuda()
    o_full, o_off = (torch.zeros(big[0], big[2], dtype=torch.float16, device="cuda") for _ in range(2))
    fresh = torch.cuda.Stream()
    torch.cuda.synchronize()
    _plain(lib, fresh.cuda_stream, *_nt_args(o_full, ab, wb, *big))
    assert lib.adr_held_workspace_declined() == declined + 1
    lib.adr_set_held_workspace_limit(0)
    _plain(lib, fresh.cuda_stream, *_nt_args(o_off, ab, wb, *big))
    torch.cuda.synchronize()
    assert torch.equal(o_full.view(torch.int16), o_off.view(torch.int16))
