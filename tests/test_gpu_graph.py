"""The entry points launch on the caller's stream without allocating or synchronising, so a
sequence of them can be captured in a HIP graph: a decode-like chain (u8 embedding lookup, u8
GEMV, fp16 matmul with an epilogue, fused attention, softmax_rows) is captured once and replayed
several times, with eager work and synchronisations between the replays, and every replay must
reproduce the eager result bit for bit."""
import numpy as np
import pytest
import torch

from adrastea_amd import (GpuKernels, TensorView, MatmulOptions, MatmulStore, MatmulMask)

pytestmark = pytest.mark.gpu


def test_graph_replays_equal_eager():
    k = GpuKernels()
    gen = torch.Generator(device="cuda").manual_seed(21)
    vocab, dim, heads, S = 512, 512, 4, 128
    hd = dim // heads
    table = torch.randint(0, 256, (vocab, dim), generator=gen, device="cuda", dtype=torch.uint8)
    tscale = (torch.rand(vocab, dim // 32, generator=gen, device="cuda") * 0.02 + 0.001).half()
    ids = torch.randint(0, vocab, (S,), generator=gen, device="cuda").to(torch.int16)
    wq = torch.randint(0, 256, (3 * dim, dim), generator=gen, device="cuda", dtype=torch.uint8)
    wscale = (torch.rand(3 * dim, dim // 32, generator=gen, device="cuda") * 0.004 + 0.001).half()
    wo = (torch.randn(dim, dim, generator=gen, device="cuda") * 0.05).half()
    x = torch.zeros(S, dim, dtype=torch.float16, device="cuda")
    qkv = torch.zeros(S, 3 * dim, dtype=torch.float16, device="cuda")
    q, kk, v = (torch.zeros(S, dim, dtype=torch.float16, device="cuda") for _ in range(3))
    att = torch.zeros(S, dim, dtype=torch.float16, device="cuda")
    hidden = torch.zeros(S, dim, dtype=torch.float16, device="cuda")
    probs = torch.zeros(heads, 16, S, dtype=torch.float16, device="cuda")

    def hv(t):
        return TensorView.of(t).shape_cast([S, heads, -1]).permute([1, 0, 2])

    def chain():
        k.embed_uint8(x, ids, table, tscale, 32)
        k.matmul_nt_fp16u8(qkv, x, wq, wscale, 32)
        q.copy_(qkv[:, :dim]); kk.copy_(qkv[:, dim:2 * dim]); v.copy_(qkv[:, 2 * dim:])
        k.attention_f16(hv(att), hv(q), hv(kk), hv(v), 1.0 / hd ** 0.5, 1.0, MatmulMask.CAUSAL)
        hidden.copy_(x)
        k.matmul_f16(TensorView.of(hidden), TensorView.of(att), TensorView.of(wo).permute([1, 0]),
                     MatmulOptions.new().store(MatmulStore.Add()))
        probs.copy_(hidden[:16 * heads].reshape(heads, 16, dim)[:, :, :S])
        k.softmax_rows_inplace(TensorView.of(probs), 0.7)

    chain()
    torch.cuda.synchronize()
    want = [t.clone() for t in (x, qkv, att, hidden, probs)]
    assert all(torch.isfinite(t.float()).all() for t in want)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()
    for replay in range(4):
        for t in (x, qkv, att, hidden, probs):
            t.fill_(float(replay))                       # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref in zip((x, qkv, att, hidden, probs), want):
            assert torch.equal(got, ref), replay


def test_three_launch_attention_of_an_odd_length_replays_equal_eager():
    """The separate launches of llama.rs:541-554 at a sequence length that is no multiple of 8
    (score rows at any even address): causal score product (its fill launch and the persistent
    kernel), softmax_rows in place, P.V through the kernel that shifts its left operand into place
    -- captured once, replayed with eager work in between, bit for bit the eager result and close
    to the fused launch."""
    k = GpuKernels()
    gen = torch.Generator(device="cuda").manual_seed(22)
    heads, S, hd = 32, 1001, 128
    dim = heads * hd
    q, kk, v = (torch.randn(S, dim, generator=gen, device="cuda", dtype=torch.float16) for _ in range(3))
    scores = torch.zeros(heads, S, S, dtype=torch.float16, device="cuda")
    out = torch.zeros(S, dim, dtype=torch.float16, device="cuda")

    def hv(t):
        return TensorView.of(t).shape_cast([S, heads, -1]).permute([1, 0, 2])

    def chain():
        k_view = TensorView.of(kk).shape_cast([S, heads, -1]).permute([1, 2, 0])
        k.matmul_f16(TensorView.of(scores), hv(q), k_view,
                     MatmulOptions.new().store(MatmulStore.Scale(1.0 / hd ** 0.5)).mask(MatmulMask.CAUSAL))
        k.softmax_rows_inplace(TensorView.of(scores), 1.0)
        k.matmul_f16(hv(out), TensorView.of(scores), hv(v), MatmulOptions.new())

    chain()
    torch.cuda.synchronize()
    want_scores, want_out = scores.clone(), out.clone()
    fused = torch.zeros_like(out)
    k.attention_f16(hv(fused), hv(q), hv(kk), hv(v), 1.0 / hd ** 0.5, 1.0, MatmulMask.CAUSAL)
    torch.cuda.synchronize()
    assert (fused.float() - want_out.float()).abs().max().item() <= 4e-3

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        chain()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        chain()
    for replay in range(3):
        scores.fill_(float(replay))
        out.fill_(float(replay))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(scores, want_scores), replay
        assert torch.equal(out, want_out), replay
