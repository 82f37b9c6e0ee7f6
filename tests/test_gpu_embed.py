"""GPU parity of adr_embed_uint8 through the C ABI: bit-exact against the CPU oracle and against
the reference's own embed_uint8 kernel (oracle/_ref/embed_uint8.co)."""
import numpy as np
import pytest
import torch

import oracle
import refgpu
from adrastea_amd import GpuKernels, _ffi
from gpu_common import to_dev, to_np
from helpers import rng

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", [(50, 96, 32, 6), (1000, 4096, 32, 77), (300, 4096, 128, 513),
                                  (64, 100, 20, 9), (40, 24, 8, 3), (32000, 128, 32, 2048)],
                         ids=lambda c: "v%d_d%d_bs%d_n%d" % c)
def test_embed_bit_exact(case):
    vocab, n_dim, bs, n_ids = case
    g = rng(vocab + n_dim)
    table = g.integers(0, 256, size=(vocab, n_dim)).astype(np.uint8)
    scales = (g.random((vocab, n_dim // bs)) * 0.02 + 1e-4).astype(np.float16)
    scales[0, 0] = np.float16(6e-8)                    # subnormal scale
    ids = g.integers(0, vocab, size=n_ids).astype(np.int16) if vocab <= 32767 else \
        g.integers(0, 32767, size=n_ids).astype(np.int16)
    ids[0] = 0
    want = oracle.embed_uint8(ids, table, scales, bs)
    t_t, s_t, i_t = to_dev(table), to_dev(scales), to_dev(ids)
    out = torch.full((n_ids, n_dim), 7.0, dtype=torch.float16, device="cuda")
    GpuKernels().embed_uint8(out, i_t, t_t, s_t, bs)
    assert np.array_equal(to_np(out).view(np.uint16), want.view(np.uint16))
    if refgpu.available() and refgpu.has("embed_uint8.co"):
        o_ref = torch.zeros_like(out)
        refgpu.RefKernels().embed_uint8(o_ref, i_t, t_t, s_t, bs)
        torch.cuda.synchronize()
        assert torch.equal(o_ref, out)


def test_embed_errors():
    lib = _ffi.lib()
    assert lib.adr_embed_uint8(None, 96, 0, None, None, None, None, 32) == 0
    assert lib.adr_embed_uint8(None, 96, 4, None, None, None, None, 32) == _ffi.ADR_ENULL
    assert lib.adr_embed_uint8(None, 100, 4, None, None, None, None, 32) == _ffi.ADR_EDIVISIBILITY
    assert lib.adr_embed_uint8(None, -1, 4, None, None, None, None, 32) == _ffi.ADR_EINVAL_SHAPE
