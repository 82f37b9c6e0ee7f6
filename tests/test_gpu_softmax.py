"""GPU parity of adr_softmax_rows (through the C ABI and the host mirror) against the CPU oracle
and against the reference's own softmax_rows kernel compiled into oracle/_ref/normalize.co."""
import numpy as np
import pytest
import torch

import oracle
import refgpu
from adrastea_amd import GpuKernels, TensorView, _ffi
from gpu_common import to_dev, to_np
from helpers import rng, ulp_diff_f16

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def kern():
    return GpuKernels()


@pytest.fixture(scope="module")
def ref():
    if not refgpu.available() or not refgpu.has("normalize.co"):
        pytest.skip("oracle/_ref/normalize.co not built")
    return refgpu.RefKernels()


def call(out_t, in_t, heads, h, w, temp):
    return _ffi.lib().adr_softmax_rows(torch.cuda.current_stream().cuda_stream, out_t.data_ptr(),
                                       in_t.data_ptr(), heads, h, w, float(temp))


SHAPES = [(1, 1, 1), (2, 3, 8), (3, 5, 77), (2, 9, 257), (4, 16, 512), (2, 7, 520), (1, 33, 1024),
          (2, 10, 2048), (1, 6, 3000), (1, 5, 4096), (1, 3, 4104), (1, 2, 10000),
          # rows that are not 16-byte aligned: aligned to 8 bytes (1500), 4 bytes (1002), 2 bytes
          (2, 11, 1500), (3, 4, 1002), (1, 9, 2001), (1, 7, 4095)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("temp", [1.0, 0.6])
def test_softmax_matches_oracle_and_reference_kernel(ref, shape, temp):
    heads, h, w = shape
    g = rng(800 + w)
    x = (g.standard_normal((heads, h, w)) * 4).astype(np.float16)
    if w > 4:
        x[0, 0, w // 2:] = -np.inf            # a causally masked tail
    want = oracle.softmax_rows(x, temp, 0)
    want64 = oracle.softmax_rows(x, temp, 1)
    x_t = to_dev(x)
    out = torch.full_like(x_t, 7.0)
    assert call(out, x_t, heads, h, w, temp) == 0
    got = to_np(out)
    assert np.max(ulp_diff_f16(got, want)) <= 1
    assert np.max(ulp_diff_f16(got, want64)) <= 1
    assert np.all(got[x == -np.inf] == 0)
    # the reference's kernel on the same input
    o_ref = torch.zeros_like(x_t)
    ref.softmax_rows(o_ref, x_t, heads, h, w, temp)
    torch.cuda.synchronize()
    assert np.max(ulp_diff_f16(got, to_np(o_ref))) <= 1
    assert np.max(ulp_diff_f16(want, to_np(o_ref))) <= 1   # the oracle restates that kernel
    # in place gives the same bits as out of place
    inplace = x_t.clone()
    assert call(inplace, inplace, heads, h, w, temp) == 0
    assert torch.equal(inplace, out)


@pytest.mark.parametrize("w", [77, 1500, 2001])
def test_softmax_of_a_tensor_that_starts_at_an_odd_element(w):
    """A score tensor inside a larger buffer, its first element at an odd index: the guard
    elements before and behind it keep their bits, in place and out of place."""
    heads, h = 2, 5
    g = rng(830 + w)
    x = (g.standard_normal((heads, h, w)) * 4).astype(np.float16)
    want = oracle.softmax_rows(x, 1.0, 0)
    n = heads * h * w
    buf = torch.full((n + 8,), 5.0, dtype=torch.float16, device="cuda")
    buf[3:3 + n] = to_dev(x).flatten()
    out = torch.full((n + 8,), 9.0, dtype=torch.float16, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    lib = _ffi.lib()
    assert lib.adr_softmax_rows(stream, out.data_ptr() + 2, buf.data_ptr() + 6, heads, h, w, 1.0) == 0
    got = to_np(out)
    assert np.max(ulp_diff_f16(got[1:1 + n].reshape(heads, h, w), want)) <= 1
    assert np.all(got[:1] == 9.0) and np.all(got[1 + n:] == 9.0)
    assert lib.adr_softmax_rows(stream, buf.data_ptr() + 6, buf.data_ptr() + 6, heads, h, w, 1.0) == 0
    got = to_np(buf)
    assert np.max(ulp_diff_f16(got[3:3 + n].reshape(heads, h, w), want)) <= 1
    assert np.all(got[:3] == 5.0) and np.all(got[3 + n:] == 5.0)


def test_softmax_closed_forms_and_errors(kern):
    x = torch.full((2, 4, 1024), 0.37, dtype=torch.float16, device="cuda")
    kern.softmax_rows_inplace(TensorView.of(x), 1.0)
    assert torch.all(x == 1.0 / 1024)
    y = torch.tensor([[0.5, float("-inf"), 0.5, float("-inf")] * 2], dtype=torch.float16, device="cuda")
    kern.softmax_rows_inplace(TensorView.of(y), 1.0)
    assert torch.equal(y, torch.tensor([[0.25, 0, 0.25, 0] * 2], dtype=torch.float16, device="cuda"))
    with pytest.raises(AssertionError):     # the reference kernel ignores strides: contiguous only
        kern.softmax_rows_inplace(TensorView.of(x).permute([0, 2, 1]), 1.0)
    lib = _ffi.lib()
    assert lib.adr_softmax_rows(None, None, None, 1, 1, 8, 1.0) == -4
    assert lib.adr_softmax_rows(None, x.data_ptr(), x.data_ptr(), -1, 1, 8, 1.0) == -1
    assert lib.adr_softmax_rows(None, None, None, 0, 4, 8, 1.0) == 0   # empty: no-op


def test_softmax_full_size_attention_scores(kern):
    """benchmark config 4 size: [32, 2048, 2048] causal scores in place; rows sum to 1, masked
    entries are 0, and a band of rows equals the oracle."""
    H, S = 32, 2048
    gen = torch.Generator(device="cuda").manual_seed(46)
    x = (torch.randn(H, S, S, generator=gen, device="cuda") * 2).half()
    mask = torch.ones(S, S, device="cuda", dtype=torch.bool).triu(1)
    x.masked_fill_(mask, float("-inf"))
    band = x[5, 1000:1016].clone()
    kern.softmax_rows_inplace(TensorView.of(x), 1.0)
    sums = x.float().sum(-1)
    assert torch.all((sums - 1).abs() <= 2e-3)
    assert torch.all(x.masked_select(mask) == 0)
    want = oracle.softmax_rows(to_np(band), 1.0, 0)
    assert np.max(ulp_diff_f16(to_np(x[5, 1000:1016]), want)) <= 1
