"""GPU parity of adr_attention_f16 (the fused QK^T / softmax / P.V launch) through the C ABI and
the host mirror: against the CPU oracle's float64 attention, against the oracle's restatement of
the reference's three-call sequence (llama.rs:541-554), and against this library's own three
kernels on the full LLaMA-7B shape."""
import numpy as np
import pytest
import torch

import oracle
from adrastea_amd import (GpuKernels, TensorView, MatmulOptions, MatmulStore, MatmulMask, _ffi,
                          AdrasteaError)
from gpu_common import to_dev, to_np
from helpers import rng, randn_f16

pytestmark = pytest.mark.gpu

# tolerance: fp16 output rounding plus the fp16 rounding of the probabilities, relative to the
# largest output magnitude; an order of magnitude inside the 1e-2 bound of the matmul tests
TOL = 2e-3


@pytest.fixture(scope="module")
def kern():
    return GpuKernels()


def rel(got, want):
    want = want.astype(np.float64)
    return np.abs(got.astype(np.float64) - want).max() / max(np.abs(want).max(), 1e-30)


# (heads, m, n, d, causal, temp)
CASES = [
    (1, 1, 1, 64, False, 1.0), (2, 32, 64, 128, False, 1.0), (2, 128, 128, 128, True, 1.0),
    (3, 77, 77, 64, True, 1.0),           # CLIP text tower: ragged rows and keys, causal
    (2, 257, 257, 64, False, 1.0),        # CLIP vision tower
    (1, 200, 330, 128, False, 0.7),       # m != n, temperature
    (2, 330, 200, 128, True, 1.0),        # more query rows than keys under the mask
    (2, 130, 321, 128, True, 1.3),        # keys beyond the diagonal are all masked
    (4, 384, 384, 128, True, 1.0), (1, 1, 500, 128, False, 1.0), (1, 5, 1500, 64, False, 1.0),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "h%d_m%d_n%d_d%d_%s_t%g" % (
    c[0], c[1], c[2], c[3], "causal" if c[4] else "full", c[5]))
def test_attention_matches_oracle(kern, case):
    heads, m, n, d, causal, temp = case
    g = rng(4000 + m * 7 + n)
    q, k, v = randn_f16(g, (heads, m, d)), randn_f16(g, (heads, n, d)), randn_f16(g, (heads, n, d))
    scale = 1.0 / np.sqrt(d)
    mask = oracle.MASK_CAUSAL if causal else oracle.MASK_NONE
    exact = oracle.attention_f16(q, k, v, scale, temp, mask, exact=True)
    steps = oracle.attention_f16(q, k, v, scale, temp, mask, threads=8)
    out = torch.full((heads, m, d), 7.0, dtype=torch.float16, device="cuda")
    kern.attention_f16(TensorView.of(out), TensorView.of(to_dev(q)), TensorView.of(to_dev(k)),
                       TensorView.of(to_dev(v)), scale, temp, mask)
    got = to_np(out)
    assert np.isfinite(got).all()
    assert rel(got, exact) <= TOL
    assert rel(got, steps) <= 2 * TOL
    # keeping the scores unrounded must not lose accuracy against the three-call sequence
    assert rel(got, exact) <= rel(steps, exact) + 1e-3


def test_attention_llama_views_and_closed_forms(kern):
    # q, k, v as the [S, heads * hd] projections, viewed per head like llama.rs:534-540
    S, heads, hd = 192, 4, 128
    g = rng(77)
    q, k, v = (randn_f16(g, (S, heads * hd)) for _ in range(3))
    qt, kt, vt = to_dev(q), to_dev(k), to_dev(v)
    out = torch.zeros(S, heads * hd, dtype=torch.float16, device="cuda")

    def hv(t):
        return TensorView.of(t).shape_cast([S, heads, -1]).permute([1, 0, 2])
    scale = 1.0 / np.sqrt(hd)
    kern.attention_f16(hv(out), hv(qt), hv(kt), hv(vt), scale, 1.0, MatmulMask.CAUSAL)
    per_head = lambda a: np.ascontiguousarray(a.reshape(S, heads, hd).transpose(1, 0, 2))
    want = oracle.attention_f16(per_head(q), per_head(k), per_head(v), scale, 1.0,
                                oracle.MASK_CAUSAL, exact=True)
    got = per_head(to_np(out))
    assert rel(got, want) <= TOL
    # under the causal mask the first query row sees only key 0: the output is value row 0
    assert np.array_equal(got[:, 0, :], per_head(v)[:, 0, :])
    # equal scores (zero queries): the output is the mean of the value rows
    zero_q = torch.zeros_like(qt)
    kern.attention_f16(hv(out), hv(zero_q), hv(kt), hv(vt), scale, 1.0, MatmulMask.NONE)
    mean = per_head(v).astype(np.float64).mean(axis=1, keepdims=True)
    assert np.abs(per_head(to_np(out)) - mean).max() <= 1e-3
    # one key that dominates every other: the output is its value row
    k_dom = k.copy()
    k_dom[17, :] = 12.0
    q_pos = np.abs(q)
    kern.attention_f16(hv(out), hv(to_dev(q_pos)), hv(to_dev(k_dom)), hv(vt), 1.0, 1.0,
                       MatmulMask.NONE)
    assert np.array_equal(per_head(to_np(out)), np.broadcast_to(per_head(v)[:, 17:18, :],
                                                                (heads, S, hd)))


def test_attention_errors():
    lib = _ffi.lib()
    x = torch.zeros(2, 64, 128, dtype=torch.float16, device="cuda")
    p = x.data_ptr()

    def call(heads=2, m=64, n=64, d=128, so=(1, 128, 8192), sq=(1, 128, 8192), sk=(1, 128, 8192),
             sv=(1, 128, 8192), scale=0.1, temp=1.0, mask=0, ptrs=(p, p, p, p)):
        return lib.adr_attention_f16(None, *ptrs, heads, m, n, d, *so, *sq, *sk, *sv, scale, temp,
                                     mask)
    assert call() == 0
    assert call(heads=0) == 0 and call(m=0) == 0
    assert call(n=0) == _ffi.ADR_EINVAL_SHAPE
    assert call(m=-1) == _ffi.ADR_EINVAL_SHAPE
    assert call(mask=2) == _ffi.ADR_EINVAL_ENUM
    assert call(ptrs=(p, None, p, p)) == _ffi.ADR_ENULL
    assert call(d=96) == _ffi.ADR_EUNSUPPORTED_LAYOUT
    assert call(sk=(128, 1, 8192)) == _ffi.ADR_EUNSUPPORTED_LAYOUT      # transposed keys
    assert call(sq=(1, 132, 8192)) == _ffi.ADR_EUNSUPPORTED_LAYOUT      # rows not 16-byte aligned
    assert call(ptrs=(p, p + 2, p, p)) == _ffi.ADR_EUNSUPPORTED_LAYOUT
    assert call(temp=0.0) == _ffi.ADR_EUNSUPPORTED_LAYOUT
    torch.cuda.synchronize()
    x96 = torch.zeros(2, 64, 96, dtype=torch.float16, device="cuda")
    with pytest.raises(AdrasteaError) as e:
        GpuKernels().attention_f16(TensorView.of(x96), TensorView.of(x96), TensorView.of(x96),
                                   TensorView.of(x96), 0.1)
    assert e.value.code == _ffi.ADR_EUNSUPPORTED_LAYOUT


def test_attention_full_size_against_three_kernels(kern):
    """LLaMA-7B prefill, 32 heads x 2048 x 2048 x 128, causal: the fused launch against this
    library's own QK^T / softmax_rows / P.V sequence, compared on the device with error_stats."""
    S, heads, hd = 2048, 32, 128
    gen = torch.Generator(device="cuda").manual_seed(5)
    q, k, v = (torch.randn(S, heads * hd, generator=gen, device="cuda", dtype=torch.float16)
               for _ in range(3))

    def hv(t):
        return TensorView.of(t).shape_cast([S, heads, -1]).permute([1, 0, 2])
    scale = 1.0 / hd ** 0.5
    scores = torch.zeros(heads, S, S, dtype=torch.float16, device="cuda")
    k_view = TensorView.of(k).shape_cast([S, heads, -1]).permute([1, 2, 0])
    kern.matmul_f16(TensorView.of(scores), hv(q), k_view,
                    MatmulOptions.new().store(MatmulStore.Scale(scale)).mask(MatmulMask.CAUSAL))
    kern.softmax_rows_inplace(TensorView.of(scores), 1.0)
    three = torch.zeros(S, heads * hd, dtype=torch.float16, device="cuda")
    kern.matmul_f16(hv(three), TensorView.of(scores), hv(v), MatmulOptions.new())
    fused = torch.zeros(S, heads * hd, dtype=torch.float16, device="cuda")
    kern.attention_f16(hv(fused), hv(q), hv(k), hv(v), scale, 1.0, MatmulMask.CAUSAL)
    stats = torch.zeros(3, dtype=torch.float32, device="cuda")
    kern.error_stats_f16(TensorView.of(stats), TensorView.of(fused), TensorView.of(three))
    mse, max_abs, mean_abs = stats.tolist()
    assert max_abs <= 4e-3 and mean_abs <= 2e-4, (mse, max_abs, mean_abs)
    # and against float64 on one head's last rows
    h = 31
    qh = q.view(S, heads, hd)[:, h].double()
    kh, vh = k.view(S, heads, hd)[:, h].double(), v.view(S, heads, hd)[:, h].double()
    sc = (qh[-64:] @ kh.T) * float(np.float16(scale))
    sc = sc.masked_fill(torch.arange(S, device="cuda")[None, :] >
                        torch.arange(S - 64, S, device="cuda")[:, None], float("-inf"))
    want = torch.softmax(sc, -1) @ vh
    got = fused.view(S, heads, hd)[-64:, h].double()
    assert (got - want).abs().max().item() <= TOL * want.abs().max().item()
