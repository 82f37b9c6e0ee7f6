"""GPU parity of adr_error_stats_f16 / _f32 against the CPU oracle and the reference's kernels
(oracle/_ref/error_stats.co).  Sums are fp32 with atomics on both sides, hence a relative
tolerance of 1e-5 on the two means; the maximum is exact."""
import numpy as np
import pytest
import torch

import oracle
import refgpu
from adrastea_amd import GpuKernels, TensorView, _ffi
from gpu_common import to_dev, to_np
from helpers import rng

pytestmark = pytest.mark.gpu
RTOL = 1e-5


@pytest.fixture(scope="module")
def kern():
    return GpuKernels()


@pytest.fixture(scope="module")
def ref():
    if not refgpu.has("error_stats.co"):
        pytest.skip("oracle/_ref/error_stats.co not built")
    return refgpu.RefKernels()


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("n", [128, 1000, 128 * 257, 128 * 4096 + 5, 3_000_001])
def test_error_stats_match_oracle_and_reference(kern, ref, dtype, n):
    g = rng(910 + n % 1000)
    a = g.standard_normal(n).astype(dtype)
    b = (a.astype(np.float64) + g.standard_normal(n) * 0.02).astype(dtype)
    b[n // 3] += dtype(4.0)          # a clear maximum inside the visited range
    b[n - 1] += dtype(100.0)         # the last element: visited only when n % 128 == 0
    want = oracle.error_stats(a, b)
    a_t, b_t = to_dev(a), to_dev(b)
    out = torch.zeros(3, dtype=torch.float32, device="cuda")
    fn = kern.error_stats_f32 if dtype == np.float32 else kern.error_stats_f16
    fn(TensorView.of(out), TensorView.of(a_t), TensorView.of(b_t))
    got = to_np(out)
    assert got[1] == want[1]
    assert np.allclose(got[[0, 2]], want[[0, 2]], rtol=RTOL)
    o_ref = torch.zeros(3, dtype=torch.float32, device="cuda")
    ref.error_stats(o_ref, a_t, b_t)
    torch.cuda.synchronize()
    r = to_np(o_ref)
    assert r[1] == got[1] and np.allclose(r[[0, 2]], got[[0, 2]], rtol=RTOL)
    # accumulation into a caller-owned output: a second call adds the means, keeps the maximum
    fn(TensorView.of(out), TensorView.of(a_t), TensorView.of(b_t))
    got2 = to_np(out)
    assert got2[1] == want[1] and np.allclose(got2[[0, 2]], 2 * want[[0, 2]], rtol=RTOL)


def test_error_stats_views_and_errors(kern):
    # matrices are flattened with shape_cast([-1]) as in kernels.rs:717-751
    x = torch.randn(64, 130, device="cuda").half()
    y = x.clone()
    y[10, 7] += 1.0
    out = torch.zeros(3, dtype=torch.float32, device="cuda")
    kern.error_stats_f16(TensorView.of(out), TensorView.of(x), TensorView.of(y))
    want = oracle.error_stats(to_np(x), to_np(y))
    assert np.allclose(to_np(out), want, rtol=RTOL)
    with pytest.raises(AssertionError):
        kern.error_stats_f16(TensorView.of(out), TensorView.of(x), TensorView.of(y[:32]))
    lib = _ffi.lib()
    d = _ffi.TensorDesc()
    d.dims = 2
    assert lib.adr_error_stats_f16(None, d, d, d) == -1


def test_error_stats_validates_a_full_size_product_on_the_device(kern):
    """The use the reference makes of it (clip.rs:896-942): compare a 268 MB result with a second
    computation without copying either to the host -- here QK^T from the MFMA kernel against the
    step-for-step slow kernel on four heads."""
    S, H, D = 2048, 4, 128
    HD = H * D
    gen = torch.Generator(device="cuda").manual_seed(47)
    q = torch.randn(S, HD, generator=gen, device="cuda").half()
    k = torch.randn(S, HD, generator=gen, device="cuda").half()
    fast = torch.zeros(H, S, S, dtype=torch.float16, device="cuda")
    slow = torch.zeros(H, S, S, dtype=torch.float16, device="cuda")
    lib = _ffi.lib()
    st = torch.cuda.current_stream().cuda_stream
    for fn, o in ((lib.adr_matmul_f16, fast), (lib.adr_matmul_f16_slow, slow)):
        assert fn(st, o.data_ptr(), q.data_ptr(), k.data_ptr(), H, S, D, S, 1, S, S * S, 1, HD, D,
                  HD, 1, D, None, 0.0, 0.0883883, 4, 0, 0) == 0
    out = torch.zeros(3, dtype=torch.float32, device="cuda")
    kern.error_stats_f16(TensorView.of(out), TensorView.of(fast), TensorView.of(slow))
    mse, mx, mae = to_np(out)
    assert mx <= 0.02 and mae <= 1e-3 and mse <= 1e-5   # scores ~ N(0,1): fp16 steps apart
