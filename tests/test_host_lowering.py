"""CPU-only checks of the host-side mirror: the TensorLayout stride algebra (the reference's
own unit tests, adrastea_models/src/tensor.rs:583-664, restated) and the lowering of views +
options to the 22-scalar argument tuple (adrastea_models/src/kernels.rs:821-890)."""
import pytest

from adrastea_amd import TensorLayout, MatmulOptions, MatmulStore, MatmulLoad, MatmulMask
from adrastea_amd.kernels import lower_matmul


def test_row_and_column_major():
    assert TensorLayout.row_major([2, 3, 4]).strides == (12, 4, 1)
    assert TensorLayout.column_major([3, 4]).strides == (1, 4)
    assert TensorLayout.row_major([3, 3]).permute([1, 0]).strides == (1, 3)
    assert TensorLayout.row_major([2, 3, 4]).largest_address() == 23
    with pytest.raises(ValueError):
        TensorLayout((2, 0), (1, 1))
    with pytest.raises(ValueError):
        TensorLayout((2, 2), (2, 0))


def test_shape_cast():  # tensor.rs:599-613
    t = TensorLayout.row_major([4, 4])
    c = t.shape_cast([-1, 8])
    assert c.dims == (2, 8) and c.strides == (8, 1)
    # like the reference, shape_cast forgets a permutation: it only keeps the volume
    assert t.permute([1, 0]).shape_cast([16]).strides == (1,)


def test_shape_cast_must_preserve_volume():  # tensor.rs:619-625 (should_panic)
    with pytest.raises(ValueError):
        TensorLayout.row_major([256]).shape_cast([16, 1])


def test_skip_and_take():  # tensor.rs:627-664
    r = TensorLayout.row_major([256]).shape_cast([16, 16])
    off, sk = r.skip([15, 0])
    assert (off, sk.dims) == (240, (1, 16))
    off, sk = r.skip([1, 0])
    tk = sk.take([1, 16])
    assert off == 16 and tk.dims == (1, 16) and tk.strides == (16, 1)
    assert r.take([-1, 4]).dims == (16, 4)
    with pytest.raises(ValueError):
        r.take([17, 1])


def test_lowering_of_llama_attention_views():
    """llama.rs:534-554 at LLaMA-7B sizes: closed-form strides of the three head views."""
    S, H, D = 2048, 32, 128
    base = TensorLayout.row_major([S, H * D])
    q = base.shape_cast([S, H, -1]).permute([1, 0, 2])
    k = base.shape_cast([S, H, -1]).permute([1, 2, 0])
    v = base.shape_cast([S, H, -1]).permute([1, 0, 2])
    qk = TensorLayout.row_major([H, S, S])
    low = lower_matmul(qk, q, k, MatmulOptions.new().store(MatmulStore.Scale(1 / D ** 0.5))
                       .mask(MatmulMask.CAUSAL))
    assert (low.batches, low.m, low.k, low.n) == (32, 2048, 128, 2048)
    assert low.stride_l == (1, 4096, 128) and low.stride_r == (4096, 1, 128)
    assert low.stride_o == (1, 2048, 2048 * 2048)
    assert (low.store, low.load, low.mask) == (4, 0, 1)
    assert abs(low.scale - 1 / 128 ** 0.5) < 1e-9 and low.beta == 0.0
    low = lower_matmul(v, qk, v, MatmulOptions.new())  # P.V into the strided qkv view
    assert (low.batches, low.m, low.k, low.n) == (32, 2048, 2048, 128)
    assert low.stride_l == (1, 2048, 2048 * 2048)
    assert low.stride_r == (1, 4096, 128) and low.stride_o == (1, 4096, 128)


def test_lowering_rules():
    out, lhs = TensorLayout.row_major([5, 7]), TensorLayout.row_major([5, 3])
    w = TensorLayout.row_major([7, 3]).permute([1, 0])
    low = lower_matmul(out, lhs, w, MatmulOptions.new())
    assert low.batches == 1 and low.stride_o == (1, 7, 0) and low.stride_r == (3, 1, 0)
    assert (low.beta, low.scale, low.store, low.load, low.mask) == (0.0, 1.0, 0, 0, 0)
    # rank-2 operands are broadcast over the output's batches with stride 0 (kernels.rs:868-880)
    low = lower_matmul(TensorLayout.row_major([4, 5, 7]), TensorLayout.row_major([4, 5, 3]), w,
                       MatmulOptions.new())
    assert low.batches == 4 and low.stride_r[2] == 0 and low.stride_l[2] == 15
    # load scale and store scale multiply into ONE float (kernels.rs:837-843)
    o = MatmulOptions.new().load(MatmulLoad.Scale(0.5)).store(MatmulStore.Scale(0.25))
    low = lower_matmul(out, lhs, w, o)
    assert low.scale == 0.125 and (low.store, low.load) == (4, 1)
    # beta only from the Beta* variants (kernels.rs:844-848)
    assert lower_matmul(out, lhs, w, MatmulOptions.new().store(MatmulStore.BetaBias(1.0, None))).beta == 1.0
    assert lower_matmul(out, lhs, w, MatmulOptions.new().store(MatmulStore.BetaGeluBias(0.5, None))).beta == 0.5
    assert lower_matmul(out, lhs, w, MatmulOptions.new().store(MatmulStore.Add())).beta == 0.0
    for bad in ((TensorLayout.row_major([5, 7]), TensorLayout.row_major([5, 4]), w),       # K
                (TensorLayout.row_major([6, 7]), lhs, w),                                   # M
                (TensorLayout.row_major([5, 8]), lhs, w)):                                  # N
        with pytest.raises(AssertionError):
            lower_matmul(*bad, MatmulOptions.new())
