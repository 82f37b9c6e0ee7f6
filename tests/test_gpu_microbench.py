"""The microbenchmark entry points (counterparts of adrastea_kernels/cpp/microbench.cu): they are
measurement aids, so the checks are about safety of the arguments and that the matrix-core loop
really multiplies (twice the trips, twice the sums)."""
import pytest
import torch

from adrastea_amd import _ffi

pytestmark = pytest.mark.gpu


def stream():
    return torch.cuda.current_stream().cuda_stream


def test_empty_and_argument_checks():
    L = _ffi.lib()
    assert L.adr_microbench_empty(stream()) == 0
    sink = torch.zeros(256, device="cuda")
    assert L.adr_microbench_mfma_f16(stream(), 0, 1, 0, sink.data_ptr()) == _ffi.ADR_EINVAL_SHAPE
    assert L.adr_microbench_mfma_f16(stream(), 1, 1, 5, sink.data_ptr()) == _ffi.ADR_EINVAL_SHAPE
    assert L.adr_microbench_mfma_f16(stream(), 1, 1, 0, None) == _ffi.ADR_ENULL
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    s32 = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert L.adr_microbench_stream_read(stream(), buf.data_ptr(), (1 << 20) + 8, 64,
                                        s32.data_ptr()) == _ffi.ADR_EINVAL_SHAPE
    assert L.adr_microbench_stream_read(stream(), buf.data_ptr(), 0, 64, s32.data_ptr()) == 0
    assert L.adr_microbench_stream_read(stream(), buf.data_ptr(), 1 << 20, 64, s32.data_ptr()) == 0
    torch.cuda.synchronize()
    assert int(s32.item()) == 0


def test_mfma_loop_multiplies():
    L = _ffi.lib()
    blocks = 3
    one = torch.full((blocks * 256,), -1.0, device="cuda")
    two = torch.full((blocks * 256,), -1.0, device="cuda")
    zero = torch.full((blocks * 256,), -1.0, device="cuda")
    assert L.adr_microbench_mfma_f16(stream(), blocks, 1, 1, one.data_ptr()) == 0
    assert L.adr_microbench_mfma_f16(stream(), blocks, 2, 1, two.data_ptr()) == 0
    assert L.adr_microbench_mfma_f16(stream(), blocks, 5, 0, zero.data_ptr()) == 0
    torch.cuda.synchronize()
    assert torch.all(zero == 0)
    assert torch.isfinite(one).all() and (one != 0).any()
    # (the matrix core adds the 16 products of a step to the accumulator in its own order)
    assert torch.allclose(two, 2 * one, rtol=1e-4, atol=1e-3)
    # the loop whose operands change with every instruction: four trips rotate the four fragments
    # of either operand once around, so eight trips sum every product twice
    r4 = torch.full((blocks * 256,), -1.0, device="cuda")
    r8 = torch.full((blocks * 256,), -1.0, device="cuda")
    assert L.adr_microbench_mfma_f16(stream(), blocks, 4, 2, r4.data_ptr()) == 0
    assert L.adr_microbench_mfma_f16(stream(), blocks, 8, 2, r8.data_ptr()) == 0
    torch.cuda.synchronize()
    assert torch.isfinite(r4).all() and (r4 != 0).any()
    assert torch.allclose(r8, 2 * r4, rtol=1e-4, atol=1e-3)
    # the two MFMA shapes on a 128 x 128 wavefront tile: an iteration sums the same products again
    for pattern in (3, 4):
        t1 = torch.full((blocks * 256,), -1.0, device="cuda")
        t2 = torch.full((blocks * 256,), -1.0, device="cuda")
        assert L.adr_microbench_mfma_f16(stream(), blocks, 1, pattern, t1.data_ptr()) == 0
        assert L.adr_microbench_mfma_f16(stream(), blocks, 2, pattern, t2.data_ptr()) == 0
        torch.cuda.synchronize()
        assert torch.isfinite(t1).all() and (t1 != 0).any()
        assert torch.allclose(t2, 2 * t1, rtol=1e-4, atol=1e-2)
