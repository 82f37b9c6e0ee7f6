"""CPU-only checks of the boundary: the built library loads, exports every declared symbol,
validates arguments on the host, and selects kernels as documented.  No device call is made."""
import ctypes as C
import os
import re

import pytest

from adrastea_amd import _ffi, TensorLayout, MatmulOptions, MatmulStore, MatmulLoad, MatmulMask
from adrastea_amd import kernels as K

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_header_symbols_are_all_exported():
    text = open(os.path.join(ROOT, "include", "adrastea_kernels.h")).read()
    declared = set(re.findall(r"\b(adr_[a-z0-9_]+)\s*\(", text))
    assert declared == set(_ffi.SYMBOLS)
    lib = _ffi.lib()
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.adr_abi_version() >= 1


def test_strerror_covers_codes():
    for code in range(-8, 1):
        assert _ffi.strerror(code)
    assert "GeluBias" in _ffi.strerror(-3)


def _plan(B, M, Kd, N, so, sl, sr, store=0, load=0, mask=0):
    buf = C.create_string_buffer(64)
    rc = _ffi.lib().adr_matmul_f16_plan(buf, 64, B, M, Kd, N, *so, *sl, *sr, store, load, mask)
    return rc, buf.value.decode()


def test_plan_validation_codes():
    nt = ((1, 64, 0), (1, 64, 0), (64, 1, 0))
    assert _plan(1, 64, 64, 64, *nt)[0] == 0
    assert _plan(1, 64, 64, 64, *nt, store=1)[0] == _ffi.ADR_ENOTIMPL
    assert _plan(1, 64, 64, 64, *nt, store=7)[0] == _ffi.ADR_EINVAL_ENUM
    assert _plan(1, 64, 64, 64, *nt, load=2)[0] == _ffi.ADR_EINVAL_ENUM
    assert _plan(1, 64, 64, 64, *nt, mask=2)[0] == _ffi.ADR_EINVAL_ENUM
    assert _plan(1, -1, 64, 64, *nt)[0] == _ffi.ADR_EINVAL_SHAPE
    assert _plan(0, 64, 64, 64, *nt) == (0, "none (empty)")


def test_kernel_selection_for_the_callers_layouts():
    # linear layers: W[N,K].permute([1,0]) (llama.rs:503-508)
    M, Kd, N = 2048, 4096, 12288
    out, lhs = TensorLayout.row_major([M, N]), TensorLayout.row_major([M, Kd])
    w = TensorLayout.row_major([N, Kd]).permute([1, 0])
    assert K.plan_matmul(out, lhs, w).startswith("gemm_nt_mfma_dma_")
    # QK^T on the head views (llama.rs:534-550)
    S, H, D = 2048, 32, 128
    q = TensorLayout.row_major([S, H * D]).shape_cast([S, H, -1]).permute([1, 0, 2])
    k = TensorLayout.row_major([S, H * D]).shape_cast([S, H, -1]).permute([1, 2, 0])
    qk = TensorLayout.row_major([H, S, S])
    opts = MatmulOptions.new().store(MatmulStore.Scale(1.0 / D ** 0.5)).mask(MatmulMask.CAUSAL)
    assert K.plan_matmul(qk, q, k, opts).startswith("gemm_nt_mfma")
    # a row-major right operand with K % 8 != 0 falls back to the general kernel
    assert K.plan_matmul(TensorLayout.row_major([10, 12]), TensorLayout.row_major([10, 7]),
                         TensorLayout.row_major([7, 12])) == "matmul_general"
    # small CLIP text GEMM
    assert K.plan_matmul(TensorLayout.row_major([77, 2304]), TensorLayout.row_major([77, 768]),
                         TensorLayout.row_major([2304, 768]).permute([1, 0])).startswith("gemm_nt_mfma")


def test_u8_plan():
    def plan(m, p, n, bs):
        buf = C.create_string_buffer(64)
        rc = _ffi.lib().adr_matmul_nt_fp16u8_plan(buf, 64, m, p, n, bs)
        return rc, buf.value.decode()
    for m in (1, 2):
        assert plan(m, 4096, 4096, 32) == (0, "gemv_u8_dot2_stream")
    assert plan(1, 11008, 4096, 32) == (0, "gemv_u8_dot2_stream")
    assert plan(2, 11008, 4096, 32) == (0, "gemv_u8_mfma16_regstream")   # two rows over a long K
    for m in (3, 4, 16):
        assert plan(m, 4096, 4096, 32) == (0, "gemv_u8_mfma16_regstream")
        assert plan(m, 11008, 4096, 32) == (0, "gemv_u8_mfma16_regstream")
        assert plan(m, 4096, 12288, 32) == (0, "gemv_u8_mfma16_regstream")
        assert plan(m, 256, 16, 32) == (0, "gemv_u8_mfma16_regstream")
    assert plan(2, 4096, 12288, 32) == (0, "gemv_u8_dot2_stream")
    # 17 to 64 rows in blocks of rows: 32 per pass for K = 4096, 16 otherwise
    assert plan(32, 4096, 12288, 32) == (0, "gemv_u8_mfma16_dma_32rows")
    assert plan(32, 11008, 4096, 32) == (0, "gemv_u8_mfma16_blocks")
    assert plan(64, 4096, 4096, 32) == (0, "gemv_u8_mfma16_blocks")
    # 33 rows and more: passes where the estimate puts them ahead of the tiled kernel (narrow
    # matrices), else the tiled kernel's small tiles
    assert plan(64, 4096, 12288, 32) == (0, "gemm_nt_u8_mfma_64x64x64_k4")
    # above 64 rows: passes of 64 rows where the estimate puts them ahead of the tiled kernel (to
    # 128 rows against a narrow matrix)
    assert plan(70, 11008, 4096, 32) == (0, "gemv_u8_mfma16_blocks")
    assert plan(70, 4096, 4096, 32) == (0, "gemv_u8_mfma16_blocks")
    assert plan(128, 11008, 4096, 32) == (0, "gemv_u8_mfma16_blocks")
    assert plan(160, 11008, 4096, 32) == (0, "gemm_nt_u8_mfma_64x64x64_k4")
    assert plan(256, 11008, 4096, 32) == (0, "gemm_nt_u8_mfma_64x64x64_k4")
    assert plan(96, 4096, 12288, 32) == (0, "gemm_nt_u8_mfma_128x64x64_k2")
    assert plan(100, 512, 9000, 32)[1].startswith("gemm_nt_u8_mfma_")
    # tiled kernel: the name carries the tile, and the K groups of the two small ones where
    # there is at most one tile per compute unit
    assert plan(2048, 4096, 4096, 32) == (0, "gemm_nt_u8_mfma_256x128x64")
    assert plan(2048, 4096, 12288, 32) == (0, "gemm_nt_u8_mfma_256x192x64")
    assert plan(2048, 4096, 11008, 32) == (0, "gemm_nt_u8_mfma_256x192x64")
    assert plan(2048, 11008, 4096, 32) == (0, "gemm_nt_u8_mfma_256x128x64")
    assert plan(1024, 11008, 4096, 32) == (0, "gemm_nt_u8_mfma_128x128x64")
    assert plan(300, 4096, 4096, 32) == (0, "gemm_nt_u8_mfma_128x64x64_k2")
    assert plan(300, 4096 + 64, 4096, 32) == (0, "gemm_nt_u8_mfma_128x64x64")      # K % 128 != 0: one group
    assert plan(600, 4096, 4096, 32)[1] in ("gemm_nt_u8_mfma_128x64x64", "gemm_nt_u8_mfma_128x128x64")
    assert plan(8, 4096, 4096, 64) == (0, "gemm_nt_u8_mfma_64x64x64_k4")
    assert plan(300, 4096 + 32, 4096, 32)[1].startswith("gemm_nt_u8_stage_")        # K % 64 != 0
    assert plan(8, 36, 64, 12) == (0, "gemm_u8_naive")
    assert plan(4, 4100, 64, 32)[0] == _ffi.ADR_EDIVISIBILITY
    assert plan(4, 64, 64, 0)[0] == _ffi.ADR_EINVAL_SHAPE


def test_offsets_beyond_int32_are_rejected():
    """Element offsets are i32 in the reference (kernels.rs:864-887): a view whose farthest
    element lies at 2^31 elements or more returns ADR_EINVAL_SHAPE."""
    big = 1 << 16
    ok = ((1, 32767, 0), (1, 64, 0), (64, 1, 0))
    assert _plan(1, 32768, 64, 32767, *ok)[0] == 0
    too_far_out = ((1, big, 0), (1, 64, 0), (64, 1, 0))
    assert _plan(1, 32769, 64, big, *too_far_out)[0] == _ffi.ADR_EINVAL_SHAPE
    far_batch = ((1, 64, 1 << 30), (1, 64, 0), (64, 1, 0))
    assert _plan(3, 64, 64, 64, *far_batch)[0] == _ffi.ADR_EINVAL_SHAPE
    assert _plan(2, 64, 64, 64, *far_batch)[0] == 0
    neg = ((1, 64, 0), (1, -(1 << 25), 0), (64, 1, 0))
    assert _plan(1, 65, 64, 64, *neg)[0] == _ffi.ADR_EINVAL_SHAPE
    lib = _ffi.lib()
    # the contiguous entry points: n * p elements of weights
    assert lib.adr_matmul_nt_fp16u8(None, 8, 8, 8, 8, 1, 1 << 16, 1 << 15, 32, 0.0) == _ffi.ADR_EINVAL_SHAPE
    assert lib.adr_matmul_nt_f16(None, 8, 8, 8, 1, 1 << 16, 1 << 15, 0.0) == _ffi.ADR_EINVAL_SHAPE


def test_no_usable_device_is_an_error_not_a_crash():
    """On a machine without a gfx950 device a launching entry point returns
    ADR_EUNSUPPORTED_DEVICE or the runtime's error code; it never launches and never aborts."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = _ffi.lib()
    rc = lib.adr_matmul_nt_f16(None, 16, 16, 16, 4, 64, 4, 0.0)
    assert rc != 0
    assert _ffi.strerror(rc)
    assert lib.adr_microbench_empty(None) == rc


def test_integration_source_list_matches_the_build():
    """The build.rs recipe of the integration guide must name every source the library is built from."""
    from adrastea_amd import build
    text = open(os.path.join(ROOT, "INTEGRATION.md")).read()
    block = text[text.index("let src = ["):]
    block = block[:block.index("];")]
    assert sorted(re.findall(r'"([a-z0-9_]+\.hip)"', block)) == sorted(build.SOURCES)


def test_workspace_plan_and_size():
    """adr_matmul_f16_ws splits K only for few output tiles and a long K, and only with enough
    workspace; the size query and the plan agree."""
    lib = _ffi.lib()

    def need(m, k, n):
        return lib.adr_matmul_f16_workspace_bytes(1, m, k, n, 1, n, 0, 1, k, 0, k, 1, 0, 0, 0, 0)

    def plan_ws(m, k, n, ws):
        buf = C.create_string_buffer(96)
        assert lib.adr_matmul_f16_ws_plan(buf, 96, 1, m, k, n, 1, n, 0, 1, k, 0, k, 1, 0, 0, 0, 0, ws) == 0
        return buf.value.decode()
    b = need(128, 11008, 4096)
    assert b > 0
    pieces = lambda name: int(name.rsplit("_splitk", 1)[1])
    full = plan_ws(128, 11008, 4096, b)
    assert "_splitk" in full and pieces(full) >= 2
    # less workspace: fewer pieces (or smaller tiles), then none
    less = plan_ws(128, 11008, 4096, b - 16)
    assert "_splitk" in less and less != full
    assert plan_ws(128, 11008, 4096, b // 8) == plan_ws(128, 11008, 4096, 0)
    # the plain entry point's plan follows the held-workspace limit as it is now
    before = lib.adr_held_workspace_limit()
    try:
        for limit in (0, b - 16, _ffi.HELD_WORKSPACE_DEFAULT_BYTES):
            lib.adr_set_held_workspace_limit(limit)
            assert _plan(1, 128, 11008, 4096, (1, 4096, 0), (1, 11008, 0), (11008, 1, 0))[1] == \
                plan_ws(128, 11008, 4096, limit)
    finally:
        lib.adr_set_held_workspace_limit(before)
    # the prefill shapes and the decode shapes are never split
    assert need(2048, 4096, 12288) == 0 and need(2048, 11008, 4096) == 0
    assert need(1, 4096, 4096) == 0 and need(16, 11008, 4096) == 0
    assert need(128, 512, 4096) == 0            # short K
    assert lib.adr_matmul_f16_workspace_bytes(1, -1, 64, 64, 1, 64, 0, 1, 64, 0, 64, 1, 0, 0, 0, 0) == _ffi.ADR_EINVAL_SHAPE


def test_u8_workspace_size_and_validation():
    """adr_matmul_nt_fp16u8_ws dequantises the matrix first from 768 rows on (below, the fused kernel's small tiles are
    ahead); the size query says when, and how much."""
    lib = _ffi.lib()
    need = lib.adr_matmul_nt_fp16u8_workspace_bytes
    assert need(2048, 4096, 12288, 32) == 12288 * 4096 * 2
    assert need(768, 11008, 4096, 32) == 4096 * 11008 * 2
    assert need(1024, 4096, 4096, 32) == 4096 * 4096 * 2
    assert need(1024, 4096, 12288, 32) == 12288 * 4096 * 2
    assert need(767, 4096, 12288, 32) == 0 and need(512, 11008, 4096, 32) == 0
    assert need(256, 4096, 12288, 32) == 0 and need(1, 4096, 12288, 32) == 0
    assert need(2048, 0, 64, 32) == 0
    assert need(-1, 64, 64, 32) == _ffi.ADR_EINVAL_SHAPE
    assert need(256, 100, 64, 32) == _ffi.ADR_EDIVISIBILITY
    ws = lib.adr_matmul_nt_fp16u8_ws
    assert ws(None, 8, 8, 8, 8, 256, 100, 64, 32, 0.0, 16, 1 << 20) == _ffi.ADR_EDIVISIBILITY
    assert ws(None, 8, 8, 8, 8, 256, 64, 64, 32, 0.0, None, 1 << 20) == _ffi.ADR_ENULL
    assert ws(None, 8, 8, 8, 8, 256, 64, 64, 32, 0.0, 24, 1 << 20) == _ffi.ADR_EINVAL_SHAPE   # unaligned
    assert ws(None, 8, 8, 8, 8, 0, 64, 64, 32, 0.0, None, 0) == 0                              # empty


def test_u8_plan_follows_the_dequantise_first_switch():
    lib = _ffi.lib()
    buf = C.create_string_buffer(96)

    def plan_u8(m, p, n):
        assert lib.adr_matmul_nt_fp16u8_plan(buf, 96, m, p, n, 32) == 0
        return buf.value.decode()
    before = lib.adr_held_workspace_limit()
    try:
        lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
        assert lib.adr_u8_dequantise_first() == 0
        assert plan_u8(2048, 4096, 12288) == "gemm_nt_u8_mfma_256x192x64"      # the default: fused
        assert lib.adr_set_u8_dequantise_first(1) == 0 and lib.adr_u8_dequantise_first() == 1
        assert plan_u8(2048, 4096, 12288) == "dequantize_absmax_u8 + fp16 gemm"
        assert plan_u8(16, 4096, 12288) == "gemv_u8_mfma16_regstream"          # never for decode
        lib.adr_set_held_workspace_limit(64 << 20)                              # the matrix does not fit
        assert plan_u8(2048, 4096, 12288) == "gemm_nt_u8_mfma_256x192x64"
    finally:
        lib.adr_set_u8_dequantise_first(0)
        lib.adr_set_held_workspace_limit(before)


def test_held_workspace_controls():
    import adrastea_amd as A
    lib = _ffi.lib()
    assert _ffi.HELD_WORKSPACE_DEFAULT_BYTES == 128 << 20
    before = lib.adr_held_workspace_limit()
    try:
        A.set_held_workspace_limit(3 << 20)
        assert A.held_workspace_limit() == lib.adr_held_workspace_limit() == 3 << 20
        assert lib.adr_set_held_workspace_limit(-1) == _ffi.ADR_EINVAL_SHAPE
        assert A.held_workspace_limit() == 3 << 20
        with pytest.raises(A.AdrasteaError):
            A.set_held_workspace_limit(-1)
        # nothing is allocated by asking
        assert A.held_workspace_bytes() == lib.adr_held_workspace_bytes() >= 0
        assert A.held_workspace_declined() == lib.adr_held_workspace_declined() >= 0
    finally:
        lib.adr_set_held_workspace_limit(before)
