"""Host-side matmul interface, mirroring ``adrastea_models/src/kernels.rs``.

``CommonKernels.matmul_f16`` / ``matmul_f16_slow`` keep the reference's names, argument meaning
and error behaviour (kernels.rs:206-213, 753-890): views in, options by value, shape mismatches
raise ``AssertionError`` (the reference ``assert_eq!``-panics), device/launcher errors raise
``AdrasteaError`` (the reference returns ``anyhow::Error``).  ``lower_matmul`` is the pure
lowering of views + options to the 22-scalar argument tuple of the C ABI.

The u8 entry points have no Rust caller in the reference (llama.rs:28-29); their methods here
follow the device kernels' argument lists (matmul_nt_fp16u8.cu:4-12, quantize.cu:3-5,46-48).
"""
from __future__ import annotations

import ctypes as C
import threading
from dataclasses import dataclass, field
from typing import Optional, Tuple

from . import _ffi
from .tensor import TensorLayout, TensorView


class AdrasteaError(RuntimeError):
    def __init__(self, code: int, what: str):
        super().__init__(f"{what}: {_ffi.strerror(code)} (code {code})")
        self.code = code


# ---- option enums (kernels.rs:81-167) ------------------------------------------------------

class MatmulMask:
    NONE = 0
    CAUSAL = 1


@dataclass(frozen=True)
class MatmulLoad:
    op: int = 0          # MatmulLoadOp: Identity = 0, Scale = 1
    scale: float = 1.0

    @staticmethod
    def Identity() -> "MatmulLoad":
        return MatmulLoad(0, 1.0)

    @staticmethod
    def Scale(scale: float) -> "MatmulLoad":
        return MatmulLoad(1, float(scale))

    def lower(self) -> int:
        return self.op


@dataclass(frozen=True)
class MatmulStore:
    op: int = 0          # MatmulStoreOp, kernels.rs:103-112
    beta: float = 0.0
    scale: Optional[float] = None
    bias: Optional[TensorView] = None

    @staticmethod
    def Identity() -> "MatmulStore":
        return MatmulStore(0)

    @staticmethod
    def GeluBias(bias) -> "MatmulStore":
        return MatmulStore(1, bias=bias)

    @staticmethod
    def BetaGeluBias(beta: float, bias) -> "MatmulStore":
        return MatmulStore(2, beta=float(beta), bias=bias)

    @staticmethod
    def BetaBias(beta: float, bias) -> "MatmulStore":
        return MatmulStore(3, beta=float(beta), bias=bias)

    @staticmethod
    def Scale(scale: float) -> "MatmulStore":
        return MatmulStore(4, scale=float(scale))

    @staticmethod
    def Add() -> "MatmulStore":
        return MatmulStore(5)

    @staticmethod
    def QuickGeluBias(bias) -> "MatmulStore":
        return MatmulStore(6, bias=bias)

    def lower(self) -> int:
        return self.op


@dataclass(frozen=True)
class MatmulOptions:
    """Builder with the reference's method names (kernels.rs:143-167)."""
    load_: MatmulLoad = field(default_factory=MatmulLoad.Identity)
    store_: MatmulStore = field(default_factory=MatmulStore.Identity)
    mask_: int = MatmulMask.NONE

    @staticmethod
    def new() -> "MatmulOptions":
        return MatmulOptions()

    def load(self, load: MatmulLoad) -> "MatmulOptions":
        return MatmulOptions(load, self.store_, self.mask_)

    def store(self, store: MatmulStore) -> "MatmulOptions":
        return MatmulOptions(self.load_, store, self.mask_)

    def mask(self, mask: int) -> "MatmulOptions":
        return MatmulOptions(self.load_, self.store_, mask)


# ---- lowering (kernels.rs:821-890) -----------------------------------------------------------

@dataclass(frozen=True)
class LoweredMatmul:
    batches: int
    m: int
    k: int
    n: int
    stride_o: Tuple[int, int, int]   # (x, y, z)
    stride_l: Tuple[int, int, int]
    stride_r: Tuple[int, int, int]
    beta: float
    scale: float
    store: int
    load: int
    mask: int

    def scalars(self):
        return (self.batches, self.m, self.k, self.n, *self.stride_o, *self.stride_l,
                *self.stride_r)


def _xyz(layout: TensorLayout) -> Tuple[int, int, int]:
    # batch stride 0 for rank-2 operands: they are broadcast over the batches (kernels.rs:868-880)
    return (layout.stride(-1), layout.stride(-2), layout.stride(-3) if len(layout.dims) > 2 else 0)


def lower_matmul(output: TensorLayout, left: TensorLayout, right: TensorLayout,
                 options: MatmulOptions) -> LoweredMatmul:
    assert left.size(-1) == right.size(-2), "K mismatch"      # kernels.rs:825
    assert output.size(-2) == left.size(-2), "M mismatch"     # kernels.rs:826
    assert output.size(-1) == right.size(-1), "N mismatch"    # kernels.rs:827
    scale = options.load_.scale if options.load_.op == 1 else 1.0
    if options.store_.op == 4:
        scale *= options.store_.scale                          # one float for both (:837-843)
    beta = options.store_.beta if options.store_.op in (2, 3) else 0.0
    batches = output.size(-3) if len(output.dims) > 2 else 1
    return LoweredMatmul(batches, left.size(-2), left.size(-1), right.size(-1), _xyz(output),
                         _xyz(left), _xyz(right), beta, scale, options.store_.lower(),
                         options.load_.lower(), options.mask_)


# ---- the kernel interface ----------------------------------------------------------------------

class CommonKernels:
    """The matmul subset of the reference trait (kernels.rs:169-229)."""

    def matmul_f16(self, output: TensorView, left: TensorView, right: TensorView,
                   options: MatmulOptions) -> None:
        raise NotImplementedError

    def matmul_f16_slow(self, output: TensorView, left: TensorView, right: TensorView,
                        options: MatmulOptions) -> None:
        raise NotImplementedError

    def softmax_rows_inplace(self, output: TensorView, temperature: float) -> None:
        raise NotImplementedError


def _current_stream() -> int:
    import torch
    return torch.cuda.current_stream().cuda_stream


class GpuKernels(CommonKernels):
    """Launches through the C ABI on torch's current HIP stream.

    `workspace_bytes` > 0 gives the instance a scratch buffer of that size, owned like any other
    tensor of the host (in the reference: one more GpuBuffer held by GpuKernels); matmul_f16 then
    goes through adr_matmul_f16_ws, which may split K over workgroups for products with few
    output tiles and a long K.  The buffer carries nothing between calls; one instance must not
    be used from streams that run concurrently.  Without it (the default) the library takes such
    a buffer from its own per-stream cache (set_held_workspace_limit)."""

    def __init__(self, workspace_bytes: int = 0):
        self._lib = _ffi.lib()
        import torch
        if not torch.cuda.is_available():
            raise RuntimeError("adrastea_amd.GpuKernels needs a GPU; there is no CPU fallback")
        self._workspace = (torch.empty(workspace_bytes, dtype=torch.uint8, device="cuda")
                           if workspace_bytes > 0 else None)

    def _matmul(self, fn, what, output, left, right, options):
        low = lower_matmul(output.layout, left.layout, right.layout, options)
        bias = options.store_.bias
        rc = fn(_current_stream(), output.data_ptr(), left.data_ptr(), right.data_ptr(),
                *low.scalars(), bias.data_ptr() if bias is not None else None, low.beta,
                low.scale, low.store, low.load, low.mask)
        if rc != 0:
            raise AdrasteaError(rc, what)

    def matmul_f16(self, output, left, right, options=MatmulOptions()):
        if self._workspace is None:
            return self._matmul(self._lib.adr_matmul_f16, "matmul_f16", output, left, right, options)
        ws = self._workspace

        def with_workspace(*args):
            return self._lib.adr_matmul_f16_ws(*args, ws.data_ptr(), ws.numel())
        self._matmul(with_workspace, "matmul_f16", output, left, right, options)

    def matmul_f16_slow(self, output, left, right, options=MatmulOptions()):
        self._matmul(self._lib.adr_matmul_f16_slow, "matmul_f16_slow", output, left, right,
                     options)

    def softmax_rows_inplace(self, output, temperature: float = 1.0):
        """kernels.rs:892-915: rows = size(-2), heads = size(-3) (1 for rank 2), width size(-1);
        like the reference's kernel, the tensor is taken to be contiguous."""
        lay = output.layout
        assert lay == TensorLayout.row_major(list(lay.dims)), "softmax_rows needs a contiguous view"
        heads = lay.size(-3) if len(lay.dims) > 2 else 1
        rc = self._lib.adr_softmax_rows(_current_stream(), output.data_ptr(), output.data_ptr(),
                                        heads, lay.size(-2), lay.size(-1), float(temperature))
        if rc != 0:
            raise AdrasteaError(rc, "softmax_rows_inplace")

    def attention_f16(self, output, query, key, value, scale: float, temperature: float = 1.0,
                      mask: int = MatmulMask.NONE):
        """The three calls of llama.rs:541-554 (QK^T with Scale and the mask, softmax_rows_inplace,
        P.V) as one launch that keeps the scores out of memory.  `query`/`output` are
        [heads, m, d] views, `key`/`value` [heads, n, d] views (rank 2 = one head).  Raises
        AdrasteaError with code ADR_EUNSUPPORTED_LAYOUT for head dimensions or strides the fused
        kernel does not cover; the three-call sequence remains available for those."""
        lo, lq, lk, lv = output.layout, query.layout, key.layout, value.layout
        rank = len(lq.dims)
        assert rank in (2, 3) and all(len(l.dims) == rank for l in (lo, lk, lv))
        heads = lq.size(-3) if rank == 3 else 1
        m, d, n = lq.size(-2), lq.size(-1), lk.size(-2)
        assert lk.size(-1) == d and lv.size(-1) == d and lv.size(-2) == n
        assert lo.size(-2) == m and lo.size(-1) == d
        if rank == 3:
            assert lo.size(-3) == heads and lk.size(-3) == heads and lv.size(-3) == heads

        def xyz(l):
            return l.stride(-1), l.stride(-2), (l.stride(-3) if rank == 3 else 0)
        rc = self._lib.adr_attention_f16(_current_stream(), output.data_ptr(), query.data_ptr(),
                                         key.data_ptr(), value.data_ptr(), heads, m, n, d,
                                         *xyz(lo), *xyz(lq), *xyz(lk), *xyz(lv), float(scale),
                                         float(temperature), int(mask))
        if rc != 0:
            raise AdrasteaError(rc, "attention_f16")

    def _error_stats(self, fn, what, output, lhs, rhs):
        # kernels.rs:717-751: both operands flattened with shape_cast(&[-1]); equal lengths
        lhs, rhs = lhs.shape_cast([-1]), rhs.shape_cast([-1])
        assert lhs.size(-1) == rhs.size(-1)
        rc = fn(_current_stream(), descriptor(output), descriptor(lhs), descriptor(rhs))
        if rc != 0:
            raise AdrasteaError(rc, what)

    def error_stats_f16(self, output, lhs, rhs):
        self._error_stats(self._lib.adr_error_stats_f16, "error_stats_f16", output, lhs, rhs)

    def error_stats_f32(self, output, lhs, rhs):
        self._error_stats(self._lib.adr_error_stats_f32, "error_stats_f32", output, lhs, rhs)

    # -- contiguous NT forms (device signatures only in the reference) --
    def matmul_nt_f16(self, output, lhs, rhs, beta: float = 0.0):
        m, p = lhs.shape
        n = rhs.shape[0]
        assert rhs.shape[1] == p and tuple(output.shape) == (m, n)
        assert output.is_contiguous() and lhs.is_contiguous() and rhs.is_contiguous()
        rc = self._lib.adr_matmul_nt_f16(_current_stream(), output.data_ptr(), lhs.data_ptr(),
                                         rhs.data_ptr(), m, p, n, beta)
        if rc != 0:
            raise AdrasteaError(rc, "matmul_nt_f16")

    def matmul_nt_fp16u8(self, output, lhs, rhs_q, scales, block_size: int, beta: float = 0.0):
        m, p = lhs.shape
        n = rhs_q.shape[0]
        assert rhs_q.shape[1] == p and tuple(output.shape) == (m, n)
        assert tuple(scales.shape) == (n, p // block_size)
        assert all(t.is_contiguous() for t in (output, lhs, rhs_q, scales))
        if self._workspace is None:
            rc = self._lib.adr_matmul_nt_fp16u8(_current_stream(), output.data_ptr(), lhs.data_ptr(),
                                                rhs_q.data_ptr(), scales.data_ptr(), m, p, n,
                                                block_size, beta)
        else:
            # with a workspace of n * p * 2 bytes or more, products of 129 rows and more may
            # dequantise the matrix once and run the fp16 kernels (same bits, less time)
            rc = self._lib.adr_matmul_nt_fp16u8_ws(_current_stream(), output.data_ptr(), lhs.data_ptr(),
                                                   rhs_q.data_ptr(), scales.data_ptr(), m, p, n,
                                                   block_size, beta, self._workspace.data_ptr(),
                                                   self._workspace.numel())
        if rc != 0:
            raise AdrasteaError(rc, "matmul_nt_fp16u8")

    def dequantize_absmax_uint8(self, output, scales, q):
        rows, cols = q.shape
        block_size = cols // scales.shape[1]
        rc = self._lib.adr_dequantize_absmax_u8(_current_stream(), output.data_ptr(),
                                                q.data_ptr(), scales.data_ptr(), rows, cols,
                                                block_size)
        if rc != 0:
            raise AdrasteaError(rc, "dequantize_absmax_uint8")

    def quantize_absmax_uint8(self, q, scales, x):
        rows, cols = x.shape
        block_size = cols // scales.shape[1]
        rc = self._lib.adr_quantize_absmax_u8(_current_stream(), q.data_ptr(), scales.data_ptr(),
                                              x.data_ptr(), rows, cols, block_size)
        if rc != 0:
            raise AdrasteaError(rc, "quantize_absmax_uint8")

    def embed_uint8(self, output, ids, table, scales, block_size: int):
        """embed_uint8.cu:3-19: output[t] = dequantised row ids[t] of the u8 table; `ids` is an
        int16 tensor, as the reference's kernel takes them."""
        import torch
        assert ids.dtype == torch.int16 and table.dtype == torch.uint8
        n_ids, n_dim = ids.numel(), table.shape[1]
        assert tuple(output.shape) == (n_ids, n_dim)
        assert tuple(scales.shape) == (table.shape[0], n_dim // block_size)
        assert all(t.is_contiguous() for t in (output, ids, table, scales))
        rc = self._lib.adr_embed_uint8(_current_stream(), n_dim, n_ids, ids.data_ptr(),
                                       output.data_ptr(), table.data_ptr(), scales.data_ptr(),
                                       block_size)
        if rc != 0:
            raise AdrasteaError(rc, "embed_uint8")


def descriptor(view: TensorView) -> _ffi.TensorDesc:
    """TensorGpuDescriptor::from (kernels.rs:38-55): dims and strides reversed, innermost first."""
    d = _ffi.TensorDesc()
    d.ptr = view.data_ptr()
    d.dims = len(view.layout.dims)
    for i, (dim, stride) in enumerate(zip(reversed(view.layout.dims),
                                          reversed(view.layout.strides))):
        d.shape[i] = dim
        d.strides[i] = stride
    return d


def plan_matmul(output: TensorLayout, left: TensorLayout, right: TensorLayout,
                options: MatmulOptions = MatmulOptions(), workspace_bytes: int = 0) -> str:
    """Name of the kernel adr_matmul_f16 (or, with a workspace, adr_matmul_f16_ws) selects for
    these layouts (no device needed)."""
    low = lower_matmul(output, left, right, options)
    buf = C.create_string_buffer(96)
    rc = _ffi.lib().adr_matmul_f16_ws_plan(buf, 96, *low.scalars(), low.store, low.load, low.mask,
                                           int(workspace_bytes))
    if rc != 0:
        raise AdrasteaError(rc, "matmul_f16_plan")
    return buf.value.decode()


def matmul_workspace_bytes(output: TensorLayout, left: TensorLayout, right: TensorLayout,
                           options: MatmulOptions = MatmulOptions()) -> int:
    """Scratch bytes adr_matmul_f16_ws would use for these layouts (0: it would not split K)."""
    low = lower_matmul(output, left, right, options)
    n = _ffi.lib().adr_matmul_f16_workspace_bytes(*low.scalars(), low.store, low.load, low.mask)
    if n < 0:
        raise AdrasteaError(int(n), "matmul_f16_workspace_bytes")
    return int(n)


def set_held_workspace_limit(nbytes: int) -> None:
    """Bytes per buffer of the workspace pool that adr_matmul_f16 and adr_matmul_nt_f16 (and, on
    request, adr_matmul_nt_fp16u8) draw from, one buffer per (device, stream); 0 switches it off."""
    rc = _ffi.lib().adr_set_held_workspace_limit(int(nbytes))
    if rc != 0:
        raise AdrasteaError(int(rc), "set_held_workspace_limit")


def held_workspace_limit() -> int:
    return int(_ffi.lib().adr_held_workspace_limit())


def held_workspace_bytes() -> int:
    """Bytes the pool holds now."""
    return int(_ffi.lib().adr_held_workspace_bytes())


def held_workspace_declined() -> int:
    """Calls so far that wanted a buffer of the pool and ran without one."""
    return int(_ffi.lib().adr_held_workspace_declined())


def release_held_workspace(stream=None) -> None:
    """Frees the pool's buffers of `stream` (a raw stream handle; default: torch's current stream)
    and those no stream owns any more, after waiting for the last launches that used them.  Call it
    before destroying a stream.  `stream="all"`: every buffer on every device."""
    L = _ffi.lib()
    rc = (L.adr_release_held_workspace_all() if stream == "all" else
          L.adr_release_held_workspace(_current_stream() if stream is None else stream))
    if rc != 0:
        raise AdrasteaError(int(rc), "release_held_workspace")


def set_u8_dequantise_first(enabled: bool) -> None:
    """Lets adr_matmul_nt_fp16u8 dequantise the weight matrix once into a buffer of the pool and
    run the fp16 kernels on it where that is faster (off by default: always the fused kernels)."""
    _ffi.lib().adr_set_u8_dequantise_first(1 if enabled else 0)


class MatmulTracer(CommonKernels):
    """Decorator recording the set of (left, right, output) layouts seen by the matmuls, then
    forwarding (kernels.rs:231-359)."""

    def __init__(self, inner: CommonKernels):
        self.inner = inner
        self._lock = threading.Lock()
        self.shapes = set()

    def clear(self):
        with self._lock:
            self.shapes.clear()

    def _record(self, output, left, right):
        with self._lock:
            self.shapes.add((left.layout, right.layout, output.layout))

    def matmul_f16(self, output, left, right, options=MatmulOptions()):
        self._record(output, left, right)
        self.inner.matmul_f16(output, left, right, options)

    def matmul_f16_slow(self, output, left, right, options=MatmulOptions()):
        self._record(output, left, right)
        self.inner.matmul_f16_slow(output, left, right, options)

    def softmax_rows_inplace(self, output, temperature: float = 1.0):
        self.inner.softmax_rows_inplace(output, temperature)   # forwarded (kernels.rs:334-338)

    def attention_f16(self, output, query, key, value, scale, temperature=1.0,
                      mask=MatmulMask.NONE):
        self.inner.attention_f16(output, query, key, value, scale, temperature, mask)

    def error_stats_f16(self, output, lhs, rhs):
        self.inner.error_stats_f16(output, lhs, rhs)            # forwarded (kernels.rs:349-358)

    def error_stats_f32(self, output, lhs, rhs):
        self.inner.error_stats_f32(output, lhs, rhs)
