"""ctypes front-end of the CPU oracle (``oracle/adr_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker / baseline.  The product package
(``adrastea_amd``) never imports this module.

fp16 data is exchanged as ``numpy.float16`` arrays (viewed as ``uint16`` for the C side).
All element strides follow the reference convention (``adrastea_models/src/kernels.rs:864-887``):
``x`` = last dim, ``y`` = second-to-last, ``z`` = batch, counted in elements.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

LOAD_IDENTITY, LOAD_SCALE = 0, 1
(STORE_IDENTITY, STORE_GELU_BIAS, STORE_BETA_GELU_BIAS, STORE_BETA_BIAS, STORE_SCALE, STORE_ADD,
 STORE_QUICK_GELU_BIAS) = range(7)
MASK_NONE, MASK_CAUSAL = 0, 1
FAITHFUL, EXACT = 0, 1


def build(force: bool = False) -> str:
    """Compile liboracle.so (and the reference code objects when the checkout exists)."""
    src = os.path.join(_HERE, "adr_oracle.c")
    stale = (not os.path.exists(_LIB_PATH)) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src)
    if force or stale:
        subprocess.check_call(["make", "-s", "-C", _HERE, os.path.join(_HERE, "liboracle.so")])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_LIB_PATH)
        u16p, u8p, f32p, f64p = (C.POINTER(C.c_uint16), C.POINTER(C.c_uint8),
                                 C.POINTER(C.c_float), C.POINTER(C.c_double))
        L.adr_o_h2f.restype = C.c_float
        L.adr_o_h2f.argtypes = [C.c_uint16]
        L.adr_o_f2h.restype = C.c_uint16
        L.adr_o_f2h.argtypes = [C.c_float]
        L.adr_o_d2h.restype = C.c_uint16
        L.adr_o_d2h.argtypes = [C.c_double]
        L.adr_o_hmul.restype = C.c_uint16
        L.adr_o_hmul.argtypes = [C.c_uint16, C.c_uint16]
        L.adr_o_hadd.restype = C.c_uint16
        L.adr_o_hadd.argtypes = [C.c_uint16, C.c_uint16]
        L.adr_o_h2f_n.argtypes = [f32p, u16p, C.c_int64]
        L.adr_o_f2h_n.argtypes = [u16p, f32p, C.c_int64]
        L.adr_o_d2h_n.argtypes = [u16p, f64p, C.c_int64]
        L.adr_o_matmul_f16.restype = C.c_int
        L.adr_o_matmul_f16.argtypes = ([u16p, u16p, u16p] + [C.c_int] * 13 +
                                       [u16p, C.c_float, C.c_float, C.c_uint32, C.c_uint32,
                                        C.c_uint32, C.c_int, C.c_int])
        L.adr_o_matmul_nt_f16.argtypes = [u16p, u16p, u16p, C.c_int, C.c_int, C.c_int, C.c_float,
                                          C.c_int]
        for name in ("adr_o_matmul_nt_fp16u8", "adr_o_matmul_nt_fp16u8_naive"):
            getattr(L, name).argtypes = [u16p, u16p, u8p, u16p, C.c_int, C.c_int, C.c_int,
                                         C.c_int, C.c_float, C.c_int]
        L.adr_o_dequantize_absmax_u8.argtypes = [u16p, u8p, u16p, C.c_int, C.c_int, C.c_int]
        L.adr_o_quantize_absmax_u8.argtypes = [u8p, u16p, u16p, C.c_int, C.c_int, C.c_int]
        L.adr_o_dequant_table.argtypes = [u16p]
        L.adr_o_embed_uint8.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p,
                                        C.c_void_p, C.c_int]
        L.adr_o_embed_uint8.restype = None
        L.adr_o_error_stats.argtypes = [C.POINTER(C.c_float), C.c_void_p, C.c_void_p, C.c_int64, C.c_int]
        L.adr_o_softmax_rows.argtypes = [u16p, u16p, C.c_int64, C.c_int, C.c_float, C.c_int]
        L.adr_o_sgemm_nt.argtypes = [f32p, f32p, f32p, C.c_int, C.c_int, C.c_int, C.c_int]
        L.adr_o_sgemm_nt.restype = None
        _lib = L
    return _lib


def _p16(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint16))


def _p8(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint8))


def _as_f16_flat(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.float16, a.dtype
    return a.reshape(-1)


def matmul_f16(out_buf, lhs_buf, rhs_buf, batches, m, k, n, so, sl, sr, bias=None, beta=0.0,
               scale=1.0, store=STORE_IDENTITY, load=LOAD_IDENTITY, mask=MASK_NONE,
               mode=FAITHFUL, threads=1, offsets=(0, 0, 0)):
    """Run the oracle matmul on flat fp16 buffers.

    ``so``/``sl``/``sr`` are ``(stride_x, stride_y, stride_z)`` triples in elements and
    ``offsets`` the element offsets of output/lhs/rhs inside their buffers.  ``out_buf`` is
    updated in place (and returned); it must be a contiguous 1-d float16 array.
    """
    assert out_buf.dtype == np.float16 and out_buf.flags.c_contiguous and out_buf.ndim == 1
    lhs_buf, rhs_buf = _as_f16_flat(lhs_buf), _as_f16_flat(rhs_buf)
    if bias is not None:
        bias = _as_f16_flat(bias)
    o_u, l_u, r_u = out_buf.view(np.uint16), lhs_buf.view(np.uint16), rhs_buf.view(np.uint16)
    rc = lib().adr_o_matmul_f16(
        _p16(o_u[offsets[0]:]), _p16(l_u[offsets[1]:]), _p16(r_u[offsets[2]:]), batches, m, k, n,
        so[0], so[1], so[2], sl[0], sl[1], sl[2], sr[0], sr[1], sr[2],
        _p16(bias.view(np.uint16)) if bias is not None else None, float(beta), float(scale),
        int(store), int(load), int(mask), int(mode), int(threads))
    if rc != 0:
        raise ValueError("oracle: unsupported store/load/mask combination or missing bias")
    return out_buf


def matmul_nt_f16(out, lhs, rhs, beta=0.0, threads=1):
    m, p = lhs.shape
    n = rhs.shape[0]
    assert out.shape == (m, n) and out.flags.c_contiguous and out.dtype == np.float16
    lhs, rhs = np.ascontiguousarray(lhs), np.ascontiguousarray(rhs)
    lib().adr_o_matmul_nt_f16(_p16(out.view(np.uint16)), _p16(lhs.view(np.uint16)),
                              _p16(rhs.view(np.uint16)), m, p, n, float(beta), threads)
    return out


def matmul_nt_fp16u8(out, lhs, rhs_q, scales, block_size, beta=0.0, threads=1, naive=False):
    m, p = lhs.shape
    n = rhs_q.shape[0]
    assert out.shape == (m, n) and out.flags.c_contiguous and out.dtype == np.float16
    assert rhs_q.dtype == np.uint8 and scales.dtype == np.float16
    assert scales.shape == (n, p // block_size)
    lhs, rhs_q, scales = map(np.ascontiguousarray, (lhs, rhs_q, scales))
    fn = lib().adr_o_matmul_nt_fp16u8_naive if naive else lib().adr_o_matmul_nt_fp16u8
    fn(_p16(out.view(np.uint16)), _p16(lhs.view(np.uint16)), _p8(rhs_q),
       _p16(scales.view(np.uint16)), m, p, n, block_size, float(beta), threads)
    return out


def sgemm_nt(a, b, threads=1):
    """out[m,n] = a[m,k] . b[n,k]^T in fp32 (blocked, OpenMP): the host-GEMM leg of the CPU
    baseline (the reference's matrixmultiply::sgemm, adrastea_core/src/mel.rs:142-157)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    m, k = a.shape
    n = b.shape[0]
    assert b.shape[1] == k
    out = np.empty((m, n), np.float32)
    f32p = C.POINTER(C.c_float)
    lib().adr_o_sgemm_nt(out.ctypes.data_as(f32p), a.ctypes.data_as(f32p), b.ctypes.data_as(f32p),
                         m, k, n, int(threads))
    return out


def dequantize_absmax_u8(q, scales, block_size):
    rows, cols = q.shape
    q, scales = np.ascontiguousarray(q), np.ascontiguousarray(scales)
    assert scales.shape == (rows, cols // block_size) and scales.dtype == np.float16
    out = np.empty((rows, cols), np.float16)
    lib().adr_o_dequantize_absmax_u8(_p16(out.view(np.uint16)), _p8(q),
                                     _p16(scales.view(np.uint16)), rows, cols, block_size)
    return out


def quantize_absmax_u8(x, block_size):
    rows, cols = x.shape
    x = np.ascontiguousarray(x)
    assert x.dtype == np.float16 and cols % block_size == 0
    q = np.empty((rows, cols), np.uint8)
    scales = np.empty((rows, cols // block_size), np.float16)
    lib().adr_o_quantize_absmax_u8(_p8(q), _p16(scales.view(np.uint16)), _p16(x.view(np.uint16)),
                                   rows, cols, block_size)
    return q, scales


def softmax_rows(x, temp=1.0, mode=0):
    """normalize.cu:147-220 over the last axis of a contiguous fp16 array.  mode 0: the
    reference's fp32 arithmetic and reduction order; mode 1: float64, one final rounding."""
    x = np.ascontiguousarray(x)
    assert x.dtype == np.float16
    w = x.shape[-1]
    out = np.empty_like(x)
    lib().adr_o_softmax_rows(_p16(out.reshape(-1).view(np.uint16)),
                             _p16(x.reshape(-1).view(np.uint16)), x.size // w, w, float(temp), mode)
    return out


def error_stats(lhs, rhs):
    """error_stats.cu:13-75 on flat fp16 or fp32 arrays: (mse, max abs, mean abs) as float32."""
    lhs, rhs = np.ascontiguousarray(lhs).reshape(-1), np.ascontiguousarray(rhs).reshape(-1)
    assert lhs.dtype == rhs.dtype and lhs.dtype in (np.float16, np.float32) and lhs.size == rhs.size
    out = np.zeros(3, np.float32)
    lib().adr_o_error_stats(out.ctypes.data_as(C.POINTER(C.c_float)), lhs.ctypes.data_as(C.c_void_p),
                            rhs.ctypes.data_as(C.c_void_p), lhs.size, int(lhs.dtype == np.float32))
    return out


def attention_f16(q, k, v, scale, temp=1.0, mask=MASK_NONE, exact=False, threads=1):
    """The attention of one layer as the reference composes it (llama.rs:541-554): scores =
    matmul_f16(q, k^T) with MatmulStore::Scale and the mask, rounded to fp16; softmax_rows in
    place, rounded to fp16; matmul_f16 with v.  q: [heads, m, d], k and v: [heads, n, d], all
    contiguous fp16; returns [heads, m, d] fp16.  exact=True: the same function in float64 with
    one final rounding (what a path that keeps the scores unrounded is measured against)."""
    q, k, v = (np.ascontiguousarray(t) for t in (q, k, v))
    heads, m, d = q.shape
    n = k.shape[1]
    assert k.shape == (heads, n, d) and v.shape == (heads, n, d)
    if exact:
        s = np.einsum("hyd,hxd->hyx", q.astype(np.float64), k.astype(np.float64))
        s = s * np.float64(np.float16(scale))
        if mask == MASK_CAUSAL:
            s = np.where(np.arange(n)[None, None, :] > np.arange(m)[None, :, None], -np.inf, s)
        s = s / temp
        e = np.exp(s - s.max(axis=-1, keepdims=True))
        p = e / e.sum(axis=-1, keepdims=True)
        return np.einsum("hyx,hxd->hyd", p, v.astype(np.float64)).astype(np.float16)
    scores = np.zeros(heads * m * n, np.float16)
    matmul_f16(scores, q, k, heads, m, d, n, (1, n, m * n), (1, d, m * d), (d, 1, n * d),
               scale=scale, store=STORE_SCALE, mask=mask, threads=threads)
    probs = softmax_rows(scores.reshape(heads, m, n), temp, 0)
    out = np.zeros(heads * m * d, np.float16)
    matmul_f16(out, probs, v, heads, m, n, d, (1, d, m * d), (1, n, m * n), (1, d, n * d),
               threads=threads)
    return out.reshape(heads, m, d)


def embed_uint8(ids, table, scales, block_size):
    """embed_uint8.cu:3-19: rows ids[t] of the u8 table, dequantised; ids int16."""
    ids, table, scales = (np.ascontiguousarray(a) for a in (ids, table, scales))
    assert ids.dtype == np.int16 and table.dtype == np.uint8 and scales.dtype == np.float16
    n_dim = table.shape[1]
    out = np.empty((ids.size, n_dim), np.float16)
    lib().adr_o_embed_uint8(n_dim, ids.size, ids.ctypes.data_as(C.c_void_p),
                            out.ctypes.data_as(C.c_void_p), table.ctypes.data_as(C.c_void_p),
                            scales.ctypes.data_as(C.c_void_p), block_size)
    return out


def dequant_table():
    out = np.empty(256 * 65536, np.uint16)
    lib().adr_o_dequant_table(_p16(out))
    return out.reshape(256, 65536)
