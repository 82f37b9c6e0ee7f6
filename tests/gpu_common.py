"""Helpers of the GPU parity tests: device buffers from numpy, calls through the C ABI."""
import numpy as np
import torch

from adrastea_amd import GpuKernels, TensorLayout, TensorView, MatmulOptions
from adrastea_amd import _ffi

import oracle

DEV = "cuda"


def to_dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().numpy()


def raw_matmul(fn_name, out_t, l_t, r_t, B, M, K, N, so, sl, sr, bias_t=None, beta=0.0, scale=1.0,
               store=0, load=0, mask=0, offsets=(0, 0, 0)):
    """Calls adr_matmul_f16 / adr_matmul_f16_slow with explicit (x, y, z) stride triples on flat
    fp16 device buffers; returns the return code."""
    fn = getattr(_ffi.lib(), fn_name)
    stream = torch.cuda.current_stream().cuda_stream
    es = 2
    return fn(stream, out_t.data_ptr() + offsets[0] * es, l_t.data_ptr() + offsets[1] * es,
              r_t.data_ptr() + offsets[2] * es, B, M, K, N, so[0], so[1], so[2], sl[0], sl[1],
              sl[2], sr[0], sr[1], sr[2], bias_t.data_ptr() if bias_t is not None else None,
              float(beta), float(scale), int(store), int(load), int(mask))


def oracle_matmul(out_np, l_np, r_np, B, M, K, N, so, sl, sr, bias=None, beta=0.0, scale=1.0,
                  store=0, load=0, mask=0, mode=oracle.EXACT, offsets=(0, 0, 0), threads=8):
    out = out_np.copy()
    oracle.matmul_f16(out, l_np, r_np, B, M, K, N, so, sl, sr, bias=bias, beta=beta, scale=scale,
                      store=store, load=load, mask=mask, mode=mode, threads=threads,
                      offsets=offsets)
    return out


def plan(B, M, K, N, so, sl, sr, store=0, load=0, mask=0):
    import ctypes as C
    buf = C.create_string_buffer(64)
    rc = _ffi.lib().adr_matmul_f16_plan(buf, 64, B, M, K, N, *so, *sl, *sr, store, load, mask)
    assert rc == 0
    return buf.value.decode()


def nan_canon(u16):
    u16 = u16.copy()
    u16[np.isnan(u16.view(np.float16))] = 0x7E00
    return u16
