"""Shared helpers for the parity tests: strided numpy views, seeded inputs, error metrics."""
import numpy as np
from numpy.lib.stride_tricks import as_strided


def view(buf, offset, shape, strides):
    """View of a flat array with element strides (reference convention: any order of dims)."""
    item = buf.itemsize
    return as_strided(buf[offset:], shape=tuple(shape), strides=tuple(s * item for s in strides),
                      writeable=False)


def largest_address(shape, strides):
    return sum((d - 1) * s for d, s in zip(shape, strides))


def rng(seed):
    return np.random.default_rng(seed)


def randn_f16(g, shape, std=1.0):
    return (g.standard_normal(shape) * std).astype(np.float32).astype(np.float16)


def ulp_diff_f16(a, b):
    """Distance in fp16 representable steps between two float16 arrays (same-sign aware)."""
    def key(x):
        u = x.view(np.uint16).astype(np.int32)
        return np.where(u & 0x8000, -(u & 0x7FFF), u & 0x7FFF)
    return np.abs(key(np.ascontiguousarray(a)) - key(np.ascontiguousarray(b)))


def max_rel_err(got, ref64):
    """max |got-ref| / max(|ref|, floor): the floor keeps near-zero outputs from dominating.

    The floor is the RMS of the reference: an element whose true value is far below the
    typical output magnitude is judged on absolute error relative to that magnitude.
    """
    got = got.astype(np.float64)
    floor = np.sqrt(np.mean(ref64 ** 2)) + 1e-30
    return float(np.max(np.abs(got - ref64) / np.maximum(np.abs(ref64), floor)))
