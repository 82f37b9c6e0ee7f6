"""ctypes binding of libadrastea_kernels_hip.so (declarations: include/adrastea_kernels.h)."""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libadrastea_kernels_hip.so")

# every symbol include/adrastea_kernels.h declares
SYMBOLS = (
    "adr_matmul_f16", "adr_matmul_f16_slow", "adr_matmul_f16_raw", "adr_matmul_nt_f16",
    "adr_matmul_f16_ws", "adr_matmul_f16_workspace_bytes", "adr_matmul_f16_ws_plan",
    "adr_matmul_f16_noalloc",
    "adr_set_held_workspace_limit", "adr_held_workspace_limit", "adr_held_workspace_bytes",
    "adr_held_workspace_declined", "adr_release_held_workspace", "adr_release_held_workspace_all",
    "adr_set_u8_dequantise_first", "adr_u8_dequantise_first",
    "adr_matmul_nt_fp16u8", "adr_matmul_nt_fp16u8_ws", "adr_matmul_nt_fp16u8_workspace_bytes",
    "adr_dequantize_absmax_u8", "adr_quantize_absmax_u8",
    "adr_dequantize_absmax_uint8", "adr_quantize_absmax_uint8", "adr_matmul_f16_plan",
    "adr_matmul_nt_fp16u8_plan", "adr_softmax_rows", "adr_error_stats_f16", "adr_error_stats_f32", "adr_attention_f16", "adr_embed_uint8",
    "adr_debug_knob", "adr_microbench_empty", "adr_microbench_mfma_f16", "adr_microbench_stream_read",
    "adr_strerror", "adr_abi_version",
)

ADR_OK, ADR_EINVAL_SHAPE, ADR_EINVAL_ENUM, ADR_ENOTIMPL, ADR_ENULL, ADR_EDIVISIBILITY = (
    0, -1, -2, -3, -4, -5)
ADR_EUNSUPPORTED_DEVICE, ADR_EUNSUPPORTED_LAYOUT, ADR_ESCRATCH = -6, -7, -8
KNOB_GEMM_TILE = 0
NOALLOC_SCRATCH_BYTES = 16 * 1024 * 1024
HELD_WORKSPACE_DEFAULT_BYTES = 128 * 1024 * 1024


class TensorDesc(C.Structure):
    """adr_tensor_desc: index 0 is the innermost dimension (kernels.rs:28-47)."""
    _fields_ = [("ptr", C.c_void_p), ("dims", C.c_uint32), ("shape", C.c_uint32 * 7),
                ("strides", C.c_uint32 * 7)]


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built: there is no fallback path."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m adrastea_amd.build` "
            "(hipcc, gfx950); adrastea_amd has no CPU or PyTorch fallback")
    # The host mirror keeps device memory in torch tensors, and torch ships a HIP runtime of its
    # own: load that one first, so that this library's libamdhip64 dependency resolves to the
    # runtime torch has initialised.  Loaded in the other order, the process holds two runtimes
    # and the library's launches fail with hipErrorNoDevice.
    import torch  # noqa: F401
    L = C.CDLL(LIB_PATH)
    vp, i32, u32, f32 = C.c_void_p, C.c_int32, C.c_uint32, C.c_float
    mm = [vp, vp, vp, vp] + [i32] * 13 + [vp, f32, f32, u32, u32, u32]
    L.adr_matmul_f16.argtypes = mm
    L.adr_matmul_f16_slow.argtypes = mm
    L.adr_matmul_f16_ws.argtypes = mm + [vp, C.c_int64]
    L.adr_matmul_f16_noalloc.argtypes = mm
    L.adr_set_held_workspace_limit.argtypes = [C.c_int64]
    L.adr_held_workspace_limit.argtypes = []
    L.adr_held_workspace_limit.restype = C.c_int64
    L.adr_held_workspace_bytes.argtypes = []
    L.adr_held_workspace_bytes.restype = C.c_int64
    L.adr_held_workspace_declined.argtypes = []
    L.adr_release_held_workspace.argtypes = [vp]
    L.adr_release_held_workspace_all.argtypes = []
    L.adr_set_u8_dequantise_first.argtypes = [C.c_int]
    L.adr_u8_dequantise_first.argtypes = []
    L.adr_matmul_f16_workspace_bytes.argtypes = [i32] * 13 + [u32, u32, u32]
    L.adr_matmul_f16_ws_plan.argtypes = [C.c_char_p, i32] + [i32] * 13 + [u32, u32, u32, C.c_int64]
    L.adr_matmul_f16_raw.argtypes = [vp, vp, vp, vp] + [i32] * 13
    L.adr_matmul_nt_f16.argtypes = [vp, vp, vp, vp, i32, i32, i32, f32]
    L.adr_matmul_nt_fp16u8.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, f32]
    L.adr_matmul_nt_fp16u8_ws.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, i32, f32, vp, C.c_int64]
    L.adr_matmul_nt_fp16u8_workspace_bytes.argtypes = [i32, i32, i32, i32]
    L.adr_matmul_nt_fp16u8_workspace_bytes.restype = C.c_int64
    L.adr_dequantize_absmax_u8.argtypes = [vp, vp, vp, vp, i32, i32, i32]
    L.adr_quantize_absmax_u8.argtypes = [vp, vp, vp, vp, i32, i32, i32]
    L.adr_dequantize_absmax_uint8.argtypes = [vp, TensorDesc, TensorDesc, TensorDesc]
    L.adr_quantize_absmax_uint8.argtypes = [vp, TensorDesc, TensorDesc, TensorDesc]
    L.adr_matmul_f16_plan.argtypes = [C.c_char_p, i32] + [i32] * 13 + [u32, u32, u32]
    L.adr_matmul_nt_fp16u8_plan.argtypes = [C.c_char_p, i32, i32, i32, i32, i32]
    L.adr_softmax_rows.argtypes = [vp, vp, vp, i32, i32, i32, f32]
    L.adr_debug_knob.argtypes = [i32, i32]
    L.adr_microbench_empty.argtypes = [vp]
    L.adr_microbench_mfma_f16.argtypes = [vp, i32, i32, i32, vp]
    L.adr_microbench_stream_read.argtypes = [vp, vp, C.c_int64, i32, vp]
    L.adr_error_stats_f16.argtypes = [vp, TensorDesc, TensorDesc, TensorDesc]
    L.adr_error_stats_f32.argtypes = [vp, TensorDesc, TensorDesc, TensorDesc]
    L.adr_attention_f16.argtypes = [vp, vp, vp, vp, vp] + [i32] * 16 + [f32, f32, u32]
    L.adr_embed_uint8.argtypes = [vp, i32, i32, vp, vp, vp, vp, i32]
    L.adr_strerror.argtypes = [C.c_int]
    L.adr_strerror.restype = C.c_char_p
    L.adr_abi_version.restype = C.c_int
    for name in SYMBOLS:
        if name not in ("adr_strerror",):
            getattr(L, name).restype = C.c_int
    L.adr_matmul_f16_workspace_bytes.restype = C.c_int64
    L.adr_held_workspace_limit.restype = C.c_int64
    L.adr_held_workspace_bytes.restype = C.c_int64
    L.adr_held_workspace_declined.restype = C.c_int64
    L.adr_matmul_nt_fp16u8_workspace_bytes.restype = C.c_int64
    _lib = L
    return L


def strerror(code: int) -> str:
    return lib().adr_strerror(code).decode()
