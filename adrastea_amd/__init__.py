"""adrastea_amd -- gfx950 (MI355X) implementation of adrastea's matrix-multiplication hot path.

The product is the C-ABI library ``lib/libadrastea_kernels_hip.so`` (hand-written HIP kernels,
declared in ``include/adrastea_kernels.h``).  This package is its host side for Python callers:
``tensor`` mirrors the reference's ``TensorLayout`` stride algebra and ``kernels`` mirrors the
``CommonKernels`` matmul interface (``adrastea_models/src/kernels.rs``), lowering tensor views
to the argument tuple of the C ABI.  There is no CPU fallback: without the built library, or
without a GPU, calls raise.
"""
from .tensor import TensorLayout, TensorView  # noqa: F401
from .kernels import (  # noqa: F401
    CommonKernels, GpuKernels, MatmulLoad, MatmulMask, MatmulOptions, MatmulStore, MatmulTracer,
    AdrasteaError, set_held_workspace_limit, held_workspace_limit, held_workspace_bytes,
    held_workspace_declined, release_held_workspace, set_u8_dequantise_first,
)
