"""The launcher of the reference's own device kernels lives with the oracle (oracle/refgpu.py);
the GPU parity tests import it under this name."""
from oracle.refgpu import *  # noqa: F401,F403
from oracle.refgpu import REF_DIR, RefKernels, available, has  # noqa: F401
