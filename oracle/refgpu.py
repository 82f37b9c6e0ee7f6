"""Loads the reference's own device kernels -- compiled from their sources where they lie in the
reference checkout into gfx950 code objects under oracle/_ref/ by oracle/Makefile -- and launches
them through the HIP module API.  Used by the GPU parity tests as a second checker beside the C
oracle, and by the baseline leg of bench.py to time the reference's own kernel on the same
device.  Test infrastructure only; skipped when oracle/_ref/ was not built.

Launch geometry follows the reference host code: adrastea_models/src/kernels.rs:783-792
(naive matmul_f16), :849-863 (matmul_f16_fast).
"""
import ctypes as C
import os

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_DIR = os.path.join(ROOT, "oracle", "_ref")
LEGACY_DIR = os.path.join(ROOT, "adrastea_amd", "lib", "legacy")

QUANTIZE_SYM = b"_Z21quantize_absmax_uint810TensorViewIhES_I6__halfES2_"
DEQUANTIZE_SYM = b"_Z23dequantize_absmax_uint810TensorViewI6__halfES1_S_IhE"


def available():
    return all(os.path.exists(os.path.join(REF_DIR, f))
               for f in ("matmul.co", "quantize.co", "matmul_nt_fp16u8.co"))


def has(name):
    return os.path.exists(os.path.join(REF_DIR, name))


class TensorDesc(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("dims", C.c_uint32), ("shape", C.c_uint32 * 7),
                ("strides", C.c_uint32 * 7)]


def desc2d(t):
    d = TensorDesc()
    d.ptr = t.data_ptr()
    d.dims = 2
    d.shape[0], d.shape[1] = t.shape[1], t.shape[0]
    d.strides[0], d.strides[1] = t.stride(1), t.stride(0)
    return d


class RefKernels:
    def __init__(self, directory=REF_DIR):
        """`directory` holds the code objects: the reference's own by default; the package's
        lib/legacy/ directory holds this build's modules with the same symbols and arguments."""
        import torch
        self.dir = directory
        torch.cuda.init()
        torch.zeros(1, device="cuda")  # make sure the primary context exists
        self.hip = C.CDLL("libamdhip64.so")
        self.hip.hipModuleLoad.argtypes = [C.POINTER(C.c_void_p), C.c_char_p]
        self.hip.hipModuleGetFunction.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_char_p]
        self.hip.hipModuleLaunchKernel.argtypes = ([C.c_void_p] + [C.c_uint] * 7 +
                                                   [C.c_void_p, C.POINTER(C.c_void_p), C.c_void_p])
        self.mods = {}
        self.fns = {}

    def _fn(self, module, name):
        key = (module, name)
        if key not in self.fns:
            if module not in self.mods:
                m = C.c_void_p()
                rc = self.hip.hipModuleLoad(C.byref(m), os.path.join(self.dir, module).encode())
                assert rc == 0, f"hipModuleLoad({module}) = {rc}"
                self.mods[module] = m
            f = C.c_void_p()
            rc = self.hip.hipModuleGetFunction(C.byref(f), self.mods[module], name)
            assert rc == 0, f"hipModuleGetFunction({name}) = {rc}"
            self.fns[key] = f
        return self.fns[key]

    def _launch(self, f, grid, block, shared, args):
        import torch
        holders = list(args)
        ptrs = (C.c_void_p * len(holders))(*[C.cast(C.byref(h), C.c_void_p) for h in holders])
        stream = torch.cuda.current_stream().cuda_stream
        rc = self.hip.hipModuleLaunchKernel(f, *grid, *block, shared, stream, ptrs, None)
        assert rc == 0, f"hipModuleLaunchKernel = {rc}"

    def _matmul_args(self, out_ptr, l_ptr, r_ptr, B, M, K, N, so, sl, sr, bias_ptr, beta, scale,
                     store, load, mask):
        ints = [B, M, K, N, so[0], so[1], so[2], sl[0], sl[1], sl[2], sr[0], sr[1], sr[2]]
        return ([C.c_void_p(out_ptr), C.c_void_p(l_ptr), C.c_void_p(r_ptr)] +
                [C.c_int(v) for v in ints] +
                [C.c_void_p(bias_ptr or 0), C.c_float(beta), C.c_float(scale), C.c_uint(store),
                 C.c_uint(load), C.c_uint(mask)])

    def matmul_f16(self, out_ptr, l_ptr, r_ptr, B, M, K, N, so, sl, sr, bias_ptr=None, beta=0.0,
                   scale=1.0, store=0, load=0, mask=0):
        """The naive kernel (matmul.cu:493-502)."""
        f = self._fn("matmul.co", b"matmul_f16")
        args = self._matmul_args(out_ptr, l_ptr, r_ptr, B, M, K, N, so, sl, sr, bias_ptr, beta,
                                 scale, store, load, mask)
        self._launch(f, ((N + 15) // 16, (M + 15) // 16, B), (16, 16, 1), 0, args)

    def matmul_f16_raw(self, out_ptr, l_ptr, r_ptr, B, M, K, N, so, sl, sr):
        """The identity-operator form (matmul.cu:515-517), launched like the naive kernel."""
        f = self._fn("matmul.co", b"matmul_f16_raw")
        args = self._matmul_args(out_ptr, l_ptr, r_ptr, B, M, K, N, so, sl, sr, None, 0.0, 1.0,
                                 0, 0, 0)[:16]
        self._launch(f, ((N + 15) // 16, (M + 15) // 16, B), (16, 16, 1), 0, args)

    def matmul_f16_fast(self, out_ptr, l_ptr, r_ptr, B, M, K, N, so, sl, sr, bias_ptr=None,
                        beta=0.0, scale=1.0, store=0, load=0, mask=0):
        """The tiled production kernel (matmul.cu:504-513)."""
        f = self._fn("matmul.co", b"matmul_f16_fast")
        args = self._matmul_args(out_ptr, l_ptr, r_ptr, B, M, K, N, so, sl, sr, bias_ptr, beta,
                                 scale, store, load, mask)
        shared = 16 * (32 + 2) * 2 + 32 * (32 + 2) * 2
        self._launch(f, ((N + 31) // 32, (M + 15) // 16, B), (32, 4, 1), shared, args)

    def matmul_nt_fp16u8(self, out, lhs, rhs_q, scales, block_size, beta=0.0):
        m, p = lhs.shape
        n = rhs_q.shape[0]
        f = self._fn("matmul_nt_fp16u8.co", b"matmul_nt_fp16u8")
        args = [C.c_void_p(out.data_ptr()), C.c_void_p(lhs.data_ptr()),
                C.c_void_p(rhs_q.data_ptr()), C.c_void_p(scales.data_ptr()), C.c_int(m),
                C.c_int(p), C.c_int(n), C.c_int(block_size), C.c_float(beta)]
        self._launch(f, ((n + 15) // 16, (m + 15) // 16, 1), (16, 16, 1), 0, args)

    def dequantize(self, out, scales, q):
        f = self._fn("quantize.co", DEQUANTIZE_SYM)
        args = [desc2d(out), desc2d(scales), desc2d(q)]
        self._launch(f, (scales.shape[1], q.shape[0], 1), (32, 1, 1), 0, args)

    def quantize(self, q, scales, x):
        f = self._fn("quantize.co", QUANTIZE_SYM)
        args = [desc2d(q), desc2d(scales), desc2d(x)]
        self._launch(f, (scales.shape[1], x.shape[0], 1), (32, 1, 1), 0, args)

    def embed_uint8(self, out, ids, table, scales, block_size):
        """embed_uint8.cu:3-19, one thread per id (256-thread blocks)."""
        f = self._fn("embed_uint8.co", b"embed_uint8")
        n_ids, n_dim = ids.numel(), table.shape[1]
        args = [C.c_int(n_dim), C.c_int(n_ids), C.c_void_p(ids.data_ptr()),
                C.c_void_p(out.data_ptr()), C.c_void_p(table.data_ptr()),
                C.c_void_p(scales.data_ptr()), C.c_int(block_size)]
        self._launch(f, ((n_ids + 255) // 256, 1, 1), (256, 1, 1), 0, args)

    def softmax_rows(self, out, inp, heads, h, w, temp=1.0):
        """normalize.cu:147-220 with the launch of kernels.rs:892-915 ((h, heads) x 256)."""
        f = self._fn("normalize.co", b"softmax_rows")
        args = [C.c_void_p(out.data_ptr()), C.c_void_p(inp.data_ptr()), C.c_int(h), C.c_int(w),
                C.c_float(temp)]
        self._launch(f, (h, heads, 1), (256, 1, 1), 0, args)

    def error_stats(self, out, lhs, rhs):
        """error_stats.cu:64-75 with the launch of kernels.rs:736-751 (128 blocks x 1024)."""
        import torch
        name = b"error_stats_f32" if lhs.dtype == torch.float32 else b"error_stats_f16"
        f = self._fn("error_stats.co", name)

        def d1(t):
            d = TensorDesc()
            d.ptr, d.dims = t.data_ptr(), 1
            d.shape[0], d.strides[0] = t.numel(), 1
            return d
        self._launch(f, (128, 1, 1), (1024, 1, 1), 0, [d1(out), d1(lhs), d1(rhs)])
