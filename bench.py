#!/usr/bin/env python3
"""Benchmark of the matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

A "step" is one pass over the LLaMA-7B per-layer GEMM set at prefill M=2048 in fp16
(QKV 4096->12288, O 4096->4096, gate and up 4096->11008, down 11008->4096; 828.9 GFLOP),
every launch going through the C ABI (adr_matmul_f16) with operands resident in HBM.
Prints ONE JSON line.  `value` is the fp16 TFLOP/s of that step; `roofline` is the dominant
kernel (the MFMA GEMM on the QKV shape) timed with HIP events on the launch stream;
`roofline_u8_gemv` is the same for the u8 decode GEMV (the other half of the metric), with a
plain streaming read of the same bytes timed beside it; `cpu_baseline` is the CPU side of every
benchmark configuration on bounded samples, timed on this machine's host cores: torch-CPU fp32
matmul on the same seeded fp16 inputs (the style of the reference's py/gen_tests generator), a
blocked OpenMP fp32 GEMM (the counterpart of its host sgemm) and the scalar restatement of its
kernel; `secondary` carries the other benchmark configurations: the u8 decode GEMV in GB/s
against the HBM peak, the u8 prefill GEMMs, the CLIP GEMMs and the attention products.

Input data is synthetic (seeded): activations ~ N(0,1), weights ~ N(0,1/sqrt(K)) in fp16;
u8 weights uniform with fp16 scales ~ U(0.001, 0.02) per 32 weights.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_F16_TFLOPS = 2516.6   # 256 CU x 4 SIMD x 1024 flop/clk x 2.4 GHz (dense, no sparsity)
PEAK_HBM_GBS = 8000.0      # HBM3E
METRIC = "fp16 GEMM TFLOP/s (% MFMA peak); u8 GEMV GB/s (% HBM peak), LLaMA-7B"

LAYER_SET = [  # (name, K, N) at M = 2048
    ("qkv", 4096, 12288), ("o", 4096, 4096), ("gate", 4096, 11008), ("up", 4096, 11008),
    ("down", 11008, 4096),
]
DECODE_SET = [(4096, 4096), (4096, 11008), (4096, 12288), (11008, 4096)]


def profile_figures(name):
    """The machine-readable lines of a rocprofv3 summary under profiles/: `@bench key=value ...`
    (figures measured with counters, which this script cannot collect itself)."""
    out = {}
    try:
        with open(os.path.join(ROOT, "profiles", name)) as f:
            for line in f:
                if line.startswith("@bench "):
                    for item in line.split()[1:]:
                        k, _, v = item.partition("=")
                        try:
                            out[k] = float(v)
                        except ValueError:
                            out[k] = v
    except OSError:
        pass
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--quick", action="store_true", help="skip secondary configs and CPU baseline")
    ap.add_argument("--decode-only", action="store_true",
                    help="run only the u8 decode GEMV configurations (for profiling that kernel)")
    ap.add_argument("--attention-only", action="store_true",
                    help="run only the attention configuration (QK^T, softmax_rows, P.V, error_stats)")
    ap.add_argument("--u8-prefill-only", action="store_true",
                    help="run only the u8-weight prefill GEMMs of the layer set (for profiling that kernel)")
    ap.add_argument("--clip-only", action="store_true",
                    help="run only the CLIP GEMM configurations (for profiling those tiles)")
    ap.add_argument("--microbenchmark", action="store_true",
                    help="launch overhead, matrix-core issue peak, streaming-read peak and the "
                         "2048x4096x4096 products of the reference's microbenchmark()")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed replays of the step for this many milliseconds before the declared "
                         "warm-up (the clocks of a cold device settle under load); reported as settle_ms")
    ap.add_argument("--step-trace", action="store_true",
                    help="time each of the first 300 replays of the step graph on its own (HIP events), "
                         "from a cold start, and print them: shows how long the device takes to settle")
    ap.add_argument("--phase-stamps", action="store_true",
                    help="per-workgroup timeline of the tiled fp16 GEMM on the layer set (prologue, K loop, "
                         "epilogue, rounds), from the diagnostic build of the library that stamps them")
    ap.add_argument("--forced-tiles", action="store_true",
                    help="every fp16 tile forced (adr_debug_knob) on the benchmark's fp16 GEMM shapes "
                         "beside the tile the dispatch chooses: guards the dispatch's fitted constants")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain 256 MiB device copy (reference point for the "
                         "FETCH_SIZE / WRITE_SIZE counters of rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures the single-GPU matmul path only; run with --gpus 1 "
              "(every GPU box of this build has one GPU; no collectives are part of it)",
              file=sys.stderr)
        sys.exit(2)

    import torch
    from adrastea_amd import _ffi
    if args.phase_stamps:
        # the diagnostic twin (adrastea_amd.build.build_stamps_library): same kernels, plus stamps
        _ffi.LIB_PATH = os.path.join(os.path.dirname(_ffi.LIB_PATH), "libadrastea_kernels_hip_stamps.so")
    lib = _ffi.lib()  # raises if the HIP library is not built: there is no fallback
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    dev = "cuda:0"
    torch.cuda.set_device(0)
    if args.copy_calibration:
        src = torch.ones(256 << 20, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": 256 << 20, "launches": 5}))
        return
    gen = torch.Generator(device=dev).manual_seed(42)
    stream = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

    def randn_h(*shape, std=1.0):
        return (torch.randn(*shape, generator=gen, device=dev) * std).half()

    def mm(out, a, w, M, K, N):
        rc = lib.adr_matmul_f16(stream(), out.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N,
                                1, N, 0, 1, K, 0, K, 1, 0, None, 0.0, 1.0, 0, 0, 0)
        if rc != 0:
            raise RuntimeError(f"adr_matmul_f16 failed: {_ffi.strerror(rc)}")

    def timed(fn, iters, warm):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(iters):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / iters  # seconds per call

    def timed_graph(fn, calls_per_graph, replays, warm_replays=3):
        """Kernels of a few microseconds cannot be issued fast enough from Python: record
        `calls_per_graph` launches into a HIP graph and time its replays (HIP events on the
        launch stream), so that the figure is the device time per launch."""
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            fn()  # first call outside capture (lazy module loading)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(calls_per_graph):
                fn()
        for _ in range(warm_replays):
            graph.replay()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(replays):
            graph.replay()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) * 1e-3 / (replays * calls_per_graph)

    # ---- u8 decode GEMV (benchmark configs[2]): weight buffers rotate through > 256 MB so
    # that repeats stream from HBM, not from the Infinity Cache
    def u8_case(m, K, N, iters, probe=False):
        per = N * K + N * (K // 32) * 2
        nbuf = max(2, int(600e6 // per) + 1)
        qs = [torch.randint(0, 256, (N, K), generator=gen, device=dev, dtype=torch.uint8)
              for _ in range(nbuf)]
        ss = [(torch.rand(N, K // 32, generator=gen, device=dev) * 0.019 + 0.001).half()
              for _ in range(nbuf)]
        a = randn_h(m, K)
        o = torch.zeros(m, N, dtype=torch.float16, device=dev)
        i = [0]

        def f():
            j = i[0] % nbuf
            i[0] += 1
            rc = lib.adr_matmul_nt_fp16u8(stream(), o.data_ptr(), a.data_ptr(),
                                          qs[j].data_ptr(), ss[j].data_ptr(), m, K, N, 32, 0.0)
            if rc != 0:
                raise RuntimeError(_ffi.strerror(rc))
        t = timed_graph(f, 2 * nbuf, max(2, iters // (2 * nbuf)))
        t_probe = None
        if probe:
            # a plain streaming read of the same weight bytes (one contiguous piece per workgroup,
            # nothing computed, nothing written) through the same rotation and the same graph
            # replays: what this part delivers for this many bytes in one launch
            sink = torch.zeros(1, dtype=torch.int32, device=dev)
            best = None
            for blocks in (1024, 2048, 4096):
                if (N * K) % (16 * blocks):
                    continue

                def g():
                    j = i[0] % nbuf
                    i[0] += 1
                    rc = lib.adr_microbench_stream_read(stream(), qs[j].data_ptr(), N * K, blocks,
                                                        sink.data_ptr())
                    if rc != 0:
                        raise RuntimeError(_ffi.strerror(rc))
                tp = timed_graph(g, 2 * nbuf, max(2, iters // (2 * nbuf)))
                best = tp if best is None else min(best, tp)
            t_probe = best
        return t, per + m * K * 2 + m * N * 2, t_probe

    # ---- the same decode shapes with fp16 weights: the call the reference's LLaMA makes once per
    # generated token (matmul_f16 on a [tokens, K] activation, llama.rs:485-591)
    def f16_decode_set():
        rows = []
        for K, N in DECODE_SET:
            per = N * K * 2
            nbuf = max(2, int(600e6 // per) + 1)
            ws = [randn_h(N, K, std=K ** -0.5) for _ in range(nbuf)]
            for m in (1, 4, 8, 16):
                a = randn_h(m, K)
                o = torch.zeros(m, N, dtype=torch.float16, device=dev)
                i = [0]

                def f():
                    j = i[0] % nbuf
                    i[0] += 1
                    mm(o, a, ws[j], m, K, N)
                t = timed_graph(f, 2 * nbuf, max(2, 200 // (2 * nbuf)))
                byts = per + m * K * 2 + m * N * 2
                rows.append({"M": m, "K": K, "N": N, "us": round(t * 1e6, 2),
                             "gbs": round(byts / t / 1e9, 1),
                             "frac_hbm_peak": round(byts / t / 1e9 / PEAK_HBM_GBS, 4)})
            del ws
        return rows

    def short_prompt_set():
        """fp16 products with the row counts of a short prompt (the reference's LLaMA issues them
        for every generated token, llama.rs:456-483), as a caller without graphs makes them: eager
        launches timed with events, weights rotated through > 600 MB.  `us`: the entry point as it
        comes (K split over workgroups where that pays, through a buffer the library holds per
        stream); `unsplit_us`: with adr_set_held_workspace_limit(0)."""
        rows = []
        for K, N in DECODE_SET:
            per = N * K * 2
            nbuf = max(2, int(600e6 // per) + 1)
            ws = [randn_h(N, K, std=K ** -0.5) for _ in range(nbuf)]
            for m in (96, 128, 256, 512):
                a = randn_h(m, K)
                o = torch.zeros(m, N, dtype=torch.float16, device=dev)
                i = [0]

                def f():
                    j = i[0] % nbuf
                    i[0] += 1
                    mm(o, a, ws[j], m, K, N)
                t = timed(f, 4 * nbuf, nbuf)
                lib.adr_set_held_workspace_limit(0)
                t0 = timed(f, 4 * nbuf, nbuf)
                lib.adr_set_held_workspace_limit(_ffi.HELD_WORKSPACE_DEFAULT_BYTES)
                rows.append({"M": m, "K": K, "N": N, "us": round(t * 1e6, 1),
                             "unsplit_us": round(t0 * 1e6, 1),
                             "tflops": round(2.0 * m * K * N / t / 1e12, 1)})
            del ws
        return rows

    def u8_short_prompt_set():
        """The same row counts against u8 weights: `us` as the entry point comes (the streaming
        kernels in passes of 64 rows, or the tiled u8 kernel on its small tiles),
        `dequantise_first_us` after adr_set_u8_dequantise_first(1) (from 768 rows on the matrix is
        dequantised once into a buffer of the library's pool and the fp16 kernels run on it; below,
        the switch changes nothing)."""
        rows = []
        for K, N in DECODE_SET:
            per = N * K + N * (K // 32) * 2
            nbuf = max(2, int(600e6 // per) + 1)
            qs = [torch.randint(0, 256, (N, K), generator=gen, device=dev, dtype=torch.uint8)
                  for _ in range(nbuf)]
            ss = [(torch.rand(N, K // 32, generator=gen, device=dev) * 0.019 + 0.001).half()
                  for _ in range(nbuf)]
            for m in (96, 128, 256, 512, 1024):
                a = randn_h(m, K)
                o = torch.zeros(m, N, dtype=torch.float16, device=dev)
                i = [0]

                def f():
                    j = i[0] % nbuf
                    i[0] += 1
                    rc = lib.adr_matmul_nt_fp16u8(stream(), o.data_ptr(), a.data_ptr(), qs[j].data_ptr(),
                                                  ss[j].data_ptr(), m, K, N, 32, 0.0)
                    if rc != 0:
                        raise RuntimeError(_ffi.strerror(rc))
                t = timed(f, 4 * nbuf, nbuf)
                lib.adr_set_u8_dequantise_first(1)
                t1 = timed(f, 4 * nbuf, nbuf)
                lib.adr_set_u8_dequantise_first(0)
                rows.append({"M": m, "K": K, "N": N, "us": round(t * 1e6, 1),
                             "dequantise_first_us": round(t1 * 1e6, 1)})
            del qs, ss
        return rows

    def decode_set(ms=(1, 4, 16)):
        gemv = []
        for K, N in DECODE_SET:
            for m in ms:
                t, byts, tp = u8_case(m, K, N, 200, probe=(m == 1))
                row = {"M": m, "K": K, "N": N, "us": round(t * 1e6, 2),
                       "gbs": round(byts / t / 1e9, 1),
                       "frac_hbm_peak": round(byts / t / 1e9 / PEAK_HBM_GBS, 4)}
                if tp is not None:
                    row["plain_read_of_the_weights_us"] = round(tp * 1e6, 2)
                gemv.append(row)
        return gemv

    def attention_set():
        # ---- attention products (configs[3]): HBM-bound by the [32, 2048, 2048] fp16 tensor
        S, H, D = 2048, 32, 128
        HD = H * D
        q_, k_, v_ = randn_h(S, HD), randn_h(S, HD), randn_h(S, HD)
        qk = torch.zeros(H, S, S, dtype=torch.float16, device=dev)

        def f_qk(mask=0):
            rc = lib.adr_matmul_f16(stream(), qk.data_ptr(), q_.data_ptr(), k_.data_ptr(), H, S, D,
                                    S, 1, S, S * S, 1, HD, D, HD, 1, D, None, 0.0,
                                    1.0 / D ** 0.5, 4, 0, mask)
            if rc != 0:
                raise RuntimeError(_ffi.strerror(rc))
        t = timed(f_qk, 50, 5)
        byts = 2 * S * HD * 2 + H * S * S * 2
        attn = {"qk_t": {"us": round(t * 1e6, 1), "tflops": round(2.0 * H * S * S * D / t / 1e12, 1),
                         "gbs": round(byts / t / 1e9, 1),
                         "frac_hbm_peak": round(byts / t / 1e9 / PEAK_HBM_GBS, 4)}}
        # the same product under the causal mask (llama.rs:534-545): the same bytes are written,
        # half of them -inf by a fill launch of their own, and half the arithmetic is done
        t = timed(lambda: f_qk(1), 50, 5)
        attn["qk_t_causal"] = {"us": round(t * 1e6, 1), "gbs": round(byts / t / 1e9, 1),
                               "frac_hbm_peak": round(byts / t / 1e9 / PEAK_HBM_GBS, 4),
                               "launches": "fill_causal_rows_kernel + gemm_nt_shortk_kernel"}
        # softmax_rows in place on the scores (read + write of the [32, 2048, 2048] tensor)
        def f_sm():
            rc = lib.adr_softmax_rows(stream(), qk.data_ptr(), qk.data_ptr(), H, S, S, 1.0)
            if rc != 0:
                raise RuntimeError(_ffi.strerror(rc))
        f_qk()
        t = timed(f_sm, 30, 3)
        sm_bytes = 2 * H * S * S * 2
        attn["softmax_rows"] = {"us": round(t * 1e6, 1), "gbs": round(sm_bytes / t / 1e9, 1),
                                "frac_hbm_peak": round(sm_bytes / t / 1e9 / PEAK_HBM_GBS, 4)}
        f_qk()
        p_ = torch.softmax(qk.float(), dim=-1).half()
        o_ = torch.zeros(S, HD, dtype=torch.float16, device=dev)

        def f_pv():
            rc = lib.adr_matmul_f16(stream(), o_.data_ptr(), p_.data_ptr(), v_.data_ptr(), H, S, S,
                                    D, 1, HD, D, 1, S, S * S, 1, HD, D, None, 0.0, 1.0, 0, 0, 0)
            if rc != 0:
                raise RuntimeError(_ffi.strerror(rc))
        t = timed(f_pv, 50, 5)
        attn["pv"] = {"us": round(t * 1e6, 1), "tflops": round(2.0 * H * S * S * D / t / 1e12, 1),
                      "gbs": round(byts / t / 1e9, 1),
                      "frac_hbm_peak": round(byts / t / 1e9 / PEAK_HBM_GBS, 4)}
        # error_stats_f16 of two [32, 2048, 2048] tensors (reads 2 x 268 MB, the on-device check)
        stat = torch.zeros(3, dtype=torch.float32, device=dev)

        def desc1(t):
            d = _ffi.TensorDesc()
            d.ptr, d.dims = t.data_ptr(), 1
            d.shape[0], d.strides[0] = t.numel(), 1
            return d
        d_out, d_l, d_r = desc1(stat), desc1(qk), desc1(p_)

        def f_es():
            rc = lib.adr_error_stats_f16(stream(), d_out, d_l, d_r)
            if rc != 0:
                raise RuntimeError(_ffi.strerror(rc))
        t = timed(f_es, 30, 3)
        attn["error_stats_f16"] = {"us": round(t * 1e6, 1), "gbs": round(sm_bytes / t / 1e9, 1),
                                   "frac_hbm_peak": round(sm_bytes / t / 1e9 / PEAK_HBM_GBS, 4)}
        # QK^T -> softmax_rows in place -> P.V back to back, as a model runs them: each launch
        # then finds its input in HBM, not in the cache its own previous run left behind
        def f_seq():
            f_qk()
            f_sm()
            rc = lib.adr_matmul_f16(stream(), o_.data_ptr(), qk.data_ptr(), v_.data_ptr(), H, S, S,
                                    D, 1, HD, D, 1, S, S * S, 1, HD, D, None, 0.0, 1.0, 0, 0, 0)
            if rc != 0:
                raise RuntimeError(_ffi.strerror(rc))
        t = timed(f_seq, 30, 3)
        seq_bytes = 2 * byts + sm_bytes
        attn["qk_softmax_pv_sequence"] = {"us": round(t * 1e6, 1), "gbs": round(seq_bytes / t / 1e9, 1),
                                          "frac_hbm_peak": round(seq_bytes / t / 1e9 / PEAK_HBM_GBS, 4)}
        # the three products and the softmax above as one launch (adr_attention_f16); the causal
        # form is what the LLaMA layer runs, and skips the masked half of the score tiles
        o_ = torch.zeros(S, HD, dtype=torch.float16, device=dev)
        for name, msk in (("fused_attention", 0), ("fused_attention_causal", 1)):
            def f_at():
                rc = lib.adr_attention_f16(stream(), o_.data_ptr(), q_.data_ptr(), k_.data_ptr(),
                                           v_.data_ptr(), H, S, S, D, 1, HD, D, 1, HD, D, 1, HD, D,
                                           1, HD, D, 1.0 / D ** 0.5, 1.0, msk)
                if rc != 0:
                    raise RuntimeError(_ffi.strerror(rc))
            t = timed(f_at, 30, 3)
            fl = 4.0 * H * S * S * D * (0.5 if msk else 1.0)
            attn[name] = {"us": round(t * 1e6, 1), "tflops": round(fl / t / 1e12, 1),
                          "frac_mfma_peak": round(fl / t / 1e12 / PEAK_F16_TFLOPS, 4)}
        return attn

    def other_lengths_set():
        # ---- P.V where the sequence length is no multiple of 64 (the probabilities' rows then
        # start at any even address) or the query rows are few: the lengths the reference's models
        # run at (llama.rs:552-554, whisper.rs:433-436, clip.rs:385-388); device time per launch
        # from graph replays
        out = {}
        for name, H, S, T, D in (("llama_S2001", 32, 2001, 2001, 128), ("llama_S1000", 32, 1000, 1000, 128),
                                 ("llama_1_row_T2047", 32, 1, 2047, 128),
                                 ("whisper_encoder_1500", 20, 1500, 1500, 64),
                                 ("whisper_cross_448_rows", 20, 448, 1500, 64),
                                 ("whisper_cross_8_rows", 20, 8, 1500, 64),
                                 ("clip_vision_257", 16, 257, 257, 64), ("clip_text_77", 12, 77, 77, 64)):
            HD = H * D
            p_ = torch.softmax(randn_h(H, S, T).float(), dim=-1).half()
            v_, o_ = randn_h(T, HD), torch.zeros(S, HD, dtype=torch.float16, device=dev)

            def f():
                rc = lib.adr_matmul_f16(stream(), o_.data_ptr(), p_.data_ptr(), v_.data_ptr(), H, S, T,
                                        D, 1, HD, D, 1, T, S * T, 1, HD, D, None, 0.0, 1.0, 0, 0, 0)
                if rc != 0:
                    raise RuntimeError(_ffi.strerror(rc))
            plan = ctypes.create_string_buffer(96)
            lib.adr_matmul_f16_plan(plan, 96, H, S, T, D, 1, HD, D, 1, T, S * T, 1, HD, D, 0, 0, 0)
            t = timed_graph(f, 10, 10)
            byts = (H * S * T + T * HD + S * HD) * 2
            out["pv_" + name] = {"us": round(t * 1e6, 1), "kernel": plan.value.decode(),
                                 "tflops": round(2.0 * H * S * T * D / t / 1e12, 1),
                                 "gbs": round(byts / t / 1e9, 1)}
        return out

    if args.attention_only:
        print(json.dumps({"llama7b_attention_fp16": attention_set(),
                          "pv_other_lengths_fp16": other_lengths_set()}))
        return

    def microbenchmark():
        """The list of adrastea/src/main.rs:486-650 (`microbenchmark()`), each entry run for about
        a second like its bench() (main.rs:409-454): per-call wall time including the
        synchronisation, reported as fastest / average / slowest rate."""
        def run(name, ops, call, unit, seconds=1.0):
            call()
            torch.cuda.synchronize()
            times = []
            t_end = time.perf_counter() + seconds
            while time.perf_counter() < t_end and len(times) < 100000:
                t0 = time.perf_counter()
                call()
                torch.cuda.synchronize()
                times.append(time.perf_counter() - t0)
            scale = 1e12 if unit == "TFLOP/s" else 1e9 if unit == "GB/s" else 1.0
            row = {"name": name, "ops": ops, "unit": unit, "runs": len(times)}
            if unit == "us":
                row.update(fast=round(min(times) * 1e6, 2), avg=round(sum(times) / len(times) * 1e6, 2),
                           slow=round(max(times) * 1e6, 2))
            else:
                row.update(fast=round(ops / min(times) / scale, 1),
                           avg=round(ops * len(times) / sum(times) / scale, 1),
                           slow=round(ops / max(times) / scale, 1))
            return row

        def ok(rc):
            if rc != 0:
                raise RuntimeError(_ffi.strerror(rc))
        rows = [run("empty_kernel", 1, lambda: ok(lib.adr_microbench_empty(stream())), "us")]
        blocks, times_ = 512, 20000   # two workgroups of four wavefronts per CU
        sink = torch.zeros(blocks * 256, dtype=torch.float32, device=dev)
        flop = blocks * 4 * times_ * 4 * 2 * 32 * 32 * 16
        for pattern, nm in ((0, "mfma_loop_f32_f16 (zero operands)"), (1, "mfma_loop_f32_f16 (random operands)"),
                            (2, "mfma_loop_f32_f16 (random operands, changing with every instruction)")):
            rows.append(run(nm, flop, lambda: ok(lib.adr_microbench_mfma_f16(
                stream(), blocks, times_, pattern, sink.data_ptr())), "TFLOP/s"))
        # the two MFMA shapes on a 128 x 128 wavefront tile, random operands: what decides which
        # one the GEMM kernels issue
        for pattern, nm, per in ((3, "mfma 32x32x16 on a 128x128 wavefront tile (random operands)", 1 << 20),
                                 (4, "mfma 16x16x32 on a 128x128 wavefront tile (random operands)", 1 << 21)):
            t_ = 4000 if pattern == 3 else 2000
            rows.append(run(nm, blocks * 4 * t_ * per, lambda: ok(lib.adr_microbench_mfma_f16(
                stream(), blocks, t_, pattern, sink.data_ptr())), "TFLOP/s"))
        nbytes = 1 << 30
        src = torch.ones(nbytes, dtype=torch.uint8, device=dev)
        sink32 = torch.zeros(1, dtype=torch.int32, device=dev)
        rows.append(run("stream_read 1 GiB", nbytes, lambda: ok(lib.adr_microbench_stream_read(
            stream(), src.data_ptr(), nbytes, 1024, sink32.data_ptr())), "GB/s"))
        del src
        # matmul_f16[_fast]_2048_4096_4096 with a row-major and a permuted right operand
        M, K, N = 2048, 4096, 4096
        left, out = randn_h(M, K), torch.zeros(M, N, dtype=torch.float16, device=dev)
        right = randn_h(K, N, std=K ** -0.5)  # rrr: [K, N] as stored; rrc: the same memory as [N, K]^T
        for fn_name, label in (("adr_matmul_f16_slow", "matmul_f16"), ("adr_matmul_f16", "matmul_f16_fast")):
            fn = getattr(lib, fn_name)
            for layout, (srx, sry) in (("rrr", (1, N)), ("rrc", (K, 1))):
                rows.append(run(f"{label}_2048_4096_4096_{layout}", 2 * M * K * N, lambda: ok(fn(
                    stream(), out.data_ptr(), left.data_ptr(), right.data_ptr(), 1, M, K, N, 1, N, 0,
                    1, K, 0, srx, sry, 0, None, 0.0, 1.0, 0, 0, 0)), "TFLOP/s"))
        # the library GEMM the reference compares itself with (rocBLAS hgemm there, main.rs:599-648;
        # torch.matmul dispatches to hipBLASLt / rocBLAS here)
        rt = right.t().contiguous()
        rows.append(run("library_hgemm_2048_4096_4096 (torch.matmul)", 2 * M * K * N,
                        lambda: torch.matmul(left, right), "TFLOP/s"))
        rows.append(run("library_hgemm_2048_4096_4096_nt (torch.matmul)", 2 * M * K * N,
                        lambda: torch.matmul(left, rt.t()), "TFLOP/s"))
        return rows

    if args.microbenchmark:
        rows = microbenchmark()
        print("%-48s %14s %12s %12s %12s" % ("name", "ops", "fast", "avg", "slow"), file=sys.stderr)
        for r in rows:
            print("%-48s %14d %12s %12s %12s  %s" % (r["name"], r["ops"], r["fast"], r["avg"], r["slow"],
                                                     r["unit"]), file=sys.stderr)
        print(json.dumps({"microbenchmark": rows}))
        return

    if args.decode_only:
        # (with the row counts of a short prompt: the reference's LLaMA re-runs the whole sequence
        # for every token, llama.rs:456-483, so these are calls it makes too)
        print(json.dumps({"u8_decode_gemv": decode_set(), "f16_decode_gemv": f16_decode_set(),
                          "u8_17_to_128_rows": decode_set((32, 64, 128)),
                          "f16_short_prompt_rows": short_prompt_set(),
                          "u8_short_prompt_rows": u8_short_prompt_set()}))
        return

    def u8_prefill_set():
        """u8 prefill GEMMs (configs[4], u8 half): the layer set at M = 2048 with u8 weights."""
        M = 2048
        act = {4096: randn_h(M, 4096), 11008: randn_h(M, 11008)}
        u8p = {}
        for name, K, N in LAYER_SET:
            if name == "up":
                continue
            q = torch.randint(0, 256, (N, K), generator=gen, device=dev, dtype=torch.uint8)
            s = (torch.rand(N, K // 32, generator=gen, device=dev) * 0.019 + 0.001).half()
            out = torch.zeros(M, N, dtype=torch.float16, device=dev)

            def f():
                rc = lib.adr_matmul_nt_fp16u8(stream(), out.data_ptr(), act[K].data_ptr(),
                                              q.data_ptr(), s.data_ptr(), M, K, N, 32, 0.0)
                if rc != 0:
                    raise RuntimeError(_ffi.strerror(rc))
            # the entry point as it comes: the fused kernels (dequantisation inside the GEMM's K
            # loop, nothing written back), eagerly and under capture alike
            # (discarded: the clocks need tens of milliseconds of load to settle)
            timed(f, 200 if not u8p else 30, 5)
            t = timed(f, 50, 5)
            # on request (adr_set_u8_dequantise_first): the matrix dequantised once per call into a
            # buffer of the library's pool, then the fp16 kernels; same bits
            lib.adr_set_u8_dequantise_first(1)
            timed(f, 5, 2)   # (allocates the buffer)
            t_pool = timed(f, 50, 5)
            lib.adr_set_u8_dequantise_first(0)
            # the same product through adr_matmul_nt_fp16u8_ws with the caller's workspace
            ws = torch.empty(N * K * 2, dtype=torch.uint8, device=dev)

            def f_ws():
                rc = lib.adr_matmul_nt_fp16u8_ws(stream(), out.data_ptr(), act[K].data_ptr(),
                                                 q.data_ptr(), s.data_ptr(), M, K, N, 32, 0.0,
                                                 ws.data_ptr(), ws.numel())
                if rc != 0:
                    raise RuntimeError(_ffi.strerror(rc))
            t_ws = timed(f_ws, 50, 5)
            u8p[name] = {"M": M, "K": K, "N": N, "us": round(t * 1e6, 1),
                         "tflops": round(2.0 * M * K * N / t / 1e12, 1),
                         "frac_mfma_peak": round(2.0 * M * K * N / t / 1e12 / PEAK_F16_TFLOPS, 4),
                         "dequantise_first_us": round(t_pool * 1e6, 1),
                         "dequantise_first_tflops": round(2.0 * M * K * N / t_pool / 1e12, 1),
                         "with_workspace_us": round(t_ws * 1e6, 1),
                         "with_workspace_tflops": round(2.0 * M * K * N / t_ws / 1e12, 1)}
            del q, s, ws
        return u8p

    def clip_set():
        """CLIP GEMMs (configs[0], configs[1])."""

        clip = {}
        for nm, m, K, N in (("text_qkv_M77", 77, 768, 2304), ("vision_mlp_up", 2056, 1024, 4096),
                            ("vision_mlp_down", 2056, 4096, 1024)):
            a, w = randn_h(m, K), randn_h(N, K, std=K ** -0.5)
            o = torch.zeros(m, N, dtype=torch.float16, device=dev)
            # (launches of a few microseconds are timed as graph replays: Python cannot issue
            # them that fast)
            t = timed_graph(lambda: mm(o, a, w, m, K, N), 50, 20) if m < 256 else \
                timed(lambda: mm(o, a, w, m, K, N), 50, 5)
            byts = (m * K + N * K + m * N) * 2
            clip[nm] = {"M": m, "K": K, "N": N, "us": round(t * 1e6, 2),
                        "tflops": round(2.0 * m * K * N / t / 1e12, 1),
                        "frac_mfma_peak": round(2.0 * m * K * N / t / 1e12 / PEAK_F16_TFLOPS, 4),
                        "gbs": round(byts / t / 1e9, 1)}
        # the same two products with the store operators the CLIP MLP uses
        # (adrastea_models/src/clip.rs:431-442: QuickGeluBias on the way up, BetaBias 1.0 = residual add
        # on the way down); the operator runs in the kernel's epilogue
        for nm, K, N, store, beta in (("vision_mlp_up_quick_gelu_bias", 1024, 4096, 6, 0.0),
                                     ("vision_mlp_down_beta_bias", 4096, 1024, 3, 1.0)):
            m = 2056
            a, w = randn_h(m, K), randn_h(N, K, std=K ** -0.5)
            bias = randn_h(N)
            o = torch.zeros(m, N, dtype=torch.float16, device=dev)

            def f_op():
                rc = lib.adr_matmul_f16(stream(), o.data_ptr(), a.data_ptr(), w.data_ptr(), 1, m, K,
                                        N, 1, N, 0, 1, K, 0, K, 1, 0, bias.data_ptr(), beta, 1.0,
                                        store, 0, 0)
                if rc != 0:
                    raise RuntimeError(_ffi.strerror(rc))
            t = timed(f_op, 50, 5)
            clip[nm] = {"M": m, "K": K, "N": N, "us": round(t * 1e6, 2),
                        "tflops": round(2.0 * m * K * N / t / 1e12, 1),
                        "frac_mfma_peak": round(2.0 * m * K * N / t / 1e12 / PEAK_F16_TFLOPS, 4)}
        return clip

    TILE_NAMES = ["256x192", "256x128", "128x256", "128x192", "128x128", "128x64", "64x64", "256x160"]
    FP16_GEMM_SHAPES = [("clip_text_qkv", 77, 768, 2304), ("clip_mlp_up", 2056, 1024, 4096),
                        ("clip_mlp_down", 2056, 4096, 1024), ("llama_qkv", 2048, 4096, 12288),
                        ("llama_o", 2048, 4096, 4096), ("llama_gate_up", 2048, 4096, 11008),
                        ("llama_down", 2048, 11008, 4096)]

    def forced_tiles_set(shapes=FP16_GEMM_SHAPES, rounds=3):
        """For every fp16 GEMM shape of the benchmark: the dispatch's own choice and every tile
        forced, interleaved over `rounds` passes (best of the passes per variant, so that clock
        drift between variants cancels).  `chosen_over_best` near 1 says the fitted tile model
        still picks well on this machine."""
        import ctypes
        rows = []
        for nm, m, K, N in shapes:
            a, w = randn_h(m, K), randn_h(N, K, std=K ** -0.5)
            o = torch.zeros(m, N, dtype=torch.float16, device=dev)
            buf = ctypes.create_string_buffer(96)
            lib.adr_matmul_f16_plan(buf, 96, 1, m, K, N, 1, N, 0, 1, K, 0, K, 1, 0, 0, 0, 0)
            f = lambda: mm(o, a, w, m, K, N)   # noqa: E731
            iters = max(40, int(0.010 / max(timed(f, 20, 5), 1e-6)))
            best = {}
            try:
                for _ in range(rounds):
                    for t in range(len(TILE_NAMES) + 1):
                        lib.adr_debug_knob(0, t)
                        # (every measurement spans some ten milliseconds: shorter ones see the
                        # clock wander by a few percent)
                        us = (timed_graph(f, 50, 40) if m < 256 else timed(f, iters, 10)) * 1e6
                        key = "chosen" if t == 0 else TILE_NAMES[t - 1]
                        best[key] = min(best.get(key, 1e30), us)
            finally:
                lib.adr_debug_knob(0, 0)
            fastest = min(v for k, v in best.items() if k != "chosen")
            rows.append({"shape": nm, "M": m, "K": K, "N": N, "plan": buf.value.decode(),
                         "chosen_us": round(best["chosen"], 2),
                         "forced_us": {k: round(v, 2) for k, v in best.items() if k != "chosen"},
                         "chosen_over_best": round(best["chosen"] / fastest, 3)})
        return rows

    if args.forced_tiles:
        print(json.dumps({"forced_tiles": forced_tiles_set()}))
        return

    def phase_stamps_set():
        """Where the time of a tiled fp16 GEMM launch goes: every workgroup's start, prologue, K
        loop and epilogue (100 MHz real-time counter, averaged over its wavefronts), the loop's
        length in shader-clock cycles, and the rounds of workgroups over the compute units."""
        import numpy as np
        lib.adr_set_held_workspace_limit(0)
        M = 2048
        rows = []
        for name, K, N in LAYER_SET:
            if name == "up":
                continue
            a, w = randn_h(M, K), randn_h(N, K, std=K ** -0.5)
            o = torch.zeros(M, N, dtype=torch.float16, device=dev)
            wide = N > 4096
            bm, bn, nw = 256, (192 if wide else 128), 8
            tiles = ((M + bm - 1) // bm) * ((N + bn - 1) // bn)
            # MFMA issue cycles of one K slice on one SIMD: two wavefronts, each bm * bn / 8 outputs as
            # 16 x 16 blocks over two k-steps of 32, sixteen clocks per v_mfma_f32_16x16x32_f16
            ideal = bm * bn // 32
            st_buf = torch.zeros(tiles * nw * 10, dtype=torch.int64, device=dev)

            def call(ws):
                rc = (lib.adr_matmul_f16(stream(), o.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N, 1, N, 0, 1, K, 0,
                                         K, 1, 0, None, 0.0, 1.0, 0, 0, 0) if ws is None else
                      lib.adr_matmul_f16_ws(stream(), o.data_ptr(), a.data_ptr(), w.data_ptr(), 1, M, K, N, 1, N, 0, 1, K,
                                            0, K, 1, 0, None, 0.0, 1.0, 0, 0, 0, ws.data_ptr(), ws.numel() * 8))
                if rc != 0:
                    raise RuntimeError(_ffi.strerror(rc))
            timed(lambda: call(None), 300, 10)   # the clocks settle under this load
            t_event = timed(lambda: call(st_buf), 20, 5) * 1e6
            torch.cuda.synchronize()
            st = st_buf.cpu().numpy().reshape(tiles, nw, 10).astype(np.float64)
            r, c = st[:, :, 4:8] * 0.01, st[:, :, 0:4]   # microseconds; shader-clock cycles
            t0 = r[:, :, 0].min()
            start, end = r[:, 0, 0] - t0, r[:, :, 3].max(axis=1) - t0
            pro = (r[:, :, 1] - r[:, :, 0]).mean(axis=1)
            loop = (r[:, :, 2] - r[:, :, 1]).mean(axis=1)
            epi = (r[:, :, 3] - r[:, :, 2]).mean(axis=1)
            cyc = (c[:, :, 2] - c[:, :, 1]).mean(axis=1)
            order = np.argsort(start)
            cus = 256
            row = {"product": name, "M": M, "K": K, "N": N, "tile": f"{bm}x{bn}", "workgroups": tiles,
                   "launch_us_hip_events": round(t_event, 1), "first_start_to_last_end_us": round(float(end.max()), 1),
                   "mfma_issue_cycles_per_slice": ideal, "rounds": []}
            for lo in range(0, tiles, cus):
                sel = order[lo:lo + cus]
                row["rounds"].append({
                    "workgroups": int(len(sel)), "start_us_mean": round(float(start[sel].mean()), 2),
                    "prologue_us": round(float(pro[sel].mean()), 2), "k_loop_us": round(float(loop[sel].mean()), 2),
                    "epilogue_us_stores_acknowledged": round(float(epi[sel].mean()), 2),
                    "end_us_min_mean_max": [round(float(end[sel].min()), 2), round(float(end[sel].mean()), 2),
                                            round(float(end[sel].max()), 2)],
                    "k_loop_cycles_per_slice": round(float(cyc[sel].mean()) / (K // 64)),
                    "shader_clock_ghz_in_k_loop": round(float((cyc[sel] / loop[sel]).mean()) / 1e3, 3)})
            row["wavefront_skew_at_loop_end_us"] = round(float((r[:, :, 2].max(axis=1) - r[:, :, 2].min(axis=1)).mean()), 2)
            rows.append(row)
        return rows

    if args.phase_stamps:
        print(json.dumps({"phase_stamps": phase_stamps_set()}))
        return

    if args.u8_prefill_only:
        print(json.dumps({"llama7b_prefill_u8": u8_prefill_set()}))
        return

    if args.clip_only:
        print(json.dumps({"clip_fp16": clip_set()}))
        return

    # ---------------- primary workload: the fp16 layer GEMM set at M = 2048
    M = 2048
    acts = {4096: randn_h(M, 4096), 11008: randn_h(M, 11008)}
    weights, outs = {}, {}
    for name, K, N in LAYER_SET:
        weights[name] = randn_h(N, K, std=K ** -0.5)
        outs[name] = torch.zeros(M, N, dtype=torch.float16, device=dev)

    def step():
        for name, K, N in LAYER_SET:
            mm(outs[name], acts[K], weights[name], M, K, N)

    # The five launches of a step are recorded once into a HIP graph (under capture the entry
    # points neither allocate nor synchronise) and the step is replayed: the timed
    # region then holds the device work of K steps, not the rate at which Python can call.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()  # first call outside capture (lazy module loading)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    step_graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(step_graph):
        step()
    step_flops = sum(2.0 * M * K * N for _, K, N in LAYER_SET)
    if args.step_trace:
        # every replay between its own pair of events, starting cold (nothing has run but the
        # capture): replay i's time and the running mean of ten
        n_tr = 300
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(n_tr + 1)]
        ev[0].record()
        for i in range(n_tr):
            step_graph.replay()
            ev[i + 1].record()
        torch.cuda.synchronize()
        us = [round(ev[i].elapsed_time(ev[i + 1]) * 1e3, 1) for i in range(n_tr)]
        tail = sorted(us[200:])
        print(json.dumps({"step_trace_us": us, "median_of_replays_200_to_299_us": tail[len(tail) // 2],
                          "mean_of_replays_0_to_24_us": round(sum(us[:25]) / 25, 1),
                          "gflop_per_step": round(step_flops / 1e9, 1)}))
        return
    # Settle phase, untimed and reported: the clocks of a device that has been idle need some
    # hundred milliseconds of this load to reach their steady state (--step-trace shows it), the
    # reference's own harness runs every entry for up to five seconds for the same reason
    # (adrastea/src/main.rs:409-454).  The declared warm-up follows it.
    settle_t0 = time.perf_counter()
    settle_steps = 0
    while (time.perf_counter() - settle_t0) * 1e3 < args.settle_ms:
        for _ in range(10):
            step_graph.replay()
        torch.cuda.synchronize()
        settle_steps += 10
    for _ in range(args.warmup):
        step_graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step_graph.replay()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = step_flops / (elapsed / args.steps) / 1e12

    # ---------------- roofline of the dominant kernel (HIP events on the launch stream)
    name, K, N = LAYER_SET[0]
    t_qkv = timed(lambda: mm(outs[name], acts[K], weights[name], M, K, N), 200, 20)
    qkv_flops = 2.0 * M * K * N
    prof = profile_figures("gemm_nt_dma_llama7b_layer_set.txt")
    roofline = {
        "kernel": prof.get("kernel", "gemm_nt_dma_kernel") + " (qkv: M2048 K4096 N12288)",
        "bound": "mfma", "achieved": round(qkv_flops / t_qkv / 1e12, 2),
        "peak": PEAK_F16_TFLOPS, "unit": "TFLOP/s",
        "frac": round(qkv_flops / t_qkv / 1e12 / PEAK_F16_TFLOPS, 4),
        "launch_us": round(t_qkv * 1e6, 2),
        # bytes moved between L2 and the memory fabric per qkv launch: rocprofv3 --pmc FETCH_SIZE and
        # WRITE_SIZE passes (scaled by a plain device copy), read from the summary under profiles/
        "traffic": prof.get("traffic_bytes"),
        "traffic_algorithmic": float((M * K + N * K + M * N) * 2),
        "traffic_source": "profiles/gemm_nt_dma_llama7b_layer_set.txt",
    }

    if not args.quick:
        # Two reference points for that figure, same launch, same shape.  (1) Operands of zeros: the
        # instruction stream and the memory traffic are identical, only the switching activity in
        # the matrix pipe is gone -- the part is power limited under this kernel, and the
        # difference is what the power limit costs on real data.  (2) The vendor library
        # (torch.matmul -> hipBLASLt) on the same random operands.
        za, zw = torch.zeros_like(acts[K]), torch.zeros_like(weights[name])
        t_zero = timed(lambda: mm(outs[name], za, zw, M, K, N), 100, 20)
        wt = weights[name].t()
        t_lib = timed(lambda: torch.matmul(acts[K], wt, out=outs[name]), 100, 20)
        roofline["probe"] = {
            "same_launch_on_zero_operands_tflops": round(qkv_flops / t_zero / 1e12, 1),
            "library_hgemm_same_operands_tflops": round(qkv_flops / t_lib / 1e12, 1),
        }
        del za, zw

    secondary = {}
    roofline_u8 = None
    if not args.quick:
        per_gemm = {}
        for name, K, N in LAYER_SET:
            if name == "up":
                continue
            t = timed(lambda: mm(outs[name], acts[K], weights[name], M, K, N), 100, 10)
            per_gemm[name] = {"M": M, "K": K, "N": N, "us": round(t * 1e6, 1),
                              "tflops": round(2.0 * M * K * N / t / 1e12, 1),
                              "frac_mfma_peak": round(2.0 * M * K * N / t / 1e12 / PEAK_F16_TFLOPS, 4)}
        secondary["llama7b_prefill_fp16"] = per_gemm

        gemv = decode_set()
        secondary["u8_decode_gemv"] = gemv
        best = max(gemv, key=lambda r: r["gbs"])
        secondary["u8_decode_gemv_best"] = {"gbs": best["gbs"], "frac_hbm_peak": best["frac_hbm_peak"],
                                            "shape": [best["M"], best["K"], best["N"]]}
        # the other half of the metric: the dominant u8 decode kernel (one token, the widest
        # matrix of the layer) against the HBM peak
        dk = next(r for r in gemv if (r["M"], r["K"], r["N"]) == (1, 4096, 12288))
        dprof = profile_figures("gemv_u8_decode_llama7b.txt")
        roofline_u8 = {
            "kernel": "gemv_u8_dot_kernel<1,4,4,1> (M1 K4096 N12288)", "bound": "hbm",
            "achieved": dk["gbs"], "peak": PEAK_HBM_GBS, "unit": "GB/s",
            "frac": dk["frac_hbm_peak"], "launch_us": dk["us"],
            "traffic": dprof.get("traffic_bytes_m1_n12288"),
            "traffic_algorithmic": float(12288 * 4096 + 12288 * 128 * 2 + 4096 * 2 + 12288 * 2),
            "traffic_source": "profiles/gemv_u8_decode_llama7b.txt",
            "plain_read_of_the_weights_us": dk.get("plain_read_of_the_weights_us"),
            "rows_4": next(r for r in gemv if (r["M"], r["K"], r["N"]) == (4, 4096, 12288)),
            "rows_16": next(r for r in gemv if (r["M"], r["K"], r["N"]) == (16, 4096, 12288)),
        }

        secondary["f16_decode_gemv"] = f16_decode_set()

        secondary["llama7b_prefill_u8"] = u8_prefill_set()
        secondary["clip_fp16"] = clip_set()

        attn = attention_set()
        secondary["llama7b_attention_fp16"] = attn
        secondary["pv_other_lengths_fp16"] = other_lengths_set()

    # ---------------- CPU baseline: every configuration on bounded samples, this machine's cores
    cpu_baseline = None
    if not args.quick:
        import numpy as np
        import oracle  # checker / baseline only; never on the product path
        nproc = os.cpu_count() or 1
        threads = max(1, min(nproc, int(os.environ.get("OMP_NUM_THREADS", "16"))))
        torch.set_num_threads(threads)
        g_cpu = torch.Generator().manual_seed(42)   # seeded CPU generator, as py/gen_tests does

        def cpu_mm(m, K, N, reps, batch=None):
            """torch-CPU fp32 matmul on fp16-rounded inputs of the configuration's distribution."""
            shape_a, shape_w = ((m, K), (N, K)) if batch is None else ((batch, m, K), (batch, N, K))
            a32 = torch.randn(*shape_a, generator=g_cpu).half().float()
            w32 = (torch.randn(*shape_w, generator=g_cpu) * K ** -0.5).half().float()
            torch.matmul(a32, w32.transpose(-1, -2))  # warm-up
            t0 = time.perf_counter()
            for _ in range(reps):
                torch.matmul(a32, w32.transpose(-1, -2))
            return (time.perf_counter() - t0) / reps

        per_config = {}
        t = cpu_mm(77, 768, 2304, 50)
        per_config["configs[0] clip_text_qkv_M77_K768_N2304"] = {
            "sample": "whole problem, 50 runs", "ms": round(t * 1e3, 3),
            "tflops": round(2.0 * 77 * 768 * 2304 / t / 1e12, 4)}
        for nm, K, N in (("up_K1024_N4096", 1024, 4096), ("down_K4096_N1024", 4096, 1024)):
            t = cpu_mm(2056, K, N, 3)
            per_config[f"configs[1] clip_vision_mlp_M2056_{nm}"] = {
                "sample": "whole problem, 3 runs", "ms": round(t * 1e3, 2),
                "tflops": round(2.0 * 2056 * K * N / t / 1e12, 4)}
        # u8 decode: dequantise (the format's formula in fp32) + fp32 matmul, from the u8 weights
        Kd, Nd = 4096, 4096
        q_c = torch.randint(0, 256, (Nd, Kd), generator=g_cpu, dtype=torch.uint8)
        s_c = (torch.rand(Nd, Kd // 32, generator=g_cpu) * 0.019 + 0.001).half()
        for m in (1, 16):
            a_c = torch.randn(m, Kd, generator=g_cpu).half().float()
            t0 = time.perf_counter()
            w_c = (q_c.float() - 127.5) * s_c.float().repeat_interleave(32, dim=1)
            torch.matmul(a_c, w_c.t())
            t = time.perf_counter() - t0
            byts = Nd * Kd + Nd * (Kd // 32) * 2 + m * Kd * 2 + m * Nd * 2
            per_config[f"configs[2] u8_decode_M{m}_K4096_N4096"] = {
                "sample": "whole problem, dequantise + matmul, 1 run", "ms": round(t * 1e3, 2),
                "gbs": round(byts / t / 1e9, 2)}
        del q_c, s_c, w_c
        # attention products: 4 of the 32 heads (the heads are independent: time x 8 for the layer)
        S_, D_ = 2048, 128
        qh = torch.randn(4, S_, D_, generator=g_cpu).half().float()
        kh = torch.randn(4, S_, D_, generator=g_cpu).half().float()
        t0 = time.perf_counter()
        sc_ = torch.matmul(qh, kh.transpose(1, 2)) * D_ ** -0.5
        t_qk = time.perf_counter() - t0
        p_ = torch.softmax(sc_, dim=-1)
        t0 = time.perf_counter()
        torch.matmul(p_, qh)
        t_pv = time.perf_counter() - t0
        per_config["configs[3] attention_S2048_H32_D128"] = {
            "sample": "4 of 32 heads, 1 run (heads are independent: whole layer = 8 x)",
            "qk_t_ms_4_heads": round(t_qk * 1e3, 2), "pv_ms_4_heads": round(t_pv * 1e3, 2),
            "qk_t_tflops": round(2.0 * 4 * S_ * S_ * D_ / t_qk / 1e12, 4),
            "pv_tflops": round(2.0 * 4 * S_ * S_ * D_ / t_pv / 1e12, 4)}
        del qh, kh, sc_, p_
        # the layer set (headline workload): the whole step, all 2048 rows of each product
        rows = M
        t_set, fl_set = 0.0, 0.0
        for nm, K, N in LAYER_SET:
            t = cpu_mm(rows, K, N, 3)
            t_set += t
            fl_set += 2.0 * rows * K * N
        per_config["configs[4] llama7b_layer_set_fp16_M2048"] = {
            "sample": "the whole step: all 2048 rows of each of the five products, mean of 3 runs each",
            "ms_sample": round(t_set * 1e3, 1), "tflops": round(fl_set / t_set / 1e12, 4)}
        torch_value = fl_set / t_set / 1e12

        # the same qkv sample on the blocked OpenMP fp32 GEMM (counterpart of the reference's host
        # sgemm) and on the scalar restatement of its kernel (fp16 products, fp32 sum)
        name, K, N = LAYER_SET[0]
        a_np = acts[K][:128].cpu().numpy()
        w_np = weights[name].cpu().numpy()
        t0 = time.perf_counter()
        oracle.sgemm_nt(a_np.astype(np.float32), w_np.astype(np.float32), threads=threads)
        dt = time.perf_counter() - t0
        sgemm = {"tflops": round(2.0 * 128 * K * N / dt / 1e12, 5), "seconds": round(dt, 2),
                 "sample": "first 128 rows of the qkv GEMM (K4096 N12288), plain-C blocked OpenMP fp32 GEMM"}
        rows_f = 64
        o_np = np.zeros(rows_f * N, np.float16)
        t0 = time.perf_counter()
        oracle.matmul_f16(o_np, a_np[:rows_f], w_np, 1, rows_f, K, N, (1, N, 0), (1, K, 0), (K, 1, 0),
                          mode=oracle.FAITHFUL, threads=threads)
        dt = time.perf_counter() - t0
        faithful = {"tflops": round(2.0 * rows_f * K * N / dt / 1e12, 6), "seconds": round(dt, 2),
                    "sample": f"first {rows_f} rows of the qkv GEMM, reference-faithful scalar arithmetic "
                              "(soft fp16 products, fp32 sum), OpenMP over rows"}
        # parity spot check of that sample against a fresh device result
        mm(outs[name], acts[K], weights[name], M, K, N)
        torch.cuda.synchronize()
        got = outs[name][:rows_f].cpu().numpy().astype(np.float64)
        ref = o_np.reshape(rows_f, N).astype(np.float64)
        rms = np.sqrt(np.mean(ref ** 2))
        faithful["max_rel_err_gpu_vs_cpu"] = float(
            np.max(np.abs(got - ref) / np.maximum(np.abs(ref), rms)))
        # The reference's own GPU kernel on this device (its matmul.cu compiled as it lies into
        # oracle/_ref/matmul.co, launched with the grid its host code uses, kernels.rs:849-863), and
        # this build's module with the same symbols at that same grid: what a host that keeps
        # calling `matmul_f16_fast` gets.  A baseline beside the figures above, never timed inside
        # the step.
        reference_gpu = None
        try:
            from oracle import refgpu
            if refgpu.available():
                name, K, N = LAYER_SET[0]
                so, sl, sr = (1, N, 0), (1, K, 0), (K, 1, 0)
                reference_gpu = {"shape": f"qkv M{M} K{K} N{N}, NT weights, grid of kernels.rs:849-863"}
                for label, directory in (("reference_matmul_f16_fast", refgpu.REF_DIR),
                                         ("this_build_legacy_symbol_matmul_f16_fast", refgpu.LEGACY_DIR)):
                    if not os.path.exists(os.path.join(directory, "matmul.co")):
                        continue
                    rk = refgpu.RefKernels(directory)
                    call = lambda: rk.matmul_f16_fast(outs[name].data_ptr(), acts[K].data_ptr(),   # noqa: E731
                                                      weights[name].data_ptr(), 1, M, K, N, so, sl, sr)
                    t = timed(call, 5, 2)
                    reference_gpu[label] = {"ms": round(t * 1e3, 3),
                                            "tflops": round(2.0 * M * K * N / t / 1e12, 2)}
                reference_gpu["adr_matmul_f16_ms"] = round(t_qkv * 1e3, 4)
        except Exception as e:  # noqa: BLE001  (a baseline leg: report, never fail the benchmark)
            reference_gpu = {"error": repr(e)}
        cpu_baseline = {
            "reference_gpu_kernel_same_device": reference_gpu,
            "value": round(torch_value, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "threads": threads, "nproc": nproc,
            "sample": per_config["configs[4] llama7b_layer_set_fp16_M2048"]["sample"] +
                      "; torch-CPU fp32 matmul on fp16-rounded inputs",
            "per_config_torch_cpu_fp32": per_config,
            "blocked_openmp_sgemm": sgemm, "faithful_scalar_port": faithful,
        }

    line = {
        "metric": METRIC, "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "settle_ms": args.settle_ms,
        "settle_steps": settle_steps, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": "llama7b_layer_gemm_set_fp16_prefill_M2048 (configs[4] of the benchmark definition, "
                               "fp16 weights: qkv, o, gate, up, down)",
                   "gflop_per_step": round(step_flops / 1e9, 1),
                   "frac_mfma_peak": round(value / PEAK_F16_TFLOPS, 4)},
        "roofline": roofline, "roofline_u8_gemv": roofline_u8, "cpu_baseline": cpu_baseline,
        "secondary": secondary,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
