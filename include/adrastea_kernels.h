/*
 * adrastea_kernels -- C ABI of the gfx950 (MI355X) matmul kernels.
 *
 * This is the boundary a Rust `extern "C"` block in adrastea_kernels binds.  Every entry
 * point takes plain pointers and scalars, launches asynchronously on the given HIP stream
 * (NULL = the null stream, which is what the reference uses: `stream: None`,
 * adrastea_models/src/kernels.rs:862), never synchronises, allocates nothing per call, and
 * returns 0 on success, a positive hipError_t, or a negative ADR_E* code.  Invalid requests are
 * rejected on the host; no entry point traps on the device.  The kernels exist for gfx950 only:
 * with any other device current, every launching entry point returns ADR_EUNSUPPORTED_DEVICE
 * (the device's architecture, compute-unit and die counts are queried once per device and
 * cached).  Beside that cache the library keeps one piece of state: the pool of workspaces that
 * adr_matmul_f16, adr_matmul_nt_f16 and (on request) adr_matmul_nt_fp16u8 draw from, grown on
 * demand and given back through adr_release_held_workspace* (adr_set_held_workspace_limit below;
 * 0 switches it off).
 *
 * fp16 data is passed as uint16_t bit patterns (Rust `half::f16` is repr(transparent) u16).
 * All strides are in ELEMENTS.  `x` is the last tensor dimension, `y` the second to last,
 * `z` the batch dimension (kernels.rs:864-887).
 */
#ifndef ADRASTEA_KERNELS_H
#define ADRASTEA_KERNELS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* A hipStream_t, declared opaquely so that this header needs no HIP include. */
typedef void* adr_stream_t;

/* Error codes (negative; positive values are hipError_t). */
enum {
  ADR_OK = 0,
  ADR_EINVAL_SHAPE = -1,   /* negative / zero-incompatible sizes, offsets beyond int32 */
  ADR_EINVAL_ENUM = -2,    /* store / load / mask value out of range */
  ADR_ENOTIMPL = -3,       /* MatmulStoreOp::GeluBias = 1: lowers from Rust
                              (kernels.rs:125) but has no device case in the reference
                              (matmul.cu:450-491 -> NYI trap); rejected here instead */
  ADR_ENULL = -4,          /* null tensor pointer, or a bias operator without a bias */
  ADR_EDIVISIBILITY = -5,  /* u8 kernels: p % block_size != 0 or block_size not supported */
  ADR_EUNSUPPORTED_DEVICE = -6, /* the current device is not gfx950 */
  ADR_EUNSUPPORTED_LAYOUT = -7, /* adr_attention_f16: head dimension, stride or alignment that the
                                   fused kernel does not cover; use the three-call sequence */
  ADR_ESCRATCH = -8             /* adr_matmul_f16_noalloc: the product needs more scratch than
                                   ADR_NOALLOC_SCRATCH_BYTES (kept for ABI stability: products are
                                   cut to fit instead) */
};

/* adrastea_models/src/kernels.rs:81-135, adrastea_kernels/cpp/matmul.cu:26-36 */
enum { ADR_LOAD_IDENTITY = 0, ADR_LOAD_SCALE = 1 };
enum {
  ADR_STORE_IDENTITY = 0,
  ADR_STORE_GELU_BIAS = 1,
  ADR_STORE_BETA_GELU_BIAS = 2,
  ADR_STORE_BETA_BIAS = 3,
  ADR_STORE_SCALE = 4,
  ADR_STORE_ADD = 5,
  ADR_STORE_QUICK_GELU_BIAS = 6
};
enum { ADR_MASK_NONE = 0, ADR_MASK_CAUSAL = 1 };

/*
 * Replaces the launch of `matmul_f16_fast` in GpuKernels::matmul_f16
 * (adrastea_models/src/kernels.rs:821-890; device adrastea_kernels/cpp/matmul.cu:504-513).
 * Same 22 arguments in the same order as the Rust tuple (kernels.rs:864-887), preceded by
 * the stream.  Launch geometry and LDS size are chosen inside.
 *
 *   O[b,y,x] = store( sum_k load(L[b,y,k]) * load(R[b,k,x]) ),  mask(x, y) -> -inf
 *
 * fp16 operands, fp32 accumulation, fp16 result.  The accumulator is narrowed to fp16
 * before the store operator, as in the reference (matmul.cu:47-52, 64-71).
 */
int adr_matmul_f16(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                   const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                   int32_t stride_ox, int32_t stride_oy, int32_t stride_oz, int32_t stride_lx,
                   int32_t stride_ly, int32_t stride_lz, int32_t stride_rx, int32_t stride_ry,
                   int32_t stride_rz, const uint16_t* bias, float beta, float scale,
                   uint32_t store, uint32_t load, uint32_t mask);

/*
 * Replaces the launch of the naive `matmul_f16` in GpuKernels::matmul_f16_slow
 * (kernels.rs:753-819; device matmul.cu:195-222, 493-502).  One thread per output element,
 * any strides; reproduces the reference arithmetic step for step (fp16-rounded products,
 * sequential fp32 sum).  It is the correctness path the fast kernels are compared with.
 */
int adr_matmul_f16_slow(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                        const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                        int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                        int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                        int32_t stride_rx, int32_t stride_ry, int32_t stride_rz,
                        const uint16_t* bias, float beta, float scale, uint32_t store,
                        uint32_t load, uint32_t mask);

/*
 * adr_matmul_f16 with a caller-provided scratch buffer (no counterpart in the reference, whose
 * kernel walks all of K in every workgroup: kernels.rs:849-863, matmul.cu:288-381).  Same
 * arguments, same result, same validation; in addition `workspace` (device memory, 16-byte
 * aligned) of `workspace_bytes` bytes.  A product with few output tiles and a long K -- a few
 * dozen to a few hundred rows against a weight matrix, what the reference's LLaMA issues for
 * every generated token since it keeps no KV cache (llama.rs:456-483) -- then runs as two
 * launches: K is split over several workgroups per tile that leave fp32 partial tiles in the
 * workspace, and a second kernel sums them in a fixed order and applies the store operator.
 * adr_matmul_f16_workspace_bytes tells how much such a product would use at best (0: it would
 * not be split); with less, K is cut into fewer pieces or not at all, and with
 * workspace_bytes == 0 the product runs unsplit.  Only the caller's buffer is used, never the
 * library's own (adr_set_held_workspace_limit below).
 * The workspace is written and read by the two launches only; it carries nothing from one call
 * to the next, so one buffer serves all calls on a stream.  Calls that may overlap (different
 * streams) need different buffers.
 */
int adr_matmul_f16_ws(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                      const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                      int32_t stride_ox, int32_t stride_oy, int32_t stride_oz, int32_t stride_lx,
                      int32_t stride_ly, int32_t stride_lz, int32_t stride_rx, int32_t stride_ry,
                      int32_t stride_rz, const uint16_t* bias, float beta, float scale,
                      uint32_t store, uint32_t load, uint32_t mask, void* workspace,
                      int64_t workspace_bytes);
/* Returns the bytes (>= 0) or a negative ADR_E* code; touches no device memory. */
int64_t adr_matmul_f16_workspace_bytes(int32_t batches, int32_t m, int32_t k, int32_t n,
                                       int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                                       int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                                       int32_t stride_rx, int32_t stride_ry, int32_t stride_rz,
                                       uint32_t store, uint32_t load, uint32_t mask);

/*
 * adr_matmul_f16_ws without the workspace argument (no counterpart in the reference).  For
 * callers that cannot allocate device memory around a call: code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  The scratch is a fixed array of
 * ADR_NOALLOC_SCRATCH_BYTES inside the library's device code, one copy per GPU the library runs
 * on, held until the process ends; the entry point allocates and frees nothing (its first call
 * on a device looks the array's address up once: make that call before a graph capture begins).  Same arguments, validation and result as
 * adr_matmul_f16_ws given a workspace of at least adr_matmul_f16_workspace_bytes bytes.
 * A product that would like more than ADR_NOALLOC_SCRATCH_BYTES (16 MiB: the LLaMA-7B down
 * projection up to 256 rows fits) is cut into as many pieces as fit, or runs unsplit: the result
 * is then that of adr_matmul_f16_ws given a workspace of exactly ADR_NOALLOC_SCRATCH_BYTES.
 * All calls on one GPU share that GPU's array: calls that may overlap in time (different streams)
 * race on it and must be serialised by the caller or use adr_matmul_f16_ws with buffers of their
 * own.  Nothing in the array has to start at zero and nothing is kept from one call to the next
 * (every partial tile is written before the reduction reads it).
 */
#define ADR_NOALLOC_SCRATCH_BYTES (16 * 1024 * 1024)
int adr_matmul_f16_noalloc(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                           const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                           int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                           int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                           int32_t stride_rx, int32_t stride_ry, int32_t stride_rz,
                           const uint16_t* bias, float beta, float scale, uint32_t store,
                           uint32_t load, uint32_t mask);

/*
 * The workspaces that adr_matmul_f16 and adr_matmul_nt_f16 hold themselves (no counterpart in the
 * reference).  Those entry points keep the reference's argument tuples and so have no workspace
 * argument; where a workspace pays -- the products adr_matmul_f16_ws splits along K -- they take
 * one from a pool inside the library.  A buffer belongs to a (device, stream) pair: it is allocated
 * with hipMalloc at the first call on that stream that wants one (16 MiB doubling up to the limit)
 * and carries an event recorded behind the last launches that used it.  When a stream wants more
 * than its buffer holds it gets a larger one and the old buffer stays in the pool for any stream
 * that wants less; when all 16 entries of the pool are taken, a stream without a buffer takes over
 * the least recently used one that is large enough.  A buffer changes hands by making the new
 * owner's stream wait for the buffer's event (hipStreamWaitEvent): nothing is freed, allocated or
 * synchronised inside a matmul call beyond those first allocations, and the pool never holds more
 * than 16 buffers of at most the limit each.  Calls on one stream share a buffer and run in stream
 * order; the pool is locked while a call that uses it launches, so any thread may call on any
 * stream.  No buffer is used or allocated -- the call runs exactly as with a limit of 0 -- while
 * the stream is being captured into a graph (the launches would tie the buffer to a graph that may
 * be replayed on another stream), on hipStreamPerThread, when the allocation fails, or when the
 * pool is full and holds no buffer large enough; a product that wants more than the limit is split
 * into fewer pieces instead.  adr_held_workspace_declined counts the calls that wanted a buffer and
 * ran without one.
 * Results: the split products sum K in pieces, so on inexact data the last bits may differ from
 * the unsplit launch (both within the stated tolerance).
 *
 * adr_set_held_workspace_limit: bytes per buffer (default ADR_HELD_WORKSPACE_DEFAULT_BYTES =
 * 128 MiB); 0 switches the pool off for later calls (buffers already allocated stay until
 * released).  adr_held_workspace_bytes: bytes the pool holds now.
 * adr_release_held_workspace(stream): waits for the last launches that used them (the buffers'
 * events, not the device) and frees, on the current device, the buffers `stream` owns and those no
 * stream owns any more; call it before destroying a stream.  adr_release_held_workspace_all: the
 * same for every buffer on every device.  (hipFree itself may wait for other work on the device:
 * these two are not for the hot path.)  Later calls allocate afresh.
 * Callers that must not allocate at all use adr_matmul_f16_noalloc or the _ws forms, which never
 * touch the pool.
 *
 * adr_set_u8_dequantise_first(1): lets adr_matmul_nt_fp16u8 take the route of
 * adr_matmul_nt_fp16u8_ws by itself, with the dequantised matrix (n * p * 2 bytes, which must fit
 * the limit above: the LLaMA-7B qkv matrix is 100.7 MB) in a buffer of this pool.  Off by default:
 * the plain entry point then always runs its fused kernels, eagerly and under capture alike.
 */
#define ADR_HELD_WORKSPACE_DEFAULT_BYTES ((int64_t)128 * 1024 * 1024)
int adr_set_held_workspace_limit(int64_t bytes);
int64_t adr_held_workspace_limit(void);
int64_t adr_held_workspace_bytes(void);
int64_t adr_held_workspace_declined(void);
int adr_release_held_workspace(adr_stream_t stream);
int adr_release_held_workspace_all(void);
int adr_set_u8_dequantise_first(int enabled);
int adr_u8_dequantise_first(void);

/* `matmul_f16_raw` (matmul.cu:515-517): identity operators, the 16 common arguments. */
int adr_matmul_f16_raw(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                       const uint16_t* rhs, int32_t batches, int32_t m, int32_t k, int32_t n,
                       int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                       int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                       int32_t stride_rx, int32_t stride_ry, int32_t stride_rz);

/*
 * fp16 NT GEMM, contiguous operands: out[m,n] = lhs[m,p] . rhs[n,p]^T + beta * out[m,n].
 * Argument list of `matmul_nt_wmma_16x128x256` / `matmul_nt_wmma_128x64x64`
 * (adrastea_kernels/cpp/matmul_nt_wmma_16x128x256.cu:8-14); their m%16 / n%128 / p%256
 * divisibility requirements do not apply here.
 */
int adr_matmul_nt_f16(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                      const uint16_t* rhs, int32_t m, int32_t p, int32_t n, float beta);

/*
 * u8-quantised-weight NT GEMM / GEMV with the dequantisation fused into the weight load.
 * Argument list of `matmul_nt_fp16u8` and `matmul_nt_wmma_16x128x256_fp16u8`
 * (adrastea_kernels/cpp/matmul_nt_fp16u8.cu:4-12, matmul_nt_wmma_16x128x256_fp16u8.cu:12-20):
 *
 *   w[c,i]   = fp16( (float(rhs[c,i]) - 127.5f) * float(scales[c, i / block_size]) )
 *   out[r,c] = fp16( sum_i lhs[r,i] * w[c,i]  +  beta * out[r,c] )      (fp32 accumulation)
 *
 * lhs [m,p] fp16, rhs [n,p] u8, scales [n, p/block_size] fp16, out [m,n] fp16, all contiguous.
 * Any m >= 1 and n >= 1; p % block_size == 0; block_size a multiple of 8.
 * Always the fused kernels (weights dequantised between the load and the matrix cores, nothing
 * written back), eagerly and under graph capture alike, unless adr_set_u8_dequantise_first(1).
 */
int adr_matmul_nt_fp16u8(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                         const uint8_t* rhs, const uint16_t* scales, int32_t m, int32_t p,
                         int32_t n, int32_t block_size, float beta);

/*
 * adr_matmul_nt_fp16u8 with a caller-provided workspace (no counterpart in the reference).  From
 * 96 activation rows on (160 against fewer than 8192 weight rows), dequantising the weight
 * matrix once into `workspace` (n * p fp16 values, bit-identical to dequantize_absmax_uint8) and
 * running the fp16 kernels on it is faster than dequantising every weight once per 256-row tile
 * inside the GEMM: M2048 K4096 N12288 232 -> 211 us, M512 K11008 N4096 140 -> 88 us.  Both paths
 * round every weight to fp16 as dequantize_absmax_uint8 does; from 257 rows on (and below
 * wherever adr_matmul_nt_fp16u8_plan names a gemm_nt_u8_ kernel) they also sum in the same order
 * and the result has the same bits.  Fewer rows, or a few hundred to 1535 rows against a wide
 * matrix (where one round of the fused kernel's tiles covers the product and it is ahead), or a
 * workspace smaller than adr_matmul_nt_fp16u8_workspace_bytes reports: exactly
 * adr_matmul_nt_fp16u8.  The workspace (16-byte aligned, device memory) is written by the call
 * and holds nothing afterwards; calls sharing one must not overlap in time.
 */
int adr_matmul_nt_fp16u8_ws(adr_stream_t stream, uint16_t* output, const uint16_t* lhs,
                            const uint8_t* rhs, const uint16_t* scales, int32_t m, int32_t p,
                            int32_t n, int32_t block_size, float beta, void* workspace,
                            int64_t workspace_bytes);
/* Bytes (>= 0; 0: the workspace would not be used) or a negative ADR_E* code. */
int64_t adr_matmul_nt_fp16u8_workspace_bytes(int32_t m, int32_t p, int32_t n, int32_t block_size);

/*
 * Flat-pointer forms of `dequantize_absmax_uint8` / `quantize_absmax_uint8`
 * (adrastea_kernels/cpp/quantize.cu:46-56 and :3-44) for contiguous [rows, cols] tensors with
 * scales [rows, cols / block_size]:
 *   dequantise: out = fp16((float(q) - 127.5f) * float(scale))
 *   quantise:   scale = fp16(absmax / 127.5f); q = u8(round(127.5f + x / float(scale)))
 */
int adr_dequantize_absmax_u8(adr_stream_t stream, uint16_t* output, const uint8_t* q,
                             const uint16_t* scales, int32_t rows, int32_t cols,
                             int32_t block_size);
int adr_quantize_absmax_u8(adr_stream_t stream, uint8_t* q, uint16_t* scales,
                           const uint16_t* input, int32_t rows, int32_t cols,
                           int32_t block_size);

/*
 * The by-value tensor descriptor the reference passes to its quantise kernels
 * (TensorGpuDescriptor, adrastea_models/src/kernels.rs:28-61; device TensorView<T>,
 * adrastea_kernels/cpp/compat.h:40-45).  Index 0 is the INNERMOST dimension.
 */
typedef struct adr_tensor_desc {
  void* ptr;
  uint32_t dims;
  uint32_t shape[7];
  uint32_t strides[7];
} adr_tensor_desc;

/* Descriptor forms with the reference's argument order (quantize.cu:3-5, 46-48).  2-d
 * tensors, any strides; block_size = output.shape[0] / scales.shape[0]. */
int adr_dequantize_absmax_uint8(adr_stream_t stream, adr_tensor_desc output,
                                adr_tensor_desc scales, adr_tensor_desc input);
int adr_quantize_absmax_uint8(adr_stream_t stream, adr_tensor_desc output,
                              adr_tensor_desc scales, adr_tensor_desc input);

/*
 * Embedding lookup in a u8-quantised table (device: adrastea_kernels/cpp/embed_uint8.cu:3-19
 * `embed_uint8(n_dim, n_ids, in_ids, out_embeddings, embeddings_table, scales, block_size)`; the
 * reference compiles it but has no host call yet, so the device signature is the interface):
 *   out[t, i] = fp16( (float(table[id_t, i]) - 127.5f) * float(scales[id_t, i / block_size]) ),
 * id_t = in_ids[t], 16-bit ids as in the reference; `table` is [vocab, n_dim] u8 and `scales`
 * [vocab, n_dim / block_size] fp16, the format of adr_quantize_absmax_u8.  Ids are not range
 * checked (the kernel has no vocabulary size, as in the reference).
 */
int adr_embed_uint8(adr_stream_t stream, int32_t n_dim, int32_t n_ids, const int16_t* in_ids,
                    uint16_t* out_embeddings, const uint8_t* embeddings_table,
                    const uint16_t* scales, int32_t block_size);

/*
 * Row-wise softmax with temperature, the step between QK^T and P.V
 * (device: adrastea_kernels/cpp/normalize.cu:147-220 `softmax_rows(output, input, h, w, temp)` on
 * a (heads, h) grid; host: CommonKernels::softmax_rows_inplace, adrastea_models/src/kernels.rs:214,
 * 892-915, which passes output twice).  `input` and `output` are contiguous [heads, h, w] fp16
 * tensors and may be the same buffer:
 *   out[i] = fp16( expf(in[i]/temp - max) / sum_j expf(in[j]/temp - max) )   over each row of w.
 * The reference's third and fourth arguments (h, w) are kept; `heads` replaces its grid.y.
 */
int adr_softmax_rows(adr_stream_t stream, uint16_t* output, const uint16_t* input, int32_t heads,
                     int32_t h, int32_t w, float temp);

/*
 * Error statistics of two tensors, the reference's on-device parity check
 * (device: adrastea_kernels/cpp/error_stats.cu:13-75 `error_stats_f16/_f32(output, lhs, rhs)` with
 * by-value descriptors; host: CommonKernels::error_stats_f16/_f32, adrastea_models/src/kernels.rs:
 * 223-228, 717-751, which flatten both operands with shape_cast(&[-1])).  1-d descriptors; `output`
 * is an fp32 vector of at least 3 values that the CALLER zeroes:
 *   output[0] += mean squared error, output[1] = max(output[1], max abs error),
 *   output[2] += mean absolute error,
 * over the first 128 * floor(length / 128) elements with the means divided by `length`, exactly as
 * the reference's 128-block walk does (its last length % 128 elements are not visited).
 */
int adr_error_stats_f16(adr_stream_t stream, adr_tensor_desc output, adr_tensor_desc lhs,
                        adr_tensor_desc rhs);
int adr_error_stats_f32(adr_stream_t stream, adr_tensor_desc output, adr_tensor_desc lhs,
                        adr_tensor_desc rhs);

/*
 * Fused attention of one layer (no single counterpart in the reference: it stands for the three
 * calls at adrastea_models/src/llama.rs:541-554 -- matmul_f16 with MatmulStore::Scale and
 * MatmulMask::Causal into a [heads, m, n] tensor, softmax_rows_inplace, matmul_f16 with the value
 * view -- and their twins at clip.rs:372-388 and whisper.rs:424-436):
 *   out[h, y, :] = sum_x softmax_x( mask(scale * <query[h, y, :], key[h, x, :]>) / temp ) * value[h, x, :]
 * `query` and `output` are [heads, m, d] views, `key` and `value` [heads, n, d] views (key NOT
 * transposed: llama.rs:537's k_view is this view with its last two axes swapped); strides are in
 * elements with x = dim -1, y = dim -2, z = dim -3, as in adr_matmul_f16.  mask = ADR_MASK_CAUSAL
 * removes x > y exactly as matmul.cu:182-184 does.  The scores never reach memory and stay in
 * fp32, so results equal the three-call sequence up to the fp16 rounding that sequence applies to
 * scores and probabilities in between.
 * Covered: d = 64 or 128, every x stride 1, y and z strides multiples of 8, 16-byte aligned
 * pointers, scale > 0, temp > 0; anything else returns ADR_EUNSUPPORTED_LAYOUT and launches
 * nothing.  n = 0 with m > 0 is ADR_EINVAL_SHAPE (a softmax over no elements).
 */
int adr_attention_f16(adr_stream_t stream, uint16_t* output, const uint16_t* query,
                      const uint16_t* key, const uint16_t* value, int32_t heads, int32_t m,
                      int32_t n, int32_t d, int32_t stride_ox, int32_t stride_oy,
                      int32_t stride_oz, int32_t stride_qx, int32_t stride_qy, int32_t stride_qz,
                      int32_t stride_kx, int32_t stride_ky, int32_t stride_kz, int32_t stride_vx,
                      int32_t stride_vy, int32_t stride_vz, float scale, float temp,
                      uint32_t mask);

/*
 * Diagnostics (no counterpart in the reference).
 *
 * adr_matmul_f16_plan: writes the name of the kernel adr_matmul_f16 would launch for these
 * arguments -- on a stream that is not being captured and with the held-workspace limit as it is
 * now ("..._splitk4": K in four pieces through a held buffer; with a limit of 0, or under
 * capture, the unsplit kernel that adr_matmul_f16_ws_plan names for a workspace of 0 bytes) --
 * into `name` (at most `cap` bytes, NUL-terminated) without touching the device.
 * Same validation and return codes as adr_matmul_f16 minus the pointer checks.  Without pointers
 * the plan assumes 16-byte aligned operands; a call with unaligned ones runs on the general
 * (u8: the per-output) kernel whatever the plan says.  On a machine without a device the plan
 * is the one for an MI355X.  adr_matmul_nt_fp16u8_plan names the tile of a tiled kernel
 * ("gemm_nt_u8_mfma_256x192x64", "gemm_nt_u8_stage_128x128x32", ...), or
 * "dequantize_absmax_u8 + fp16 gemm" where adr_set_u8_dequantise_first(1) routes the product.
 */
int adr_matmul_f16_plan(char* name, int32_t cap, int32_t batches, int32_t m, int32_t k,
                        int32_t n, int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                        int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                        int32_t stride_rx, int32_t stride_ry, int32_t stride_rz, uint32_t store,
                        uint32_t load, uint32_t mask);
int adr_matmul_nt_fp16u8_plan(char* name, int32_t cap, int32_t m, int32_t p, int32_t n,
                              int32_t block_size);
/* The plan of adr_matmul_f16_ws for a workspace of the given size ("..._splitk4": K in four pieces). */
int adr_matmul_f16_ws_plan(char* name, int32_t cap, int32_t batches, int32_t m, int32_t k,
                           int32_t n, int32_t stride_ox, int32_t stride_oy, int32_t stride_oz,
                           int32_t stride_lx, int32_t stride_ly, int32_t stride_lz,
                           int32_t stride_rx, int32_t stride_ry, int32_t stride_rz, uint32_t store,
                           uint32_t load, uint32_t mask, int64_t workspace_bytes);

/*
 * For tests and benchmarks only (no counterpart in the reference): forces a kernel choice that
 * the dispatch otherwise makes from the arguments, process-wide, so that the chosen kernel can be
 * compared with the others on the same operands.  id 0: the tile of the fp16 tiled GEMM (value 0:
 * the dispatch decides; 1 + i: tile i of 256x192, 256x128, 128x256, 128x192, 128x128, 128x64, 64x64,
 * 256x160 where the product is one the tiled kernels cover).  id 1: the tile of the u8-weight tiled
 * GEMM (0: the dispatch decides; 1 + i: tile i of 256x192, 256x128, 128x128, 128x64, 64x64, 128x64
 * with K split over two groups of wavefronts, 64x64 with K split over four; 8: the register-staged
 * kernels that otherwise serve a K that is no multiple of 64; 9: the passes of 64 rows for products
 * of 17 to 256 rows); a forced tile also keeps products of 17 to 256 rows off those passes.  Unknown
 * ids return ADR_EINVAL_ENUM.
 */
int adr_debug_knob(int32_t id, int32_t value);

/*
 * Microbenchmark aids (the device kernels of adrastea_kernels/cpp/microbench.cu:28-51 -- empty_kernel,
 * wmma_loop_f32_f16 -- as adrastea/src/main.rs:486-553 drives them, plus a streaming read): the
 * measured peaks that the fractions of the 2516.6 TFLOP/s and 8 TB/s figures are put beside.
 *   adr_microbench_empty     one empty launch (launch overhead)
 *   adr_microbench_mfma_f16  `blocks` workgroups of four wavefronts, each issuing times x 4
 *                            v_mfma_f32_32x32x16_f16 on register operands: 2*32*32*16 flop each,
 *                            i.e. blocks * 4 * times * 4 * 32768 flop per launch.  pattern 0:
 *                            zero operands, 1: pseudo-random fp16 operands, 2: pseudo-random
 *                            operands that change with every instruction as in a product's
 *                            inner loop (2 x 2 sub-tiles, fragments rotated in registers).
 *                            Patterns 3 and 4 compare the two MFMA shapes on a wavefront's
 *                            128 x 128 tile, random operands alternating between two register
 *                            sets per k-step: 3: times x 32 v_mfma_f32_32x32x16_f16 (2^20 flop
 *                            per wavefront and unit of `times`), 4: times x 128
 *                            v_mfma_f32_16x16x32_f16 (2^21 flop).
 *                            `sink` receives blocks * 256 floats.
 *   adr_microbench_stream_read  reads `bytes` (a multiple of 16 * blocks) from `src` with
 *                            `blocks` workgroups, one contiguous piece each; `sink`: 4 bytes.
 */
int adr_microbench_empty(adr_stream_t stream);
int adr_microbench_mfma_f16(adr_stream_t stream, int blocks, int times, int pattern, float* sink);
int adr_microbench_stream_read(adr_stream_t stream, const void* src, int64_t bytes, int blocks,
                               uint32_t* sink);

/* Human-readable text for an ADR_E* code or hipError_t. */
const char* adr_strerror(int code);
/* ABI version of this library (bumped on any signature change). */
int adr_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* ADRASTEA_KERNELS_H */
