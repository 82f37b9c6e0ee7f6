/*
 * CPU oracle for the adrastea matmul hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is a plain-C restatement of the reference's
 * device algorithms, used as the checker by tests/, by the smoke test and by the
 * cpu_baseline leg of bench.py.  Nothing on the product path may link or call it.
 *
 * fp16 values travel as raw uint16_t bit patterns; all fp16 arithmetic is done by
 * an integer-only soft-float (round-to-nearest-even, subnormals kept), so results
 * do not depend on the host compiler's _Float16 support.
 *
 * Parity pins (tests/test_oracle_*.py):
 *   - fp16 conversions: exhaustive against numpy's float16 (all 65536 patterns
 *     widening; boundary + random patterns narrowing from f32 and f64).
 *   - dequantize: exhaustive 256 x 65536 (q, scale-bits) table against an
 *     independent float64 -> float16 computation.
 *   - matmul: integer-exact cases, identity/permutation operands, brute-force
 *     stride permutations against numpy einsum in float64, batch broadcast,
 *     closed-form epilogues, causal mask bit pattern.
 *   - quantize: constructed rows with closed-form answers + round-trip bound.
 * The reference holds no golden vectors for any of these functions (it has no
 * matmul / quantize test), so the pins above are mathematical, not fixtures.
 */
#ifndef ADR_ORACLE_H
#define ADR_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* enum values: adrastea_kernels/cpp/matmul.cu:26-36, adrastea_models/src/kernels.rs:81-135 */
enum { ADR_O_LOAD_IDENTITY = 0, ADR_O_LOAD_SCALE = 1 };
enum {
  ADR_O_STORE_IDENTITY = 0,
  ADR_O_STORE_GELU_BIAS = 1, /* no device case in the reference (matmul.cu:450-491) */
  ADR_O_STORE_BETA_GELU_BIAS = 2,
  ADR_O_STORE_BETA_BIAS = 3,
  ADR_O_STORE_SCALE = 4,
  ADR_O_STORE_ADD = 5,
  ADR_O_STORE_QUICK_GELU_BIAS = 6
};
enum { ADR_O_MASK_NONE = 0, ADR_O_MASK_CAUSAL = 1 };

/* accumulation modes of adr_o_matmul_f16 */
enum {
  ADR_O_FAITHFUL = 0, /* fp16-rounded products, sequential fp32 sum (matmul.cu:214-218) */
  ADR_O_EXACT = 1     /* exact products, float64 sum, one rounding to fp32 */
};

float adr_o_h2f(uint16_t h);
uint16_t adr_o_f2h(float f);
uint16_t adr_o_d2h(double d);
uint16_t adr_o_hmul(uint16_t a, uint16_t b);
uint16_t adr_o_hadd(uint16_t a, uint16_t b);

/* bulk converters used by the tests to pin the soft-float */
void adr_o_h2f_n(float* out, const uint16_t* in, int64_t n);
void adr_o_f2h_n(uint16_t* out, const float* in, int64_t n);
void adr_o_d2h_n(uint16_t* out, const double* in, int64_t n);

/* matmul.cu:186-222 (naive kernel) + :418-502 (enum dispatch).  Returns 0, or -1 for
 * an enum value the reference has no device case for. */
int adr_o_matmul_f16(uint16_t* output, const uint16_t* lhs, const uint16_t* rhs, int batches,
                     int m, int k, int n, int stride_ox, int stride_oy, int stride_oz,
                     int stride_lx, int stride_ly, int stride_lz, int stride_rx, int stride_ry,
                     int stride_rz, const uint16_t* bias, float beta, float scale,
                     uint32_t store, uint32_t load, uint32_t mask, int mode, int threads);

/* matmul_nt_wmma_16x128x256.cu:8-68 semantics: out = A[m,p] . B[n,p]^T + beta*out */
void adr_o_matmul_nt_f16(uint16_t* output, const uint16_t* lhs, const uint16_t* rhs, int m, int p,
                         int n, float beta, int threads);

/* matmul_nt_fp16u8.cu:4-24: the naive u8 kernel (double-precision product, fp32 sum). */
void adr_o_matmul_nt_fp16u8_naive(uint16_t* output, const uint16_t* lhs, const uint8_t* rhs,
                                  const uint16_t* scales, int m, int p, int n, int block_size,
                                  float beta, int threads);

/* matmul_nt_wmma_16x128x256_fp16u8.cu:5-7,43-83: dequantise to fp16 first, then an
 * fp16 x fp16 -> fp32 product sum (here: exact products, float64 sum). */
void adr_o_matmul_nt_fp16u8(uint16_t* output, const uint16_t* lhs, const uint8_t* rhs,
                            const uint16_t* scales, int m, int p, int n, int block_size,
                            float beta, int threads);

/* quantize.cu:46-56 */
void adr_o_dequantize_absmax_u8(uint16_t* output, const uint8_t* q, const uint16_t* scales,
                                int rows, int cols, int block_size);
/* quantize.cu:3-44 */
/* embed_uint8.cu:3-19: out[t, i] = dequant(table[ids[t], i], scales[ids[t], i / block_size]). */
void adr_o_embed_uint8(int n_dim, int n_ids, const int16_t* in_ids, uint16_t* out,
                       const uint8_t* table, const uint16_t* scales, int block_size);
void adr_o_quantize_absmax_u8(uint8_t* q, uint16_t* scales, const uint16_t* input, int rows,
                              int cols, int block_size);

/* normalize.cu:147-220 softmax_rows on a contiguous [rows, w] fp16 tensor (rows = heads * h).
 * mode 0: the reference's arithmetic and reduction order in fp32 (256 threads striding the row,
 * xor trees over 32-lane groups, then over the 8 group results); mode 1: float64 throughout,
 * one rounding to fp16 at the end. */
void adr_o_softmax_rows(uint16_t* output, const uint16_t* input, int64_t rows, int w, float temp,
                        int mode);

/* error_stats.cu:13-75 on flat arrays: out[0] = sum d^2 / length, out[1] = max |d|,
 * out[2] = sum |d| / length over the first 128 * (length / 128) elements (the reference's 128
 * blocks of length / 128), d = float(lhs) - float(rhs) in fp32; sums carried in float64 here.
 * is_f32 selects fp32 inputs (else fp16 bit patterns). */
void adr_o_error_stats(float* out, const void* lhs, const void* rhs, int64_t length, int is_f32);

/* Blocked OpenMP fp32 GEMM out[m,n] = a[m,k] . b[n,k]^T: the CPU-baseline counterpart of the
 * reference's host GEMM (matrixmultiply::sgemm, adrastea_core/src/mel.rs:142-157). */
void adr_o_sgemm_nt(float* out, const float* a, const float* b, int m, int k, int n, int threads);

/* exhaustive dequant table: out[q * 65536 + s] = dequant(q, scale bits s) */
void adr_o_dequant_table(uint16_t* out);

#ifdef __cplusplus
}
#endif
#endif
