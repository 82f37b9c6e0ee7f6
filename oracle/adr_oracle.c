/*
 * CPU oracle for the adrastea matmul hot path -- TEST INFRASTRUCTURE ONLY.
 * See adr_oracle.h for what it is allowed to be used for and how it is pinned.
 *
 * Build: gcc -O2 -ffp-contract=off -fopenmp -shared -fPIC (oracle/Makefile).
 * -ffp-contract=off matters: the faithful mode must perform every fp32 add and
 * multiply as its own correctly-rounded operation.
 */
#include "adr_oracle.h"

#include <math.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------ soft fp16 */

static inline uint32_t f32_bits(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
}
static inline float bits_f32(uint32_t u) {
  float f;
  memcpy(&f, &u, 4);
  return f;
}
static inline uint64_t f64_bits(double d) {
  uint64_t u;
  memcpy(&u, &d, 8);
  return u;
}

/* fp16 -> fp32, exact (every fp16 value is an fp32 value). */
float adr_o_h2f(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  if (exp == 0) {
    if (man == 0) return bits_f32(sign);
    /* subnormal: value = man * 2^-24; normalise */
    int e = 0;
    while (!(man & 0x400u)) {
      man <<= 1;
      e++;
    }
    man &= 0x3ffu;
    return bits_f32(sign | ((uint32_t)(113 - e) << 23) | (man << 13));
  }
  if (exp == 31) return bits_f32(sign | 0x7f800000u | (man << 13));
  return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
}

/* fp64 -> fp16 with a single round-to-nearest-even, integer arithmetic only. */
uint16_t adr_o_d2h(double d) {
  uint64_t u = f64_bits(d);
  uint16_t sign = (uint16_t)((u >> 48) & 0x8000u);
  int e = (int)((u >> 52) & 0x7ff);
  uint64_t m = u & ((1ull << 52) - 1);
  if (e == 0x7ff) {
    if (m) return (uint16_t)(sign | 0x7e00u | (uint16_t)(m >> 42));
    return (uint16_t)(sign | 0x7c00u);
  }
  if (e == 0) return sign; /* fp64 zero / subnormal: far below half of the smallest fp16 */
  int E = e - 1023;        /* value = 1.m * 2^E */
  if (E > 15) return (uint16_t)(sign | 0x7c00u);
  m |= 1ull << 52; /* 53-bit significand, value = m * 2^(E-52) */
  int shift;
  uint32_t base;
  if (E >= -14) {
    shift = 42; /* keep 11 significant bits */
    base = (uint32_t)(E + 15) << 10;
  } else {
    shift = 28 - E; /* result in units of 2^-24 */
    base = 0;
  }
  if (shift >= 64) return sign;
  uint64_t r = m >> shift;
  uint64_t rem = m & ((1ull << shift) - 1);
  uint64_t half = 1ull << (shift - 1);
  if (rem > half || (rem == half && (r & 1))) r++;
  uint32_t out;
  if (E >= -14) {
    out = base + (uint32_t)r - 0x400u; /* a mantissa carry bumps the exponent by itself */
  } else {
    out = (uint32_t)r; /* r == 0x400 is the smallest normal, encoded naturally */
  }
  if (out >= 0x7c00u) out = 0x7c00u;
  return (uint16_t)(sign | out);
}

/* fp32 -> fp16: the widening to fp64 is exact, so this is still one rounding. */
uint16_t adr_o_f2h(float f) { return adr_o_d2h((double)f); }

/* fp16 * fp16 -> fp16: the fp64 product of two 11-bit significands is exact. */
uint16_t adr_o_hmul(uint16_t a, uint16_t b) {
  return adr_o_d2h((double)adr_o_h2f(a) * (double)adr_o_h2f(b));
}

/* fp16 + fp16 -> fp16: fp16 values span 2^-24 .. 2^16, so the fp64 sum is exact. */
uint16_t adr_o_hadd(uint16_t a, uint16_t b) {
  return adr_o_d2h((double)adr_o_h2f(a) + (double)adr_o_h2f(b));
}

void adr_o_h2f_n(float* out, const uint16_t* in, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = adr_o_h2f(in[i]);
}
void adr_o_f2h_n(uint16_t* out, const float* in, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = adr_o_f2h(in[i]);
}
void adr_o_d2h_n(uint16_t* out, const double* in, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = adr_o_d2h(in[i]);
}

/* ------------------------------------------------------------------ epilogue */

/* Store operators of matmul.cu:418-491.  `sum` is the fp32 accumulator; every
 * operator first narrows it to fp16 (the operators take a __half argument,
 * matmul.cu:47-52, 64-71, 80-87), `o` is the previous content of the output element. */
static inline uint16_t store_op(float sum, uint16_t o, uint16_t bias, float beta, uint16_t hscale,
                                uint32_t store) {
  uint16_t s16 = adr_o_f2h(sum);
  switch (store) {
    case ADR_O_STORE_IDENTITY:
      return s16;
    case ADR_O_STORE_SCALE: /* half * half, matmul.cu:64-71 */
      return adr_o_hmul(s16, hscale);
    case ADR_O_STORE_ADD: /* half + half, matmul.cu:163-176 */
      return adr_o_hadd(s16, o);
    case ADR_O_STORE_BETA_BIAS: { /* matmul.cu:92-107, 146-161, 472-478 */
      float v = adr_o_h2f(s16) + adr_o_h2f(bias);
      float bo = beta * adr_o_h2f(o);
      return adr_o_f2h(v + bo);
    }
    case ADR_O_STORE_QUICK_GELU_BIAS: { /* matmul.cu:122-144, 465-471 */
      float v = adr_o_h2f(s16) + adr_o_h2f(bias);
      float t = 1.702f * v;
      float sg = 1.0f / (1.0f + expf(-t));
      return adr_o_f2h(v * sg);
    }
    case ADR_O_STORE_BETA_GELU_BIAS: { /* matmul.cu:109-124, 457-464 */
      float v = adr_o_h2f(s16) + adr_o_h2f(bias);
      float v3 = 0.044715f * v * v * v;
      float th = tanhf(0.7978845608028654f * (v + v3));
      float g = 0.5f * v * (1.0f + th);
      float bo = beta * adr_o_h2f(o);
      return adr_o_f2h(g + bo);
    }
    default:
      return 0;
  }
}

int adr_o_matmul_f16(uint16_t* output, const uint16_t* lhs, const uint16_t* rhs, int batches,
                     int m, int k, int n, int stride_ox, int stride_oy, int stride_oz,
                     int stride_lx, int stride_ly, int stride_lz, int stride_rx, int stride_ry,
                     int stride_rz, const uint16_t* bias, float beta, float scale,
                     uint32_t store, uint32_t load, uint32_t mask, int mode, int threads) {
  if (store == ADR_O_STORE_GELU_BIAS || store > ADR_O_STORE_QUICK_GELU_BIAS) return -1;
  if (load > ADR_O_LOAD_SCALE || mask > ADR_O_MASK_CAUSAL) return -1;
  const int needs_bias = store == ADR_O_STORE_BETA_GELU_BIAS || store == ADR_O_STORE_BETA_BIAS ||
                         store == ADR_O_STORE_QUICK_GELU_BIAS;
  if (needs_bias && !bias) return -1;
  /* the scale argument is narrowed to fp16 where it is used (Scale<T> holds a T,
   * matmul.cu:57-75, 439-443, 479-483); one value serves load and store. */
  const uint16_t hscale = adr_o_f2h(scale);
  if (threads < 1) threads = 1;
  const int64_t rows = (int64_t)batches * m;
#pragma omp parallel for schedule(static) num_threads(threads)
  for (int64_t row = 0; row < rows; row++) {
    int b = (int)(row / m), y = (int)(row % m);
    uint16_t* o = output + (int64_t)b * stride_oz;
    const uint16_t* l = lhs + (int64_t)b * stride_lz;
    const uint16_t* r = rhs + (int64_t)b * stride_rz;
    for (int x = 0; x < n; x++) {
      int64_t oi = (int64_t)y * stride_oy + (int64_t)x * stride_ox;
      if (mask == ADR_O_MASK_CAUSAL && x > y) { /* matmul.cu:182-184, 210-213 */
        o[oi] = 0xfc00u;
        continue;
      }
      float sum;
      if (mode == ADR_O_FAITHFUL) {
        sum = 0.0f;
        for (int i = 0; i < k; i++) {
          uint16_t a = l[(int64_t)y * stride_ly + (int64_t)i * stride_lx];
          uint16_t w = r[(int64_t)i * stride_ry + (int64_t)x * stride_rx];
          if (load == ADR_O_LOAD_SCALE) {
            a = adr_o_hmul(a, hscale);
            w = adr_o_hmul(w, hscale);
          }
          sum += adr_o_h2f(adr_o_hmul(a, w)); /* half product, fp32 sum: matmul.cu:216-217 */
        }
      } else {
        double acc = 0.0;
        for (int i = 0; i < k; i++) {
          uint16_t a = l[(int64_t)y * stride_ly + (int64_t)i * stride_lx];
          uint16_t w = r[(int64_t)i * stride_ry + (int64_t)x * stride_rx];
          if (load == ADR_O_LOAD_SCALE) {
            a = adr_o_hmul(a, hscale);
            w = adr_o_hmul(w, hscale);
          }
          acc += (double)adr_o_h2f(a) * (double)adr_o_h2f(w);
        }
        sum = (float)acc;
      }
      uint16_t bv = needs_bias ? bias[x] : 0;
      o[oi] = store_op(sum, o[oi], bv, beta, hscale, store);
    }
  }
  return 0;
}

void adr_o_matmul_nt_f16(uint16_t* output, const uint16_t* lhs, const uint16_t* rhs, int m, int p,
                         int n, float beta, int threads) {
  if (threads < 1) threads = 1;
#pragma omp parallel for schedule(static) num_threads(threads)
  for (int r = 0; r < m; r++) {
    for (int c = 0; c < n; c++) {
      double acc = 0.0;
      for (int i = 0; i < p; i++)
        acc += (double)adr_o_h2f(lhs[(int64_t)r * p + i]) * (double)adr_o_h2f(rhs[(int64_t)c * p + i]);
      int64_t oi = (int64_t)r * n + c;
      float bo = beta * adr_o_h2f(output[oi]);
      output[oi] = adr_o_f2h((float)acc + bo);
    }
  }
}

static inline uint16_t dequant_one(uint8_t q, uint16_t s) {
  /* quantize.cu:53-54 / matmul_nt_wmma_16x128x256_fp16u8.cu:5-7:
   * __float2half((float(q) - 127.5f) * __half2float(s)); the fp32 product is exact
   * (9 x 11 significant bits), so this is one rounding of the true product. */
  float v = ((float)q - 127.5f) * adr_o_h2f(s);
  return adr_o_f2h(v);
}

void adr_o_matmul_nt_fp16u8_naive(uint16_t* output, const uint16_t* lhs, const uint8_t* rhs,
                                  const uint16_t* scales, int m, int p, int n, int block_size,
                                  float beta, int threads) {
  if (threads < 1) threads = 1;
  int block_count = p / block_size;
#pragma omp parallel for schedule(static) num_threads(threads)
  for (int r = 0; r < m; r++) {
    for (int c = 0; c < n; c++) {
      float sum = 0.0f;
      for (int i = 0; i < p; i++) {
        /* 127.5 is a double literal in the reference (matmul_nt_fp16u8.cu:19): the
         * product is formed in double and the += narrows it back to float. */
        double prod = (double)adr_o_h2f(lhs[(int64_t)r * p + i]) *
                      ((double)(float)rhs[(int64_t)c * p + i] - 127.5) *
                      (double)adr_o_h2f(scales[(int64_t)c * block_count + i / block_size]);
        sum = (float)((double)sum + prod);
      }
      int64_t oi = (int64_t)r * n + c;
      float bo = beta * adr_o_h2f(output[oi]);
      output[oi] = adr_o_f2h(sum + bo);
    }
  }
}

void adr_o_matmul_nt_fp16u8(uint16_t* output, const uint16_t* lhs, const uint8_t* rhs,
                            const uint16_t* scales, int m, int p, int n, int block_size,
                            float beta, int threads) {
  if (threads < 1) threads = 1;
  int block_count = p / block_size;
#pragma omp parallel for schedule(static) num_threads(threads)
  for (int c = 0; c < n; c++) {
    for (int r = 0; r < m; r++) {
      double acc = 0.0;
      for (int i = 0; i < p; i++) {
        uint16_t w =
            dequant_one(rhs[(int64_t)c * p + i], scales[(int64_t)c * block_count + i / block_size]);
        acc += (double)adr_o_h2f(lhs[(int64_t)r * p + i]) * (double)adr_o_h2f(w);
      }
      int64_t oi = (int64_t)r * n + c;
      float bo = beta * adr_o_h2f(output[oi]);
      output[oi] = adr_o_f2h((float)acc + bo);
    }
  }
}

void adr_o_dequantize_absmax_u8(uint16_t* output, const uint8_t* q, const uint16_t* scales,
                                int rows, int cols, int block_size) {
  int block_count = cols / block_size;
  for (int r = 0; r < rows; r++)
    for (int i = 0; i < cols; i++)
      output[(int64_t)r * cols + i] =
          dequant_one(q[(int64_t)r * cols + i], scales[(int64_t)r * block_count + i / block_size]);
}

void adr_o_embed_uint8(int n_dim, int n_ids, const int16_t* in_ids, uint16_t* out,
                       const uint8_t* table, const uint16_t* scales, int block_size) {
  int block_count = n_dim / block_size; /* embed_uint8.cu:11 */
  for (int t = 0; t < n_ids; t++) {
    int id = in_ids[t]; /* :13 */
    for (int i = 0; i < n_dim; i++) /* :14-17 */
      out[(int64_t)t * n_dim + i] =
          dequant_one(table[(int64_t)id * n_dim + i], scales[(int64_t)id * block_count + i / block_size]);
  }
}

void adr_o_quantize_absmax_u8(uint8_t* q, uint16_t* scales, const uint16_t* input, int rows,
                              int cols, int block_size) {
  int block_count = cols / block_size;
  for (int r = 0; r < rows; r++) {
    for (int blk = 0; blk < block_count; blk++) {
      const uint16_t* x = input + (int64_t)r * cols + (int64_t)blk * block_size;
      float absmax = 0.0f;
      for (int i = 0; i < block_size; i++) absmax = fmaxf(absmax, fabsf(adr_o_h2f(x[i])));
      uint16_t hs = adr_o_f2h(absmax / 127.5f); /* quantize.cu:33 */
      scales[(int64_t)r * block_count + blk] = hs;
      float fs = adr_o_h2f(hs);
      for (int i = 0; i < block_size; i++) {
        /* quantize.cu:41-42: round half away from zero, then a float -> uint8 cast.
         * The cast is undefined for NaN / out-of-range (scale 0 or inf); here: NaN -> 0,
         * otherwise clamped.  Callers must not rely on that corner. */
        float v = roundf(127.5f + adr_o_h2f(x[i]) / fs);
        uint8_t out;
        if (!(v == v))
          out = 0;
        else if (v <= 0.0f)
          out = 0;
        else if (v >= 255.0f)
          out = 255;
        else
          out = (uint8_t)v;
        q[(int64_t)r * cols + (int64_t)blk * block_size + i] = out;
      }
    }
  }
}

void adr_o_dequant_table(uint16_t* out) {
#pragma omp parallel for schedule(static)
  for (int q = 0; q < 256; q++)
    for (int s = 0; s < 65536; s++) out[(int64_t)q * 65536 + s] = dequant_one((uint8_t)q, (uint16_t)s);
}

/* ---- softmax_rows (normalize.cu:147-220) ------------------------------------------------ */

/* xor-butterfly over `n` values (n a power of two), as __shfl_xor_sync with offsets n/2 .. 1
 * leaves it in lane 0; op 0 = fmaxf, 1 = + */
static float xor_tree(float* v, int n, int op) {
  float tmp[32];
  for (int off = n / 2; off > 0; off /= 2) {
    for (int i = 0; i < n; i++) {
      float o = v[i ^ off];
      tmp[i] = op ? v[i] + o : fmaxf(v[i], o);
    }
    memcpy(v, tmp, sizeof(float) * n);
  }
  return v[0];
}

void adr_o_softmax_rows(uint16_t* output, const uint16_t* input, int64_t rows, int w, float temp,
                        int mode) {
  for (int64_t r = 0; r < rows; r++) {
    const uint16_t* in = input + r * w;
    uint16_t* out = output + r * w;
    if (mode == 1) {
      double mx = -INFINITY, sum = 0.0;
      for (int i = 0; i < w; i++) mx = fmax(mx, (double)adr_o_h2f(in[i]) / (double)temp);
      for (int i = 0; i < w; i++) sum += exp((double)adr_o_h2f(in[i]) / (double)temp - mx);
      for (int i = 0; i < w; i++)
        out[i] = adr_o_d2h(exp((double)adr_o_h2f(in[i]) / (double)temp - mx) / sum);
      continue;
    }
    /* :160-163 per-thread maxima, thread t takes i = t, t + 256, ... */
    float part[256], grp[8];
    for (int t = 0; t < 256; t++) {
      float m = -INFINITY;
      for (int i = t; i < w; i += 256) m = fmaxf(m, adr_o_h2f(in[i]) / temp);
      part[t] = m;
    }
    /* :166-184 32-lane trees, then the 8 leaders */
    for (int g = 0; g < 8; g++) grp[g] = xor_tree(part + 32 * g, 32, 0);
    const float mx = xor_tree(grp, 8, 0);
    /* :186-191 */
    for (int t = 0; t < 256; t++) {
      float sacc = 0.0f;
      for (int i = t; i < w; i += 256) sacc += expf(adr_o_h2f(in[i]) / temp - mx);
      part[t] = sacc;
    }
    /* :193-211 */
    for (int g = 0; g < 8; g++) grp[g] = xor_tree(part + 32 * g, 32, 1);
    const float sum = xor_tree(grp, 8, 1);
    /* :213-216 */
    for (int i = 0; i < w; i++) out[i] = adr_o_f2h(expf(adr_o_h2f(in[i]) / temp - mx) / sum);
  }
}

/* ---- error_stats (error_stats.cu:13-75) ---------------------------------------------------- */
void adr_o_error_stats(float* out, const void* lhs, const void* rhs, int64_t length, int is_f32) {
  const int64_t counted = (length / 128) * 128; /* :27-30 */
  double sum_sq = 0.0, sum = 0.0;
  float mx = 0.0f;
  for (int64_t i = 0; i < counted; i++) {
    const float a = is_f32 ? ((const float*)lhs)[i] : adr_o_h2f(((const uint16_t*)lhs)[i]);
    const float b = is_f32 ? ((const float*)rhs)[i] : adr_o_h2f(((const uint16_t*)rhs)[i]);
    const float d = a - b; /* :32 */
    sum_sq += (double)(d * d);
    sum += (double)fabsf(d);
    mx = fmaxf(mx, fabsf(d));
  }
  out[0] = (float)(sum_sq / (double)length);
  out[1] = mx;
  out[2] = (float)(sum / (double)length);
}

/* ---- blocked fp32 GEMM, the CPU-baseline counterpart of the reference's only host GEMM ------
 * (matrixmultiply::sgemm with its `threading` feature, adrastea_core/src/mel.rs:142-157 and
 * adrastea_core/Cargo.toml:12): out[m,n] = sum_k a[m,k] * b[n,k], all row-major fp32, B given as
 * [n,k] like the weights of the path.  Cache blocking (64 x 256 panels of B, 4 x 4 register
 * tiles over k) and OpenMP over row blocks; plain C, no intrinsics.  Baseline material for
 * bench.py only -- no parity claim rests on it beyond its test against numpy. */
void adr_o_sgemm_nt(float* out, const float* a, const float* b, int m, int k, int n, int threads) {
  enum { MB = 64, NB = 64, KB = 256 };
  if (threads < 1) threads = 1;
#pragma omp parallel for num_threads(threads) schedule(dynamic, 1) collapse(2)
  for (int i0 = 0; i0 < m; i0 += MB)
    for (int j0 = 0; j0 < n; j0 += NB) {
      const int i1 = i0 + MB < m ? i0 + MB : m, j1 = j0 + NB < n ? j0 + NB : n;
      for (int i = i0; i < i1; i++)
        for (int j = j0; j < j1; j++) out[(int64_t)i * n + j] = 0.0f;
      for (int k0 = 0; k0 < k; k0 += KB) {
        const int k1 = k0 + KB < k ? k0 + KB : k;
        int i = i0;
        for (; i + 4 <= i1; i += 4) {
          int j = j0;
          for (; j + 4 <= j1; j += 4) {
            float c[4][4] = {{0}};
            for (int kk = k0; kk < k1; kk++) {
              float av[4], bv[4];
              for (int u = 0; u < 4; u++) av[u] = a[(int64_t)(i + u) * k + kk];
              for (int v = 0; v < 4; v++) bv[v] = b[(int64_t)(j + v) * k + kk];
              for (int u = 0; u < 4; u++)
                for (int v = 0; v < 4; v++) c[u][v] += av[u] * bv[v];
            }
            for (int u = 0; u < 4; u++)
              for (int v = 0; v < 4; v++) out[(int64_t)(i + u) * n + j + v] += c[u][v];
          }
          for (; j < j1; j++)
            for (int u = 0; u < 4; u++) {
              float c = 0.0f;
              for (int kk = k0; kk < k1; kk++) c += a[(int64_t)(i + u) * k + kk] * b[(int64_t)j * k + kk];
              out[(int64_t)(i + u) * n + j] += c;
            }
        }
        for (; i < i1; i++)
          for (int j = j0; j < j1; j++) {
            float c = 0.0f;
            for (int kk = k0; kk < k1; kk++) c += a[(int64_t)i * k + kk] * b[(int64_t)j * k + kk];
            out[(int64_t)i * n + j] += c;
          }
      }
    }
}
