// Shared device/host definitions of the gfx950 matmul kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/adrastea_kernels.h"

namespace adr {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// The 22 matmul arguments (adrastea_models/src/kernels.rs:864-887) as one POD.
struct MatmulArgs {
  half_t* output;
  const half_t* lhs;
  const half_t* rhs;
  int batches, m, k, n;
  int stride_ox, stride_oy, stride_oz;
  int stride_lx, stride_ly, stride_lz;
  int stride_rx, stride_ry, stride_rz;
  const half_t* bias;
  float beta;
  float scale;
  uint32_t store, load, mask;
  // u8-quantised right operand (adr_matmul_nt_fp16u8): rhs is then unused
  const uint8_t* rhs_q;
  const half_t* scales;
  int block_size;
  // caller-provided scratch for kernels that split K over workgroups (adr_matmul_f16_ws): fp32
  // partial tiles, fully rewritten by every launch that uses them; null / 0: no such kernel
  float* workspace;
  int64_t workspace_bytes;
};

// Internal store operator of the contiguous NT entry points (matmul_nt_wmma_16x128x256.cu:63-66):
// out = fp16(acc + beta * out), the accumulator is NOT narrowed first.  Not part of the ABI enum.
constexpr uint32_t STORE_ACC_BETA = 7;

__device__ __forceinline__ half_t bits_to_half(uint16_t b) { return __builtin_bit_cast(half_t, b); }
__device__ __forceinline__ uint16_t half_to_bits(half_t h) { return __builtin_bit_cast(uint16_t, h); }

// Store operators (adrastea_kernels/cpp/matmul.cu:418-491).  `acc` is the fp32 accumulator;
// it is narrowed to fp16 first because every reference operator takes a __half argument
// (matmul.cu:47-52, 64-71, 80-87).  `prev` is the element already in the output; callers
// load it only for the operators that read it (needs_prev()).
struct Epilogue {
  const half_t* bias;
  float beta;
  half_t hscale;
  uint32_t store;
  // false: expf / tanhf as the reference calls them (the step-for-step kernel).  true: the tiled
  // kernels' forms on the hardware's exp2 and reciprocal -- a few instructions per value instead
  // of some forty, relative error below 2e-6 before the narrowing to fp16:
  //   quick GELU   v sigmoid(1.702 v)                 = v / (1 + 2^(-1.702 log2e v))
  //   tanh GELU    0.5 v (1 + tanh(u)) = v sigmoid(2u) = v / (1 + 2^(-2 log2e u)),
  //                u = 0.79788456 (v + 0.044715 v^3)
  // (the second form has no 1 + tanh cancellation for negative v; infinities and NaN come out
  // as from the reference's expressions).
  bool fast = false;

  __host__ __device__ static bool needs_prev(uint32_t store) {
    return store == ADR_STORE_ADD || store == ADR_STORE_BETA_BIAS ||
           store == ADR_STORE_BETA_GELU_BIAS || store == STORE_ACC_BETA;
  }
  __host__ __device__ static bool needs_bias(uint32_t store) {
    return store == ADR_STORE_BETA_BIAS || store == ADR_STORE_BETA_GELU_BIAS ||
           store == ADR_STORE_QUICK_GELU_BIAS;
  }

  // Operators on the already narrowed accumulator (everything but STORE_ACC_BETA).
  __device__ __forceinline__ half_t apply_s16(half_t s16, half_t prev, half_t bias_x) const {
    switch (store) {
      default:
      case ADR_STORE_IDENTITY:
        return s16;
      case ADR_STORE_SCALE:
        return s16 * hscale;
      case ADR_STORE_ADD:
        return s16 + prev;
      case ADR_STORE_BETA_BIAS: {
        float v = (float)s16 + (float)bias_x;
        return (half_t)(v + beta * (float)prev);
      }
      case ADR_STORE_QUICK_GELU_BIAS: {
        float v = (float)s16 + (float)bias_x;
        if (fast) {
          const float e = __builtin_amdgcn_exp2f(-1.702f * 1.44269504088896341f * v);
          return (half_t)(v * __builtin_amdgcn_rcpf(1.0f + e));
        }
        return (half_t)(v * (1.0f / (1.0f + expf(-1.702f * v))));
      }
      case ADR_STORE_BETA_GELU_BIAS: {
        float v = (float)s16 + (float)bias_x;
        if (fast) {
          const float inner = fmaf(0.044715f * v * v, v, v);  // v + 0.044715 v^3
          const float e = __builtin_amdgcn_exp2f(-2.0f * 0.7978845608028654f * 1.44269504088896341f * inner);
          const float g = v * __builtin_amdgcn_rcpf(1.0f + e);
          return (half_t)(g + beta * (float)prev);
        }
        float g = 0.5f * v * (1.0f + tanhf(0.7978845608028654f * (v + 0.044715f * v * v * v)));
        return (half_t)(g + beta * (float)prev);
      }
    }
  }

  __device__ __forceinline__ half_t apply(float acc, half_t prev, half_t bias_x) const {
    if (store == STORE_ACC_BETA) return (half_t)(acc + beta * (float)prev);
    return apply_s16((half_t)acc, prev, bias_x);
  }
};

__device__ __forceinline__ half_t neg_inf_half() { return bits_to_half(0xFC00u); }

// One output element of the general strided/batched matmul, with the arithmetic of the
// reference's naive kernel (adrastea_kernels/cpp/matmul.cu:195-222) step for step: operands
// optionally scaled in fp16, the product formed in fp16, widened, and summed sequentially in
// fp32; then the mask and the store operator.  The caller guarantees y < m, x < n.
__device__ __forceinline__ void matmul_one_output(const MatmulArgs& a, int b, int y, int x) {
  half_t* out = a.output + (int64_t)b * a.stride_oz + (int64_t)y * a.stride_oy +
                (int64_t)x * a.stride_ox;
  if (a.mask == ADR_MASK_CAUSAL && x > y) {  // matmul.cu:210-213
    *out = neg_inf_half();
    return;
  }
  const half_t* l = a.lhs + (int64_t)b * a.stride_lz + (int64_t)y * a.stride_ly;
  const half_t* r = a.rhs + (int64_t)b * a.stride_rz + (int64_t)x * a.stride_rx;
  const half_t hscale = (half_t)a.scale;
  float sum = 0.0f;
  if (a.load == ADR_LOAD_SCALE) {
    for (int i = 0; i < a.k; i++) {
      half_t lv = l[(int64_t)i * a.stride_lx] * hscale;
      half_t rv = r[(int64_t)i * a.stride_ry] * hscale;
      half_t p = lv * rv;
      sum += (float)p;
    }
  } else {
    for (int i = 0; i < a.k; i++) {
      half_t p = l[(int64_t)i * a.stride_lx] * r[(int64_t)i * a.stride_ry];
      sum += (float)p;
    }
  }
  Epilogue ep{a.bias, a.beta, hscale, a.store};
  half_t prev = Epilogue::needs_prev(a.store) ? *out : (half_t)0;
  half_t bias_x = Epilogue::needs_bias(a.store) ? a.bias[x] : (half_t)0;
  *out = ep.apply(sum, prev, bias_x);
}

// Four u8 weights (one dword) -> four fp16 values (q - 127.5) * s with ONE rounding each, the
// reference's dequantisation (adrastea_kernels/cpp/quantize.cu:53-54) bit for bit:
// 0x6000 | (q << 1) is the fp16 number 512 + q (the step at 512 is 0.5); subtracting 639.5
// gives q - 127.5 exactly, and an fp16 multiply rounds the exact product once -- the same
// value as narrowing the (exact) fp32 product.  fp16 denormals are never flushed on gfx950.
__device__ __forceinline__ void dequant4(uint32_t w, half2_t s2, half2_t& lo, half2_t& hi) {
  uint32_t p01 = __builtin_amdgcn_perm(0u, w, 0x0c010c00u);  // 0x00 b1 00 b0
  uint32_t p23 = __builtin_amdgcn_perm(0u, w, 0x0c030c02u);  // 0x00 b3 00 b2
  p01 = (p01 << 1) | 0x60006000u;
  p23 = (p23 << 1) | 0x60006000u;
  const half2_t bias = {(half_t)639.5f, (half_t)639.5f};
  lo = (__builtin_bit_cast(half2_t, p01) - bias) * s2;
  hi = (__builtin_bit_cast(half2_t, p23) - bias) * s2;
}

// Eight consecutive u8 weights sharing one scale -> eight fp16 values in memory order.
__device__ __forceinline__ half8_t dequant8(uint32_t w0, uint32_t w1, half2_t s2) {
  half2_t a, b, c, d;
  dequant4(w0, s2, a, b);
  dequant4(w1, s2, c, d);
  half8_t r;
  r[0] = a[0]; r[1] = a[1]; r[2] = b[0]; r[3] = b[1];
  r[4] = c[0]; r[5] = c[1]; r[6] = d[0]; r[7] = d[1];
  return r;
}

typedef _Float16 h2_t __attribute__((ext_vector_type(2)));

// Eight halves from / to any even address in global memory, for tensors whose rows are not 16-byte
// aligned (a score tensor [heads, S, T] with T no multiple of 8).  Vector accesses need 4-byte
// alignment only: a chunk at a 4-byte aligned address moves as one dwordx4; a chunk 2 bytes off
// is read as the five dwords around it and shifted (v_alignbyte_b32), and written as its first
// half, three dwords and its last half -- whole dwords across a chunk's ends would touch halves that
// other lanes or other workgroups own.
typedef uint32_t u32x4_dword_aligned_t __attribute__((ext_vector_type(4), aligned(4)));
typedef uint32_t u32x2_dword_aligned_t __attribute__((ext_vector_type(2), aligned(4)));
#define ADR_GLOBAL_AS __attribute__((address_space(1)))

// `last`: the last dword that may be read (loads past it read it again: what they return lies
// beyond the row's end and must be masked by the caller)
__device__ __forceinline__ void load5_any(const half_t* p, uintptr_t last, uint32_t (&d)[5]) {
  const uintptr_t base = (uintptr_t)p & ~(uintptr_t)3;
  // (a wavefront-uniform branch: a load under a lane mask is waited for where the lanes rejoin)
  if (__builtin_amdgcn_ballot_w64(base + 16 > last) == 0) {
    const u32x4_t q = *(const ADR_GLOBAL_AS u32x4_dword_aligned_t*)base;
    d[0] = q[0]; d[1] = q[1]; d[2] = q[2]; d[3] = q[3];
    d[4] = *(const ADR_GLOBAL_AS uint32_t*)(base + 16);
  } else {
#pragma unroll
    for (int j = 0; j < 5; j++)
      d[j] = *(const ADR_GLOBAL_AS uint32_t*)(base + 4 * j < last ? base + 4 * j : last);
  }
}

// the eight halves that begin `shift` (0 or 2) bytes into the five dwords of load5_any
__device__ __forceinline__ u32x4_t align5(const uint32_t (&d)[5], uint32_t shift) {
  u32x4_t r;
#pragma unroll
  for (int j = 0; j < 4; j++) r[j] = __builtin_amdgcn_alignbyte(d[j + 1], d[j], shift);
  return r;
}

// load5_any in two halves with no branch around the loads, for loops that keep several slices of
// loads in flight (a branch that holds loads makes every later wait count for all of them).  The
// 16-byte load never starts beyond last - 12: near the end of the tensor it reads from further back
// and load5_finish picks the dwords that belong to the chunk.  What lies beyond `last` is
// unspecified, as for load5_any.  The tensor must hold at least 24 bytes.
__device__ __forceinline__ void load5_issue(const half_t* p, uintptr_t last, uint32_t (&d)[5]) {
  const uintptr_t base = (uintptr_t)p & ~(uintptr_t)3, lim = last - 12;
  const u32x4_t q = *(const ADR_GLOBAL_AS u32x4_dword_aligned_t*)(base < lim ? base : lim);
  d[0] = q[0]; d[1] = q[1]; d[2] = q[2]; d[3] = q[3];
  d[4] = *(const ADR_GLOBAL_AS uint32_t*)(base + 16 < last ? base + 16 : last);
}

__device__ __forceinline__ u32x4_t load5_finish(const half_t* p, uintptr_t last, const uint32_t (&d)[5]) {
  const uintptr_t base = (uintptr_t)p & ~(uintptr_t)3, lim = last - 12;
  uint32_t e[5] = {d[0], d[1], d[2], d[3], d[4]};
  if (__builtin_amdgcn_ballot_w64(base > lim) != 0) {
    // the 16 bytes were read s dwords further back: dword j of the chunk is dword j + s of them
    // (j + s <= 3 for every dword at or before `last`)
    const uintptr_t back = base > lim ? (base - lim) >> 2 : 0;
    const int s = back < 3 ? (int)back : 3;
    e[0] = s == 0 ? d[0] : s == 1 ? d[1] : s == 2 ? d[2] : d[3];
    e[1] = s == 0 ? d[1] : s == 1 ? d[2] : d[3];
    e[2] = s == 0 ? d[2] : d[3];
  }
  return align5(e, (uint32_t)((uintptr_t)p & 2));
}

__device__ __forceinline__ half8_t load8_any(const half_t* p, uintptr_t last) {
  uint32_t d[5];
  load5_any(p, last, d);
  return __builtin_bit_cast(half8_t, align5(d, (uint32_t)((uintptr_t)p & 2)));
}

__device__ __forceinline__ void store8_any(half_t* p, half8_t v) {
  const uintptr_t u = (uintptr_t)p;
  const u32x4_t r = __builtin_bit_cast(u32x4_t, v);
  if ((u & 2) == 0) {
    __builtin_nontemporal_store(r, (ADR_GLOBAL_AS u32x4_dword_aligned_t*)u);
  } else {
    typedef uint16_t ADR_GLOBAL_AS* gptr16_t;
    __builtin_nontemporal_store((uint16_t)(r[0] & 0xffffu), (gptr16_t)u);
    const u32x2_t m01 = {__builtin_amdgcn_alignbyte(r[1], r[0], 2u), __builtin_amdgcn_alignbyte(r[2], r[1], 2u)};
    __builtin_nontemporal_store(m01, (ADR_GLOBAL_AS u32x2_dword_aligned_t*)(u + 2));
    __builtin_nontemporal_store(__builtin_amdgcn_alignbyte(r[3], r[2], 2u), (ADR_GLOBAL_AS uint32_t*)(u + 10));
    __builtin_nontemporal_store((uint16_t)(r[3] >> 16), (gptr16_t)(u + 14));
  }
}

template <int CTRL, int ROWMASK>
__device__ __forceinline__ float dpp_add(float v) {
  int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROWMASK, 0xf, true);
  return v + __builtin_bit_cast(float, t);
}
// Sum over the 64 lanes with data-parallel-primitive adds (no LDS); the total is in lane 63.
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v = dpp_add<0x111, 0xf>(v);  // row_shr:1
  v = dpp_add<0x112, 0xf>(v);  // row_shr:2
  v = dpp_add<0x114, 0xf>(v);  // row_shr:4
  v = dpp_add<0x118, 0xf>(v);  // row_shr:8   lane 15 of each 16-lane row = row sum
  v = dpp_add<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v = dpp_add<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// The current device as the launchers see it (device.hip): status is ADR_OK on a gfx950 device,
// ADR_EUNSUPPORTED_DEVICE on any other, or the hipError_t of the failed query; cus / xcds are the
// device's compute-unit and die (XCD) counts -- MI355X: 256 and 8, which are also the values
// reported beside a non-zero status.  Queried once per device, immutable afterwards.
struct DeviceInfo {
  int status;
  int cus;
  int xcds;
};
DeviceInfo device_info();
DeviceInfo device_info_for_plan();  // as above, but an MI355X where no usable device is current

// Switches for tests and benchmarks (adr_debug_knob): they force a kernel choice that the
// dispatch would make by itself from the arguments.  0 = the dispatch decides.
enum Knob {
  KNOB_GEMM_TILE = 0,  // fp16 tiled GEMM: 1 + index into the tile list (gemm_mfma.hip: forced tile)
  KNOB_U8_TILE,        // u8-weight tiled GEMM: 1 + index into its tile list; one past the list: the staged kernels
  KNOB_LAB_B,
  KNOB_LAB_C,
  KNOB_COUNT
};
int knob(int id);

// Launchers implemented in the kernel translation units; all return a hipError_t.
hipError_t launch_matmul_general(hipStream_t stream, const MatmulArgs& a);
// Returns true and fills `name` when the MFMA kernel family covers these arguments.
bool mfma_gemm_supported(const MatmulArgs& a, const char** name);
hipError_t launch_mfma_gemm(hipStream_t stream, const MatmulArgs& a);
// Scratch bytes the split-K form of these arguments would use when at most `avail` bytes can be
// had (0: no split pays here, or none fits); the kernel family splits that way when a.workspace
// holds at least this much.
int64_t mfma_gemm_workspace_bytes(const MatmulArgs& a, int64_t avail = INT64_MAX);
// fp16 skinny matmul (m <= 32, K-contiguous operands): true when a streaming kernel covers it.
bool gemv_f16_supported(const MatmulArgs& a, const char** name);
hipError_t launch_gemv_f16(hipStream_t stream, const MatmulArgs& a);

hipError_t launch_gemm_u8(hipStream_t stream, half_t* out, const half_t* lhs, const uint8_t* rhs,
                          const half_t* scales, int m, int p, int n, int block_size, float beta);
const char* gemm_u8_plan(int m, int p, int n, int block_size);

hipError_t launch_dequantize(hipStream_t stream, adr_tensor_desc out, adr_tensor_desc scales,
                             adr_tensor_desc in);
hipError_t launch_quantize(hipStream_t stream, adr_tensor_desc out, adr_tensor_desc scales,
                           adr_tensor_desc in);
hipError_t launch_embed_u8(hipStream_t stream, int n_dim, int n_ids, const int16_t* in_ids,
                           half_t* out, const uint8_t* table, const half_t* scales,
                           int block_size);
hipError_t launch_microbench_empty(hipStream_t stream);
hipError_t launch_microbench_mfma(hipStream_t stream, int blocks, int times, int pattern, float* sink);
hipError_t launch_microbench_read(hipStream_t stream, const void* p, int64_t bytes, int blocks,
                                  uint32_t* sink);
hipError_t launch_error_stats(hipStream_t stream, float* out, const void* lhs, const void* rhs,
                              int64_t length, int64_t sl, int64_t sr, bool f32);
hipError_t launch_attention(hipStream_t stream, half_t* out, const half_t* q, const half_t* k,
                            const half_t* v, int heads, int m, int n, int d, int so_y, int so_z,
                            int sq_y, int sq_z, int sk_y, int sk_z, int sv_y, int sv_z, float scale,
                            float temp, uint32_t mask);
hipError_t launch_softmax_rows(hipStream_t stream, half_t* out, const half_t* in, int64_t rows,
                               int w, float temp);

}  // namespace adr
