// u8 absmax quantisation format kernels.
//
// Format (adrastea_kernels/cpp/quantize.cu:3-56): weights [rows, cols] u8, one fp16 scale per
// (row, block of `block_size` consecutive columns), implicit midpoint 127.5, nothing else stored.
//   dequantise: out = fp16((float(q) - 127.5f) * float(scale))
//   quantise:   scale = fp16(absmax / 127.5f);  q = u8(round(127.5f + x / float(scale)))
//
// Both kernels take the reference's by-value descriptors (index 0 = innermost dimension) so
// that strided views work; the flat-pointer C entry points build contiguous descriptors.
#include "adr_common.hpp"

namespace adr {

// (q - 127.5) has at most 9 significant bits and an fp16 scale 11, so the fp32 product is exact
// and the narrowing is the only rounding: the result is bit-identical to the reference on any
// hardware with IEEE conversions.
__device__ __forceinline__ half_t dequant_one(uint8_t q, half_t s) {
  return (half_t)(((float)q - 127.5f) * (float)s);
}

// One workgroup per (row, group of blocks): 256 threads, each converts 8 consecutive weights
// when the row is contiguous and 8-aligned, else one at a time.
__global__ __launch_bounds__(256) void dequantize_kernel(adr_tensor_desc out, adr_tensor_desc scales,
                                                         adr_tensor_desc in, int block_size) {
  const uint32_t row = blockIdx.x;  // rows on the x grid dimension: no 65535 cap
  const uint32_t cols = out.shape[0];
  half_t* o = (half_t*)out.ptr + (size_t)row * out.strides[1];
  const uint8_t* q = (const uint8_t*)in.ptr + (size_t)row * in.strides[1];
  const half_t* s = (const half_t*)scales.ptr + (size_t)row * scales.strides[1];
  const bool vec = out.strides[0] == 1 && in.strides[0] == 1 && (block_size % 8) == 0 &&
                   (((uintptr_t)o | (uintptr_t)(o + out.strides[1])) % 16) == 0 &&
                   (((uintptr_t)q | (uintptr_t)(q + in.strides[1])) % 8) == 0;
  if (vec) {
    for (uint32_t c = (blockIdx.y * 256 + threadIdx.x) * 8; c < cols; c += gridDim.y * 256 * 8) {
      u32x2_t w = *(const u32x2_t*)(q + c);
      half_t sc = s[(size_t)(c / block_size) * scales.strides[0]];
      half8_t r;
#pragma unroll
      for (int j = 0; j < 8; j++) r[j] = dequant_one((uint8_t)((j < 4 ? w[0] : w[1]) >> (8 * (j & 3))), sc);
      *(half8_t*)(o + c) = r;
    }
  } else {
    for (uint32_t c = blockIdx.y * 256 + threadIdx.x; c < cols; c += gridDim.y * 256) {
      half_t sc = s[(size_t)(c / block_size) * scales.strides[0]];
      o[(size_t)c * out.strides[0]] = dequant_one(q[(size_t)c * in.strides[0]], sc);
    }
  }
}

// One wavefront per (row, block): absmax by a butterfly over the 64 lanes, then quantise.
__global__ __launch_bounds__(256) void quantize_kernel(adr_tensor_desc out, adr_tensor_desc scales,
                                                       adr_tensor_desc in, int block_size,
                                                       int blocks_per_row) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int blk = blockIdx.y * 4 + wave;
  const uint32_t row = blockIdx.x;
  if (blk >= blocks_per_row) return;
  const half_t* x = (const half_t*)in.ptr + (size_t)row * in.strides[1];
  uint8_t* q = (uint8_t*)out.ptr + (size_t)row * out.strides[1];
  const int c0 = blk * block_size;
  float absmax = 0.0f;
  for (int i = lane; i < block_size; i += 64)
    absmax = fmaxf(absmax, fabsf((float)x[(size_t)(c0 + i) * in.strides[0]]));
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) absmax = fmaxf(absmax, __shfl_xor(absmax, off, 64));
  const half_t hs = (half_t)(absmax / 127.5f);  // quantize.cu:33
  if (lane == 0) ((half_t*)scales.ptr)[(size_t)row * scales.strides[1] + (size_t)blk * scales.strides[0]] = hs;
  const float fs = (float)hs;
  for (int i = lane; i < block_size; i += 64) {
    // quantize.cu:41-42.  roundf = half away from zero.  The reference's float -> uint8 cast is
    // undefined for NaN / out-of-range values (zero or infinite scale); here NaN gives 0 and the
    // rest saturates.
    float v = roundf(127.5f + (float)x[(size_t)(c0 + i) * in.strides[0]] / fs);
    uint8_t r = (v != v) ? 0 : (uint8_t)fminf(fmaxf(v, 0.0f), 255.0f);
    q[(size_t)(c0 + i) * out.strides[0]] = r;
  }
}

// Contiguous rows, block sizes 8 * 2^k <= 512: a lane takes 8 consecutive values (one 16-byte
// load, one 8-byte store), the bs/8 lanes of a block find the absmax with xor shuffles.  Same
// arithmetic, operation for operation, as quantize_kernel.
__global__ __launch_bounds__(256) void quantize_vec_kernel(adr_tensor_desc out, adr_tensor_desc scales,
                                                           adr_tensor_desc in, int block_size) {
  const uint32_t row = blockIdx.x;
  const uint32_t cols = in.shape[0];
  const uint32_t c = (blockIdx.y * 256 + threadIdx.x) * 8;
  const bool live = c < cols;  // cols % block_size == 0, so a block is all live or all dead
  const half_t* x = (const half_t*)in.ptr + (size_t)row * in.strides[1];
  uint8_t* q = (uint8_t*)out.ptr + (size_t)row * out.strides[1];
  half8_t v = {0, 0, 0, 0, 0, 0, 0, 0};
  if (live) v = *(const half8_t*)(x + c);
  float absmax = 0.0f;
#pragma unroll
  for (int e = 0; e < 8; e++) absmax = fmaxf(absmax, fabsf((float)v[e]));
  const int lanes = block_size / 8;
  for (int off = 1; off < lanes; off <<= 1) absmax = fmaxf(absmax, __shfl_xor(absmax, off, 64));
  if (!live) return;
  const half_t hs = (half_t)(absmax / 127.5f);  // quantize.cu:33
  if ((c % block_size) == 0)
    ((half_t*)scales.ptr)[(size_t)row * scales.strides[1] + (size_t)(c / block_size) * scales.strides[0]] = hs;
  const float fs = (float)hs;
  uint32_t w[2] = {0, 0};
#pragma unroll
  for (int e = 0; e < 8; e++) {
    float r = roundf(127.5f + (float)v[e] / fs);  // quantize.cu:41-42
    uint32_t b = (r != r) ? 0u : (uint32_t)fminf(fmaxf(r, 0.0f), 255.0f);
    w[e >> 2] |= b << (8 * (e & 3));
  }
  *(u32x2_t*)(q + c) = u32x2_t{w[0], w[1]};
}

// Embedding lookup in a u8-quantised table (adrastea_kernels/cpp/embed_uint8.cu:3-19):
//   out[t, i] = fp16( (float(table[id_t, i]) - 127.5f) * float(scales[id_t, i / block_size]) )
// with id_t = in_ids[t] (16-bit ids, as in the reference).  A gather of n_ids rows: one
// workgroup column per id, eight weights per lane (8-byte load, one scale, 16-byte store).
__global__ __launch_bounds__(256) void embed_u8_vec_kernel(int n_dim, const int16_t* in_ids,
                                                           half_t* out, const uint8_t* table,
                                                           const half_t* scales, int block_size) {
  const int t = blockIdx.x;
  const int i = (blockIdx.y * 256 + threadIdx.x) * 8;
  if (i >= n_dim) return;
  const int64_t id = in_ids[t];
  const u32x2_t w = *(const u32x2_t*)(table + id * n_dim + i);
  const half_t sv = scales[id * (n_dim / block_size) + i / block_size];
  half8_t r;
#pragma unroll
  for (int j = 0; j < 8; j++) r[j] = dequant_one((uint8_t)((j < 4 ? w[0] : w[1]) >> (8 * (j & 3))), sv);
  *(half8_t*)(out + (int64_t)t * n_dim + i) = r;
}

__global__ __launch_bounds__(256) void embed_u8_kernel(int n_dim, const int16_t* in_ids,
                                                       half_t* out, const uint8_t* table,
                                                       const half_t* scales, int block_size) {
  const int t = blockIdx.x;
  const int64_t id = in_ids[t];
  const int block_count = n_dim / block_size;
  for (int i = blockIdx.y * 256 + threadIdx.x; i < n_dim; i += gridDim.y * 256) {
    const float sv = (float)scales[id * block_count + i / block_size];
    out[(int64_t)t * n_dim + i] = (half_t)(((float)table[id * n_dim + i] - 127.5f) * sv);
  }
}

hipError_t launch_dequantize(hipStream_t stream, adr_tensor_desc out, adr_tensor_desc scales,
                             adr_tensor_desc in) {
  const uint32_t cols = out.shape[0], rows = out.shape[1];
  const int block_size = cols / scales.shape[0];
  uint32_t gy = (cols + 256 * 8 - 1) / (256 * 8);
  if (gy > 64) gy = 64;
  hipLaunchKernelGGL(dequantize_kernel, dim3(rows, gy, 1), dim3(256, 1, 1), 0, stream, out, scales,
                     in, block_size);
  return hipGetLastError();
}

hipError_t launch_quantize(hipStream_t stream, adr_tensor_desc out, adr_tensor_desc scales,
                           adr_tensor_desc in) {
  const uint32_t cols = out.shape[0], rows = out.shape[1];
  const int blocks_per_row = scales.shape[0];
  const int block_size = cols / blocks_per_row;
  const int lanes = block_size / 8;
  const bool vec = block_size % 8 == 0 && lanes <= 64 && (lanes & (lanes - 1)) == 0 &&
                   in.strides[0] == 1 && out.strides[0] == 1 && in.strides[1] % 8 == 0 &&
                   out.strides[1] % 8 == 0 && (uintptr_t)in.ptr % 16 == 0 &&
                   (uintptr_t)out.ptr % 8 == 0 && (cols + 2047) / 2048 <= 65535;
  if (vec) {
    hipLaunchKernelGGL(quantize_vec_kernel, dim3(rows, (cols + 2047) / 2048, 1), dim3(256, 1, 1), 0,
                       stream, out, scales, in, block_size);
    return hipGetLastError();
  }
  if ((blocks_per_row + 3) / 4 > 65535) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(quantize_kernel, dim3(rows, (blocks_per_row + 3) / 4, 1), dim3(256, 1, 1), 0,
                     stream, out, scales, in, block_size, blocks_per_row);
  return hipGetLastError();
}

hipError_t launch_embed_u8(hipStream_t stream, int n_dim, int n_ids, const int16_t* in_ids,
                           half_t* out, const uint8_t* table, const half_t* scales,
                           int block_size) {
  const bool vec = n_dim % 8 == 0 && block_size % 8 == 0 && (uintptr_t)table % 8 == 0 &&
                   (uintptr_t)out % 16 == 0;
  if (vec) {
    hipLaunchKernelGGL(embed_u8_vec_kernel, dim3(n_ids, (n_dim + 2047) / 2048, 1), dim3(256), 0,
                       stream, n_dim, in_ids, out, table, scales, block_size);
  } else {
    int gy = (n_dim + 255) / 256;
    if (gy > 64) gy = 64;
    hipLaunchKernelGGL(embed_u8_kernel, dim3(n_ids, gy, 1), dim3(256), 0, stream, n_dim, in_ids,
                       out, table, scales, block_size);
  }
  return hipGetLastError();
}

}  // namespace adr
