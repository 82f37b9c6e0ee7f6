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
  if ((blocks_per_row + 3) / 4 > 65535) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL(quantize_kernel, dim3(rows, (blocks_per_row + 3) / 4, 1), dim3(256, 1, 1), 0,
                     stream, out, scales, in, block_size, blocks_per_row);
  return hipGetLastError();
}

}  // namespace adr
