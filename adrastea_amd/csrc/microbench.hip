// Device kernels of the microbenchmark (the counterparts of adrastea_kernels/cpp/microbench.cu:28-51,
// driven like adrastea/src/main.rs:486-553): an empty kernel for the launch overhead, a loop
// of matrix-core instructions on register operands for the issue peak of this part, and a plain
// streaming read for the memory peak one launch can reach.  Measurement aids only: nothing in
// the product calls them.
#include "adr_common.hpp"

namespace adr {

namespace {

__global__ void empty_kernel(int) {}

// Every wavefront issues `times` x 4 independent v_mfma_f32_32x32x16_f16 (four accumulators keep
// the pipe full without waiting for a result).  pattern 0: all-zero operands (the instruction
// rate alone); pattern 1: pseudo-random fp16 operands in [-1, 1) (what the part sustains when
// the multipliers toggle -- the power limit shows here).
__global__ __launch_bounds__(256) void mfma_loop_kernel(int times, int pattern, float* sink) {
  const uint32_t id = blockIdx.x * 256 + threadIdx.x;
  half8_t a, b;
#pragma unroll
  for (int e = 0; e < 8; e++) {
    uint32_t h = (id * 8 + e) * 2654435761u;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    // sign, exponent 14 (values in [0.5, 1)) and ten mantissa bits
    a[e] = pattern ? bits_to_half((uint16_t)((h & 0x83ffu) | 0x3800u)) : (half_t)0;
    b[e] = pattern ? bits_to_half((uint16_t)(((h >> 16) & 0x83ffu) | 0x3800u)) : (half_t)0;
  }
  float16_t acc[4];
#pragma unroll
  for (int q = 0; q < 4; q++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[q][r] = 0.0f;
  for (int i = 0; i < times; i++) {
#pragma unroll
    for (int q = 0; q < 4; q++) acc[q] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[q], 0, 0, 0);
  }
  float s = 0.0f;
#pragma unroll
  for (int q = 0; q < 4; q++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[q][r];
  sink[id] = s;
}

// The same count of instructions as a GEMM's inner loop issues them: 2 x 2 sub-tiles, every
// instruction with another pair of operands, and the operands themselves replaced after every
// four instructions (rotated through four random fragments each, in registers: still no memory
// traffic at all).  What the matrix pipe sustains when its inputs switch like a product's do.
__global__ __launch_bounds__(256) void mfma_rotating_kernel(int times, float* sink) {
  const uint32_t id = blockIdx.x * 256 + threadIdx.x;
  half8_t a[4], b[4];
#pragma unroll
  for (int i = 0; i < 4; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      uint32_t h = (id * 64 + i * 8 + e) * 2654435761u;
      h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
      a[i][e] = bits_to_half((uint16_t)((h & 0x83ffu) | 0x3800u));
      b[i][e] = bits_to_half((uint16_t)(((h >> 16) & 0x83ffu) | 0x3800u));
    }
  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
  for (int t = 0; t < times; t++) {
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int j = 0; j < 2; j++)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(b[j], a[i], acc[i][j], 0, 0, 0);
    const half8_t ta = a[0], tb = b[0];
    a[0] = a[1]; a[1] = a[2]; a[2] = a[3]; a[3] = ta;
    b[0] = b[1]; b[1] = b[2]; b[2] = b[3]; b[3] = tb;
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < 2; i++)
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) s += acc[i][j][r];
  sink[id] = s;
}

// The two MFMA shapes on a wavefront's 128 x 128 tile, as a GEMM's k-steps issue them: every
// block (row fragment i, column fragment j) of the tile once per k-step, fragments alternating
// between two register sets from one k-step to the next, random data, no memory traffic.
// WIDE: 4 x 4 blocks of v_mfma_f32_32x32x16_f16 (2 k-steps = 32 instructions = 2^20 flop per
// iteration); otherwise 8 x 8 blocks of v_mfma_f32_16x16x32_f16 (2 k-steps = 128 instructions =
// 2^21 flop).  Same flops per clock, but not the same power: the kernels choose between the
// two by this measurement.  (Inline assembly ties every accumulator to its registers; the
// builtins let the compiler move the 256 of them around between instructions.)
template <bool WIDE>
__global__ __launch_bounds__(256) void mfma_tile_kernel(int times, float* sink) {
  constexpr int F = WIDE ? 4 : 8;
  const uint32_t id = blockIdx.x * 256 + threadIdx.x;
  half8_t a[2][F], b[2][F];
#pragma unroll
  for (int q = 0; q < 2; q++)
#pragma unroll
    for (int i = 0; i < F; i++)
#pragma unroll
      for (int e = 0; e < 8; e++) {
        uint32_t h = ((id * 2 + q) * 64 + i * 8 + e) * 2654435761u;
        h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
        a[q][i][e] = bits_to_half((uint16_t)((h & 0x83ffu) | 0x3800u));
        b[q][i][e] = bits_to_half((uint16_t)(((h >> 16) & 0x83ffu) | 0x3800u));
      }
  typedef typename std::conditional<WIDE, float16_t, float4_t>::type acc_t;
  acc_t acc[F][F];
#pragma unroll
  for (int i = 0; i < F; i++)
#pragma unroll
    for (int j = 0; j < F; j++)
#pragma unroll
      for (int r = 0; r < (WIDE ? 16 : 4); r++) acc[i][j][r] = 0.0f;
  for (int t = 0; t < times; t++) {
#pragma unroll
    for (int q = 0; q < 2; q++)
#pragma unroll
      for (int i = 0; i < F; i++)
#pragma unroll
        for (int j = 0; j < F; j++) {
          if constexpr (WIDE)
            asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b[q][j]), "v"(a[q][i]));
          else
            asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(b[q][j]), "v"(a[q][i]));
        }
  }
  float s = 0.0f;
#pragma unroll
  for (int i = 0; i < F; i++)
#pragma unroll
    for (int j = 0; j < F; j++)
#pragma unroll
      for (int r = 0; r < (WIDE ? 16 : 4); r++) s += acc[i][j][r];
  sink[id] = s;
}

// Every workgroup reads one contiguous piece with 16-byte streaming loads (the access shape
// that reads fastest on this part), four loads in flight per lane.
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4_t* p, int64_t n16,
                                                          uint32_t* sink) {
  const int64_t piece = n16 / gridDim.x;
  const u32x4_t* q = p + (int64_t)blockIdx.x * piece;
  u32x4_t acc = {0, 0, 0, 0};
  int64_t i = threadIdx.x;
  for (; i + 3 * 256 < piece; i += 4 * 256) {
    u32x4_t v[4];
#pragma unroll
    for (int u = 0; u < 4; u++) v[u] = __builtin_nontemporal_load(q + i + u * 256);
#pragma unroll
    for (int u = 0; u < 4; u++) acc ^= v[u];
  }
  for (; i < piece; i += 256) acc ^= q[i];
  const uint32_t r = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (r == 0x9e3779b9u) sink[0] = r;  // keeps the loads alive; practically never taken
}

}  // namespace

hipError_t launch_microbench_empty(hipStream_t stream) {
  hipLaunchKernelGGL(empty_kernel, dim3(1), dim3(1), 0, stream, 0);
  return hipGetLastError();
}

hipError_t launch_microbench_mfma(hipStream_t stream, int blocks, int times, int pattern, float* sink) {
  if (pattern == 4)
    hipLaunchKernelGGL(mfma_tile_kernel<false>, dim3(blocks), dim3(256), 0, stream, times, sink);
  else if (pattern == 3)
    hipLaunchKernelGGL(mfma_tile_kernel<true>, dim3(blocks), dim3(256), 0, stream, times, sink);
  else if (pattern == 2)
    hipLaunchKernelGGL(mfma_rotating_kernel, dim3(blocks), dim3(256), 0, stream, times, sink);
  else
    hipLaunchKernelGGL(mfma_loop_kernel, dim3(blocks), dim3(256), 0, stream, times, pattern, sink);
  return hipGetLastError();
}

hipError_t launch_microbench_read(hipStream_t stream, const void* p, int64_t bytes, int blocks,
                                  uint32_t* sink) {
  hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(256), 0, stream, (const u32x4_t*)p,
                     bytes / 16, sink);
  return hipGetLastError();
}

}  // namespace adr
