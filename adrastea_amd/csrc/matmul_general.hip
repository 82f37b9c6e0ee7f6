// General strided/batched fp16 matmul: one thread per output element, any element strides.
//
// This is the correctness path (adr_matmul_f16_slow, and the fallback of adr_matmul_f16 for
// layouts no tiled kernel covers): matmul_one_output() per thread, the arithmetic of the
// reference's naive kernel (adrastea_kernels/cpp/matmul.cu:195-222) step for step.
#include "adr_common.hpp"

namespace adr {

// 64 x 4 threads: consecutive lanes walk the x (column) dimension, so for row-major
// right operands and outputs a wavefront touches 64 consecutive elements.
constexpr int GEN_TX = 64;
constexpr int GEN_TY = 4;

__global__ __launch_bounds__(GEN_TX* GEN_TY) void matmul_general_kernel(MatmulArgs a) {
  // blockIdx.x enumerates (row block, column block) so that M is not capped by the 65535
  // limit of the y grid dimension
  const int nbx = (a.n + GEN_TX - 1) / GEN_TX;
  const int x = (blockIdx.x % nbx) * GEN_TX + threadIdx.x;
  const int y = (blockIdx.x / nbx) * GEN_TY + threadIdx.y;
  const int b = blockIdx.z;
  if (y >= a.m || x >= a.n) return;
  matmul_one_output(a, b, y, x);
}

hipError_t launch_matmul_general(hipStream_t stream, const MatmulArgs& a) {
  const int64_t blocks = (int64_t)((a.n + GEN_TX - 1) / GEN_TX) * ((a.m + GEN_TY - 1) / GEN_TY);
  if (blocks > 0x7fffffffLL || a.batches > 65535) return hipErrorInvalidConfiguration;
  dim3 grid((unsigned)blocks, 1, a.batches);
  dim3 block(GEN_TX, GEN_TY, 1);
  hipLaunchKernelGGL(matmul_general_kernel, grid, block, 0, stream, a);
  return hipGetLastError();
}

}  // namespace adr
