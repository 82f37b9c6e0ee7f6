// General strided/batched fp16 matmul: one thread per output element, any element strides.
//
// This is the correctness path (adr_matmul_f16_slow, and the fallback of adr_matmul_f16 for
// layouts no tiled kernel covers).  It reproduces the arithmetic of the reference's naive
// kernel (adrastea_kernels/cpp/matmul.cu:195-222) step for step: operands optionally scaled
// in fp16, the product formed in fp16, widened, and summed sequentially in fp32.
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

hipError_t launch_matmul_general(hipStream_t stream, const MatmulArgs& a) {
  const int64_t blocks = (int64_t)((a.n + GEN_TX - 1) / GEN_TX) * ((a.m + GEN_TY - 1) / GEN_TY);
  if (blocks > 0x7fffffffLL || a.batches > 65535) return hipErrorInvalidConfiguration;
  dim3 grid((unsigned)blocks, 1, a.batches);
  dim3 block(GEN_TX, GEN_TY, 1);
  hipLaunchKernelGGL(matmul_general_kernel, grid, block, 0, stream, a);
  return hipGetLastError();
}

}  // namespace adr
