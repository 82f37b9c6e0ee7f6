// Row-wise softmax with temperature over a contiguous [heads, h, w] fp16 tensor
// (adrastea_kernels/cpp/normalize.cu:147-220; host call adrastea_models/src/kernels.rs:892-915,
// in place between QK^T and P.V at llama.rs:551, clip.rs:385, whisper.rs:432):
//   v_i   = float(in_i) / temp
//   out_i = fp16( expf(v_i - max_j v_j) / sum_j expf(v_j - max_j v_j) )
// The operation is bound by reading and writing the tensor once each.  Rows of up to 4096
// elements are held in registers by one wavefront (16-byte loads, one pass over memory, shuffle
// reductions); anything else takes a three-pass kernel with one workgroup per row.
#include "adr_common.hpp"

namespace adr {

namespace {

// e^x for x <= 0 (and NaN): 2^(x log2 e) with the product carried in two floats, so that the
// argument of the hardware exp2 (1 ulp) is exact to well below its own error: the result is
// within 2 ulp of expf over the whole range, which is 2^-11 of one fp16 step.  Six VALU
// instructions instead of the library routine's two dozen: this kernel is otherwise bound by them.
__device__ __forceinline__ float exp_neg(float x) {
  const float L2E_HI = 1.44269502162933349609375f;       // fp32(log2 e)
  const float L2E_LO = 1.92596299112661746e-8f;          // log2 e - L2E_HI
  const float t = x * L2E_HI;
  const float lo = fmaf(x, L2E_LO, fmaf(x, L2E_HI, -t));  // x log2 e - t
  const float p = __builtin_amdgcn_exp2f(t);
  // 2^t * 2^lo ~ p (1 + lo ln 2); x = -inf makes lo NaN but p exactly 0
  return p == 0.0f ? 0.0f : fmaf(p, lo * 0.693147180559945309f, p);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// NV 16-byte vectors per lane: rows of w <= 512 * NV elements, w % 8 == 0, 16-byte aligned rows.
template <int NV>
__global__ __launch_bounds__(256) void softmax_rows_reg_kernel(half_t* out, const half_t* in,
                                                               int64_t rows, int w, float temp) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  const half_t* src = in + row * w;
  half_t* dst = out + row * w;
  float v[NV][8];
  float mx = -INFINITY;
  const bool unit_temp = temp == 1.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int c = (i * 64 + lane) * 8;
    if (c < w) {
      const half8_t x = *(const half8_t*)(src + c);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        v[i][e] = unit_temp ? (float)x[e] : (float)x[e] / temp;  // x / 1 == x: skip the division
        mx = fmaxf(mx, v[i][e]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) v[i][e] = -INFINITY;
    }
  }
  mx = wave_max(mx);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int c = (i * 64 + lane) * 8;
    if (c < w) {
#pragma unroll
      for (int e = 0; e < 8; e++) {
        v[i][e] = exp_neg(v[i][e] - mx);
        sum += v[i][e];
      }
    }
  }
  sum = wave_sum(sum);
  // v / sum for 32+ values per lane: one reciprocal per row, then a product and one residual
  // correction per value (q = v * r; q += (v - q * sum) * r), which gives the correctly
  // rounded quotient for these operands (1 <= sum <= w, 0 <= v <= 1) at a third of the
  // instructions of a full division
  const float rs = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int c = (i * 64 + lane) * 8;
    if (c < w) {
      half8_t r;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float q = v[i][e] * rs;
        q = fmaf(fmaf(-q, sum, v[i][e]), rs, q);
        r[e] = (half_t)q;
      }
      // streaming store: the probabilities are consumed by a later launch
      __builtin_nontemporal_store(r, (half8_t*)(dst + c));
    }
  }
}

// Any width and alignment: one workgroup per row, three passes over the row.
__global__ __launch_bounds__(256) void softmax_rows_general_kernel(half_t* out, const half_t* in,
                                                                   int w, float temp) {
  __shared__ float red[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int64_t row = blockIdx.x;
  const half_t* src = in + row * w;
  half_t* dst = out + row * w;
  float mx = -INFINITY;
  for (int i = tid; i < w; i += 256) mx = fmaxf(mx, (float)src[i] / temp);
  mx = wave_max(mx);
  if (lane == 0) red[wave] = mx;
  __syncthreads();
  mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  float sum = 0.0f;
  for (int i = tid; i < w; i += 256) sum += expf((float)src[i] / temp - mx);
  sum = wave_sum(sum);
  if (lane == 0) red[wave] = sum;
  __syncthreads();
  sum = (red[0] + red[1]) + (red[2] + red[3]);
  // in place: an element is read and then written by the same thread
  for (int i = tid; i < w; i += 256) dst[i] = (half_t)(expf((float)src[i] / temp - mx) / sum);
}

}  // namespace

hipError_t launch_softmax_rows(hipStream_t stream, half_t* out, const half_t* in, int64_t rows,
                               int w, float temp) {
  const bool vec = w % 8 == 0 && w <= 4096 && ((uintptr_t)out % 16) == 0 && ((uintptr_t)in % 16) == 0;
  if (vec) {
    const int64_t blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    const dim3 grid((unsigned)blocks), block(256);
    if (w <= 512)
      hipLaunchKernelGGL(softmax_rows_reg_kernel<1>, grid, block, 0, stream, out, in, rows, w, temp);
    else if (w <= 1024)
      hipLaunchKernelGGL(softmax_rows_reg_kernel<2>, grid, block, 0, stream, out, in, rows, w, temp);
    else if (w <= 2048)
      hipLaunchKernelGGL(softmax_rows_reg_kernel<4>, grid, block, 0, stream, out, in, rows, w, temp);
    else
      hipLaunchKernelGGL(softmax_rows_reg_kernel<8>, grid, block, 0, stream, out, in, rows, w, temp);
  } else {
    if (rows > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL(softmax_rows_general_kernel, dim3((unsigned)rows), dim3(256), 0, stream, out,
                       in, w, temp);
  }
  return hipGetLastError();
}

}  // namespace adr
