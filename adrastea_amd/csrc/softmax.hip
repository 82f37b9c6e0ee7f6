// Row-wise softmax with temperature over a contiguous [heads, h, w] fp16 tensor
// (adrastea_kernels/cpp/normalize.cu:147-220; host call adrastea_models/src/kernels.rs:892-915,
// in place between QK^T and P.V at llama.rs:551, clip.rs:385, whisper.rs:432):
//   v_i   = float(in_i) / temp
//   out_i = fp16( expf(v_i - max_j v_j) / sum_j expf(v_j - max_j v_j) )
// The operation is bound by reading and writing the tensor once each.  Rows of up to 4096
// elements are held in registers by one wavefront (one pass over memory, shuffle reductions):
// 16-byte accesses where the rows are 16-byte aligned, shifted dword accesses where they start
// at any even address (a row length that is no multiple of 8); longer rows take a three-pass
// kernel with one workgroup per row.
#include "adr_common.hpp"

namespace adr {

namespace {

// e^x for x <= 0 (and NaN, and -inf -> 0) as the hardware's 2^t of t = x * log2 e.  The rounding
// of the product and of the constant put t off by at most 7.3e-8 |t|, the exp2 unit adds one ulp:
// a relative error below 1.4e-6 wherever the result can still be seen in fp16 (|t| < 25), 0.3 %
// of one fp16 step.  Carrying the product in two floats brings that to 2 ulp of expf but costs six
// more VALU instructions per element, and this kernel is bound by them as much as by memory
// (106 us against 95 us on 65536 rows of 2048).
__device__ __forceinline__ float exp_neg(float x) {
  return __builtin_amdgcn_exp2f(x * 1.44269502162933349609375f);
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
  // v / sum for 32+ values per lane: one reciprocal per row and a product per value (within
  // 1.5 ulp of the quotient, before the narrowing to fp16 takes 13 bits off)
  const float rs = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int c = (i * 64 + lane) * 8;
    if (c < w) {
      half8_t r;
#pragma unroll
      for (int e = 0; e < 8; e++) {
        r[e] = (half_t)(v[i][e] * rs);
      }
      // streaming store: the probabilities are consumed by a later launch
      __builtin_nontemporal_store(r, (half8_t*)(dst + c));
    }
  }
}

// The same for rows that start at any even address and hold any number of elements (w <= 512 * NV):
// a sequence length that is no multiple of 8 (Whisper's 1500 positions, CLIP's 77 and 257, any odd
// prompt length).  Chunks of eight halves counted from the row's first element, moved with
// load8_any / store8_any; the row's last, partial chunk is stored element by element.
template <int NV>
__global__ __launch_bounds__(256) void softmax_rows_anyrow_kernel(half_t* out, const half_t* in,
                                                                  int64_t rows, int w, float temp) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row = (int64_t)blockIdx.x * 4 + wave;
  if (row >= rows) return;
  const half_t* src = in + row * w;
  half_t* dst = out + row * w;
  const uintptr_t end = (uintptr_t)(in + rows * w);  // one past the tensor's last element
  const uintptr_t last = ((end + 3) & ~(uintptr_t)3) - 4;
  float v[NV][8];
  float mx = -INFINITY;
  const bool unit_temp = temp == 1.0f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int c = (i * 64 + lane) * 8;
    // (chunks past the row read the row's first chunk again: no load under a lane mask)
    const half8_t x = load8_any(src + (c < w ? c : 0), last);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      const float t = unit_temp ? (float)x[e] : (float)x[e] / temp;
      v[i][e] = c + e < w ? t : -INFINITY;
      mx = fmaxf(mx, v[i][e]);
    }
  }
  mx = wave_max(mx);
  float sum = 0.0f;
#pragma unroll
  for (int i = 0; i < NV; i++)
#pragma unroll
    for (int e = 0; e < 8; e++) {
      v[i][e] = exp_neg(v[i][e] - mx);  // (-inf - mx: 0 for the elements past the row)
      sum += v[i][e];
    }
  sum = wave_sum(sum);
  const float rs = 1.0f / sum;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int c = (i * 64 + lane) * 8;
    half8_t r;
#pragma unroll
    for (int e = 0; e < 8; e++) r[e] = (half_t)(v[i][e] * rs);
    if (c + 8 <= w) {
      store8_any(dst + c, r);
    } else if (c < w) {
#pragma unroll
      for (int e = 0; e < 8; e++)
        if (c + e < w) dst[c + e] = r[e];
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
  } else if (w <= 4096) {
    const int64_t blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    const dim3 grid((unsigned)blocks), block(256);
    if (w <= 512)
      hipLaunchKernelGGL(softmax_rows_anyrow_kernel<1>, grid, block, 0, stream, out, in, rows, w, temp);
    else if (w <= 1024)
      hipLaunchKernelGGL(softmax_rows_anyrow_kernel<2>, grid, block, 0, stream, out, in, rows, w, temp);
    else if (w <= 2048)
      hipLaunchKernelGGL(softmax_rows_anyrow_kernel<4>, grid, block, 0, stream, out, in, rows, w, temp);
    else
      hipLaunchKernelGGL(softmax_rows_anyrow_kernel<8>, grid, block, 0, stream, out, in, rows, w, temp);
  } else {
    if (rows > 0x7fffffffLL) return hipErrorInvalidConfiguration;
    hipLaunchKernelGGL(softmax_rows_general_kernel, dim3((unsigned)rows), dim3(256), 0, stream, out,
                       in, w, temp);
  }
  return hipGetLastError();
}

}  // namespace adr
