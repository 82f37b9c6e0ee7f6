// Error statistics of two tensors on the device (adrastea_kernels/cpp/error_stats.cu:13-75; host
// call adrastea_models/src/kernels.rs:736-751 and the f16 twin above it): for 1-d views lhs, rhs of
// `length` elements, accumulated into a caller-zeroed fp32 output of three values,
//   output[0] += sum (l - r)^2 / length     output[1] = max(output[1], max |l - r|)
//   output[2] += sum |l - r| / length
// The reference walks the data with 128 blocks of floor(length / 128) elements each, so the last
// length % 128 elements do not enter the statistics while the means still divide by `length`;
// that is kept.  Differences are formed in fp32 from the stored values, as there.
// Bound by reading both tensors once: 16-byte loads on contiguous views, shuffle reductions,
// one atomic triple per workgroup of 1024 threads.
#include "adr_common.hpp"

namespace adr {

namespace {

__device__ __forceinline__ void atomic_max_nonneg(float* addr, float v) {
  // non-negative floats order like their bit patterns
  atomicMax((int*)addr, __builtin_bit_cast(int, v));
}

// Every workgroup ends in three atomics on the same three addresses, and the workgroups finish
// together: the atomics queue up behind each other at the end of the launch (1024 workgroups:
// 27 us of a 105 us launch).  Hence few, large workgroups -- one per CU, 16 wavefronts each.
constexpr int ES_NT = 1024;
constexpr int ES_MAX_BLOCKS = 256;

template <typename T>
__global__ __launch_bounds__(ES_NT) void error_stats_kernel(float* out, const T* lhs, const T* rhs,
                                                          int64_t counted, int64_t length,
                                                          int64_t sl, int64_t sr, bool vec) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(VEC)));
  float sum_sq = 0.0f, mx = 0.0f, sum = 0.0f;
  const int64_t tid = (int64_t)blockIdx.x * ES_NT + threadIdx.x, nthreads = (int64_t)gridDim.x * ES_NT;
  auto take = [&](float a, float b) {
    const float d = a - b;
    sum_sq += d * d;
    mx = fmaxf(mx, fabsf(d));
    sum += fabsf(d);
  };
  if (vec) {
    const int64_t nv = counted / VEC;
    int64_t i = tid;
    for (; i + nthreads < nv; i += 2 * nthreads) {  // four loads in flight per lane
      const vec_t a0 = __builtin_nontemporal_load((const vec_t*)(lhs + i * VEC));
      const vec_t b0 = __builtin_nontemporal_load((const vec_t*)(rhs + i * VEC));
      const vec_t a1 = __builtin_nontemporal_load((const vec_t*)(lhs + (i + nthreads) * VEC));
      const vec_t b1 = __builtin_nontemporal_load((const vec_t*)(rhs + (i + nthreads) * VEC));
#pragma unroll
      for (int e = 0; e < VEC; e++) take((float)a0[e], (float)b0[e]);
#pragma unroll
      for (int e = 0; e < VEC; e++) take((float)a1[e], (float)b1[e]);
    }
    for (; i < nv; i += nthreads) {
      const vec_t a = *(const vec_t*)(lhs + i * VEC), b = *(const vec_t*)(rhs + i * VEC);
#pragma unroll
      for (int e = 0; e < VEC; e++) take((float)a[e], (float)b[e]);
    }
    for (int64_t j = nv * VEC + tid; j < counted; j += nthreads) take((float)lhs[j], (float)rhs[j]);
  } else {
    for (int64_t i = tid; i < counted; i += nthreads) take((float)lhs[i * sl], (float)rhs[i * sr]);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    sum_sq += __shfl_xor(sum_sq, off, 64);
    mx = fmaxf(mx, __shfl_xor(mx, off, 64));
    sum += __shfl_xor(sum, off, 64);
  }
  constexpr int NW = ES_NT / 64;
  __shared__ float red[3][NW];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) { red[0][wave] = sum_sq; red[1][wave] = mx; red[2][wave] = sum; }
  __syncthreads();
  if (threadIdx.x == 0) {
    sum_sq = 0.0f; mx = 0.0f; sum = 0.0f;
    for (int w = 0; w < NW; w++) {
      sum_sq += red[0][w];
      mx = fmaxf(mx, red[1][w]);
      sum += red[2][w];
    }
    atomicAdd(out + 0, sum_sq / (float)length);  // error_stats.cu:59-61
    atomic_max_nonneg(out + 1, mx);
    atomicAdd(out + 2, sum / (float)length);
  }
}

template <typename T>
hipError_t launch_t(hipStream_t stream, float* out, const T* lhs, const T* rhs, int64_t length,
                    int64_t sl, int64_t sr) {
  const int64_t counted = (length / 128) * 128;  // error_stats.cu:27-30: 128 blocks of length/128
  const bool vec = sl == 1 && sr == 1 && ((uintptr_t)lhs % 16) == 0 && ((uintptr_t)rhs % 16) == 0;
  int64_t blocks = (counted / (16 / (int64_t)sizeof(T)) + ES_NT - 1) / ES_NT;
  if (blocks > ES_MAX_BLOCKS) blocks = ES_MAX_BLOCKS;
  if (blocks < 1) blocks = 1;
  hipLaunchKernelGGL(error_stats_kernel<T>, dim3((unsigned)blocks), dim3(ES_NT), 0, stream, out, lhs,
                     rhs, counted, length, sl, sr, vec);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_error_stats(hipStream_t stream, float* out, const void* lhs, const void* rhs,
                              int64_t length, int64_t sl, int64_t sr, bool f32) {
  return f32 ? launch_t<float>(stream, out, (const float*)lhs, (const float*)rhs, length, sl, sr)
             : launch_t<half_t>(stream, out, (const half_t*)lhs, (const half_t*)rhs, length, sl, sr);
}

}  // namespace adr
