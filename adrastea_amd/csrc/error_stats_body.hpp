// Device code of the error statistics (see error_stats.hip for the definition of the operation).
#pragma once

#include "adr_common.hpp"

namespace adr {

__device__ __forceinline__ void atomic_max_nonneg(float* addr, float v) {
  // non-negative floats order like their bit patterns
  atomicMax((int*)addr, __builtin_bit_cast(int, v));
}

// Every workgroup ends in three atomics on the same three addresses, and the workgroups finish
// together: the atomics queue up behind each other at the end of the launch (1024 workgroups:
// 27 us of a 105 us launch).  Hence few, large workgroups -- one per CU, 16 wavefronts each.
constexpr int ES_NT = 1024;
constexpr int ES_MAX_BLOCKS = 256;

// The whole kernel as a device function: the library's kernel and the code object built for an
// unmodified host (legacy_error_stats.hip) both run it.  Expects ES_NT threads per workgroup.
template <typename T>
__device__ __forceinline__ void error_stats_body(float* out, const T* lhs, const T* rhs,
                                                 int64_t counted, int64_t length, int64_t sl,
                                                 int64_t sr, bool vec) {
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

// error_stats.cu:27-30: 128 blocks of floor(length / 128) elements are visited
__host__ __device__ inline int64_t error_stats_counted(int64_t length) { return (length / 128) * 128; }

}  // namespace adr
