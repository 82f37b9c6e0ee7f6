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
#include "error_stats_body.hpp"

namespace adr {

namespace {

template <typename T>
__global__ __launch_bounds__(ES_NT) void error_stats_kernel(float* out, const T* lhs, const T* rhs,
                                                            int64_t counted, int64_t length,
                                                            int64_t sl, int64_t sr, bool vec) {
  error_stats_body<T>(out, lhs, rhs, counted, length, sl, sr, vec);
}

template <typename T>
hipError_t launch_t(hipStream_t stream, float* out, const T* lhs, const T* rhs, int64_t length,
                    int64_t sl, int64_t sr) {
  const int64_t counted = error_stats_counted(length);
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
