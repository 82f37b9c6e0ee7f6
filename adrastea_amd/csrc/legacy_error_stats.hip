// gfx950 code object "error_stats" for an UNMODIFIED host: the two device symbols the reference's
// Rust side looks up in its error_stats module (adrastea_kernels/cpp/error_stats.cu:64-75; bound
// at adrastea_models/src/kernels.rs:485-486), taking its three by-value tensor descriptors and
// launched as it launches them: 128 blocks x 1024 threads (kernels.rs:968-975, 986-993).  The
// kernel body is the library's own; 1024 threads per block is what it expects.
#include "error_stats_body.hpp"

using namespace adr;

namespace {

template <typename T>
__device__ __forceinline__ void run(const adr_tensor_desc& output, const adr_tensor_desc& lhs,
                                    const adr_tensor_desc& rhs) {
  const int64_t length = rhs.shape[0];  // error_stats.cu:25: the width of the right tensor
  const int64_t sl = lhs.strides[0], sr = rhs.strides[0];
  const bool vec = sl == 1 && sr == 1 && !(((uintptr_t)lhs.ptr | (uintptr_t)rhs.ptr) & 15);
  error_stats_body<T>((float*)output.ptr, (const T*)lhs.ptr, (const T*)rhs.ptr,
                      error_stats_counted(length), length, sl, sr, vec);
}

}  // namespace

extern "C" __global__ __launch_bounds__(ES_NT) void error_stats_f16(adr_tensor_desc output,
                                                                   adr_tensor_desc lhs,
                                                                   adr_tensor_desc rhs) {
  run<half_t>(output, lhs, rhs);
}

extern "C" __global__ __launch_bounds__(ES_NT) void error_stats_f32(adr_tensor_desc output,
                                                                   adr_tensor_desc lhs,
                                                                   adr_tensor_desc rhs) {
  run<float>(output, lhs, rhs);
}
