// u8-quantised-weight skinny GEMM / GEMV for decode (m <= 16):
//   out[r,c] = fp16( sum_i lhs[r,i] * w[c,i] + beta * out[r,c] ),
//   w[c,i]   = fp16( (float(q[c,i]) - 127.5f) * float(scales[c, i/block_size]) )
// (adrastea_kernels/cpp/matmul_nt_wmma_16x128x256_fp16u8.cu:5-7, 43-83; format quantize.cu).
//
// The problem is bound by streaming the u8 weights from HBM once.  Each workgroup owns 16
// consecutive weight rows; its wavefronts split K in 256-element macro steps.  Per macro step
// a lane (row r = lane % 16, group g = lane / 16) streams 64 consecutive weight bytes of its
// row with four 128-bit loads -- four lanes cover 256 contiguous bytes of a row, whole cache
// lines -- plus one dword holding the two fp16 scales of those 64 weights.  The weights are
// dequantised in registers to packed fp16 and fed to v_mfma_f32_16x16x32_f16 as the A operand
// (16 weight rows x 32 k); the activations are the B operand (32 k x 16 activation rows, rows
// beyond m are zero).  The k slots of an MFMA may hold any 32 distinct k as long as both
// operands agree, which is what lets a lane use contiguous bytes.  Partial sums of the
// wavefronts are reduced through LDS.
#include "adr_common.hpp"

namespace adr {

namespace {

constexpr int MACRO_K = 256;  // k elements per macro step
constexpr int ROWS = 16;      // weight rows per workgroup

struct Stage {
  u32x4_t w[4];   // 64 weight bytes of this lane's row
  uint32_t sc;    // two fp16 scales (block_size 32) covering them
  u32x4_t x[8];   // 64 activation halves of this lane's activation row
};

template <int NW>
__global__ __launch_bounds__(NW * 64) void gemv_u8_kernel(half_t* __restrict__ out,
                                                          const half_t* __restrict__ lhs,
                                                          const uint8_t* __restrict__ rhs,
                                                          const half_t* __restrict__ scales,
                                                          int m, int p, int n, float beta) {
  __shared__ float partial[NW][ROWS * 16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * ROWS;
  const int row = min(n0 + r, n - 1);  // tail rows are clamped; their sums are not stored
  const int nblk = p / 32;
  const uint8_t* wrow = rhs + (int64_t)row * p + g * 64;
  const half_t* srow = scales + (int64_t)row * nblk + g * 2;
  const bool xvalid = r < m;
  const half_t* xrow = lhs + (int64_t)(xvalid ? r : 0) * p + g * 64;
  const int steps = p / MACRO_K;

  auto load = [&](Stage& s, int ms) {
    const uint8_t* wp = wrow + (int64_t)ms * MACRO_K;
#pragma unroll
    for (int j = 0; j < 4; j++) s.w[j] = __builtin_nontemporal_load((const u32x4_t*)(wp + j * 16));
    s.sc = *(const uint32_t*)(srow + ms * (MACRO_K / 32));
    const half_t* xp = xrow + (int64_t)ms * MACRO_K;
#pragma unroll
    for (int j = 0; j < 8; j++)
      s.x[j] = xvalid ? *(const u32x4_t*)(xp + j * 8) : u32x4_t{0, 0, 0, 0};
  };

  float4_t acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
  auto compute = [&](const Stage& s) {
    const half2_t sc = __builtin_bit_cast(half2_t, s.sc);
    const half2_t s_lo = {sc[0], sc[0]}, s_hi = {sc[1], sc[1]};
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const half2_t s2 = j < 2 ? s_lo : s_hi;
      half8_t a0 = dequant8(s.w[j][0], s.w[j][1], s2);
      half8_t a1 = dequant8(s.w[j][2], s.w[j][3], s2);
      half8_t b0 = __builtin_bit_cast(half8_t, s.x[2 * j]);
      half8_t b1 = __builtin_bit_cast(half8_t, s.x[2 * j + 1]);
      acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, acc0, 0, 0, 0);
      acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, acc1, 0, 0, 0);
    }
  };

  // two-stage software pipeline over this wavefront's macro steps (wave, wave+NW, ...)
  Stage s0, s1;
  int ms = wave;
  if (ms < steps) load(s0, ms);
  while (ms < steps) {
    const int nxt = ms + NW;
    if (nxt < steps) load(s1, nxt);
    compute(s0);
    ms = nxt;
    if (ms >= steps) break;
    const int nxt2 = ms + NW;
    if (nxt2 < steps) load(s0, nxt2);
    compute(s1);
    ms = nxt2;
  }

  // accumulator element i of lane (col = lane % 16, grp = lane / 16) is D[4*grp + i][col]:
  // weight row 4*grp + i, activation row col
#pragma unroll
  for (int i = 0; i < 4; i++) partial[wave][(4 * g + i) * 16 + r] = acc0[i] + acc1[i];
  __syncthreads();
  for (int e = tid; e < ROWS * 16; e += NW * 64) {
    const int mm = e / ROWS, nn = e % ROWS;  // consecutive threads -> consecutive output columns
    if (mm < m && n0 + nn < n) {
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; w++) sum += partial[w][nn * 16 + mm];
      half_t* o = out + (int64_t)mm * n + n0 + nn;
      // the previous output is read even for beta == 0, as the reference does
      *o = (half_t)(sum + beta * (float)*o);
    }
  }
}

// Safety net for shapes / alignments the streaming kernel does not take: one thread per
// output, dequantising each weight to fp16 exactly as above and accumulating in fp32.
__global__ __launch_bounds__(256) void gemm_u8_naive_kernel(half_t* out, const half_t* lhs,
                                                            const uint8_t* rhs,
                                                            const half_t* scales, int m, int p,
                                                            int n, int block_size, float beta) {
  const int c = blockIdx.x * 64 + (threadIdx.x & 63);
  const int r = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (r >= m || c >= n) return;
  const int nblk = p / block_size;
  float sum = 0.0f;
  for (int i = 0; i < p; i++) {
    half_t w = (half_t)(((float)rhs[(int64_t)c * p + i] - 127.5f) *
                        (float)scales[(int64_t)c * nblk + i / block_size]);
    sum += (float)lhs[(int64_t)r * p + i] * (float)w;
  }
  half_t* o = out + (int64_t)r * n + c;
  *o = (half_t)(sum + beta * (float)*o);
}

enum U8Choice { U8_NAIVE = 0, U8_GEMV, U8_GEMM };

U8Choice choose_u8(const void* lhs, const void* rhs, const void* scales, int m, int p, int n,
                   int block_size) {
  const bool aligned = ((uintptr_t)lhs % 16 == 0) && ((uintptr_t)rhs % 16 == 0) &&
                       ((uintptr_t)scales % 4 == 0);
  if (!aligned) return U8_NAIVE;
  if (m <= 16 && block_size == 32 && p % MACRO_K == 0) return U8_GEMV;
  if (block_size % 8 == 0 && p % 8 == 0) return U8_GEMM;
  return U8_NAIVE;
}

}  // namespace

hipError_t launch_gemm_u8_mfma(hipStream_t stream, half_t* out, const half_t* lhs,
                               const uint8_t* rhs, const half_t* scales, int m, int p, int n,
                               int block_size, float beta);

const char* gemm_u8_plan(int m, int p, int n, int block_size) {
  switch (choose_u8(nullptr, nullptr, nullptr, m, p, n, block_size)) {
    case U8_GEMV: return "gemv_u8_mfma16_stream";
    case U8_GEMM: return "gemm_nt_u8_mfma";
    default: return "gemm_u8_naive";
  }
}

hipError_t launch_gemm_u8(hipStream_t stream, half_t* out, const half_t* lhs, const uint8_t* rhs,
                          const half_t* scales, int m, int p, int n, int block_size, float beta) {
  switch (choose_u8(lhs, rhs, scales, m, p, n, block_size)) {
    case U8_GEMV: {
      const int blocks = (n + ROWS - 1) / ROWS;
      const int steps = p / MACRO_K;
      // enough wavefronts per workgroup to keep every macro step of a small problem in flight
      if (steps >= 16 && blocks <= 1024)
        hipLaunchKernelGGL(gemv_u8_kernel<8>, dim3(blocks), dim3(512), 0, stream, out, lhs, rhs,
                           scales, m, p, n, beta);
      else
        hipLaunchKernelGGL(gemv_u8_kernel<4>, dim3(blocks), dim3(256), 0, stream, out, lhs, rhs,
                           scales, m, p, n, beta);
      return hipGetLastError();
    }
    case U8_GEMM:
      return launch_gemm_u8_mfma(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
    default: {
      if ((m + 3) / 4 > 65535) return hipErrorInvalidConfiguration;
      hipLaunchKernelGGL(gemm_u8_naive_kernel, dim3((n + 63) / 64, (m + 3) / 4), dim3(256), 0,
                         stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      return hipGetLastError();
    }
  }
}

}  // namespace adr
