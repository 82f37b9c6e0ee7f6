// gfx950 code object "matmul" for an UNMODIFIED host: the three device symbols the reference's
// Rust side looks up in its matmul module -- matmul_f16, matmul_f16_fast, matmul_f16_raw
// (adrastea_kernels/cpp/matmul.cu:493-517; bound at adrastea_models/src/kernels.rs:472-473) --
// with the same kernel-argument layout, written for the launch geometry that host code bakes in:
//   matmul_f16       grid (ceil(N/16), ceil(M/16), B) x block (16, 16, 1)      kernels.rs:783-792
//   matmul_f16_fast  grid (ceil(N/32), ceil(M/16), B) x block (32, 4, 1),
//                    3264 bytes of dynamic LDS (unused here)                    kernels.rs:849-863
// Built with `hipcc --genco`; the library's own entry points choose their geometry themselves
// and are the fast way in -- two wavefronts per 16 x 32 tile cannot feed the matrix cores well.
//
// matmul_f16_fast: the two wavefronts of a block each own a 16 x 16 half of the tile and run
// v_mfma_f32_16x16x32_f16 on fragments loaded straight from global memory (16 bytes per lane)
// when both operands are K-contiguous and 16-byte aligned -- the layout of every weight product
// (W[N,K].permute) and of QK^T on the head views; any other layout takes the per-output path,
// four outputs per thread.
#include "adr_common.hpp"

using namespace adr;

#define LEGACY_PARAMS                                                                            \
  half_t *output, const half_t *lhs, const half_t *rhs, int batches, int m, int k, int n,        \
      int stride_ox, int stride_oy, int stride_oz, int stride_lx, int stride_ly, int stride_lz,  \
      int stride_rx, int stride_ry, int stride_rz
#define LEGACY_OPS const half_t *bias, float beta, float scale, uint32_t store, uint32_t load, uint32_t mask

namespace {

__device__ __forceinline__ MatmulArgs pack(LEGACY_PARAMS, LEGACY_OPS) {
  MatmulArgs a;
  a.output = output; a.lhs = lhs; a.rhs = rhs;
  a.batches = batches; a.m = m; a.k = k; a.n = n;
  a.stride_ox = stride_ox; a.stride_oy = stride_oy; a.stride_oz = stride_oz;
  a.stride_lx = stride_lx; a.stride_ly = stride_ly; a.stride_lz = stride_lz;
  a.stride_rx = stride_rx; a.stride_ry = stride_ry; a.stride_rz = stride_rz;
  a.bias = bias; a.beta = beta; a.scale = scale;
  a.store = store; a.load = load; a.mask = mask;
  a.rhs_q = nullptr; a.scales = nullptr; a.block_size = 0;
  return a;
}

// one thread per output, whatever block shape the host launched
__device__ __forceinline__ void per_thread(const MatmulArgs& a) {
  const int x = blockIdx.x * blockDim.x + threadIdx.x;
  const int y = blockIdx.y * blockDim.y + threadIdx.y;
  if (x < a.n && y < a.m && (int)blockIdx.z < a.batches) matmul_one_output(a, blockIdx.z, y, x);
}

__device__ __forceinline__ bool k_contiguous_aligned(const MatmulArgs& a) {
  return a.stride_lx == 1 && a.stride_ry == 1 && a.k % 8 == 0 &&
         !((a.stride_ly | a.stride_lz | a.stride_rx | a.stride_rz) & 7) &&
         !(((uintptr_t)a.lhs | (uintptr_t)a.rhs) & 15);
}

}  // namespace

extern "C" __global__ void matmul_f16(LEGACY_PARAMS, LEGACY_OPS) {
  const MatmulArgs a = pack(output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                            stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, bias,
                            beta, scale, store, load, mask);
  per_thread(a);
}

// matmul.cu:515-517: the identity-operator form, 16 arguments
extern "C" __global__ void matmul_f16_raw(LEGACY_PARAMS) {
  const MatmulArgs a = pack(output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                            stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz,
                            nullptr, 0.0f, 1.0f, ADR_STORE_IDENTITY, ADR_LOAD_IDENTITY,
                            ADR_MASK_NONE);
  per_thread(a);
}

extern "C" __global__ void matmul_f16_fast(LEGACY_PARAMS, LEGACY_OPS) {
  const MatmulArgs a = pack(output, lhs, rhs, batches, m, k, n, stride_ox, stride_oy, stride_oz,
                            stride_lx, stride_ly, stride_lz, stride_rx, stride_ry, stride_rz, bias,
                            beta, scale, store, load, mask);
  constexpr int TILE_M = 16, TILE_N = 32;
  const int b = blockIdx.z;
  const int m0 = blockIdx.y * TILE_M, n0 = blockIdx.x * TILE_N;
  const int tid = threadIdx.x + threadIdx.y * blockDim.x;
  const bool geometry = blockDim.x * blockDim.y == 128 && blockDim.z == 1;
  if (!geometry || !k_contiguous_aligned(a)) {
    // per-output path over the block's tile, whatever the block shape
    const int nthreads = blockDim.x * blockDim.y * blockDim.z;
    const int t = tid + threadIdx.z * blockDim.x * blockDim.y;
    for (int e = t; e < TILE_M * TILE_N; e += nthreads) {
      const int y = m0 + e / TILE_N, x = n0 + e % TILE_N;
      if (y < a.m && x < a.n) matmul_one_output(a, b, y, x);
    }
    return;
  }
  // lane (r, g): fragment row / column r, k-group g (8 consecutive k of every 32)
  const int wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
  const int nw = n0 + wave * 16;  // this wavefront's 16 columns
  if (nw >= a.n) return;
  if (a.mask == ADR_MASK_CAUSAL && nw > m0 + TILE_M - 1) {
    // entirely above the diagonal (matmul.cu:210-213): -inf, no arithmetic
#pragma unroll
    for (int v = 0; v < 4; v++) {
      const int y = m0 + 4 * g + v, x = nw + r;
      if (y < a.m && x < a.n)
        a.output[(int64_t)b * a.stride_oz + (int64_t)y * a.stride_oy + (int64_t)x * a.stride_ox] =
            neg_inf_half();
    }
    return;
  }
  // rows / columns past the edge read the last one; their results are not stored
  const half_t* lp = a.lhs + (int64_t)b * a.stride_lz + (int64_t)min(m0 + r, a.m - 1) * a.stride_ly + g * 8;
  const half_t* rp = a.rhs + (int64_t)b * a.stride_rz + (int64_t)min(nw + r, a.n - 1) * a.stride_rx + g * 8;
  const half_t hscale = (half_t)a.scale;
  const bool load_scale = a.load == ADR_LOAD_SCALE;
  const half8_t zero = {0, 0, 0, 0, 0, 0, 0, 0};
  float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
  for (int k0 = 0; k0 < a.k; k0 += 32) {
    // K % 8 == 0: a group of eight lies inside the matrix or is zero
    const bool in = k0 + g * 8 < a.k;
    half8_t fa = in ? *(const half8_t*)(lp + k0) : zero;
    half8_t fb = in ? *(const half8_t*)(rp + k0) : zero;
    if (load_scale) {  // both operands times fp16(scale) in fp16 (matmul.cu:439-443)
      fa = fa * hscale;
      fb = fb * hscale;
    }
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(fa, fb, acc, 0, 0, 0);
  }
  // the lane holds rows 4g .. 4g+3 of column r
  Epilogue ep{a.bias, a.beta, hscale, a.store};
  const int x = nw + r;
  if (x >= a.n) return;
  const half_t bias_x = Epilogue::needs_bias(a.store) ? a.bias[x] : (half_t)0;
#pragma unroll
  for (int v = 0; v < 4; v++) {
    const int y = m0 + 4 * g + v;
    if (y >= a.m) continue;
    half_t* o = a.output + (int64_t)b * a.stride_oz + (int64_t)y * a.stride_oy + (int64_t)x * a.stride_ox;
    if (a.mask == ADR_MASK_CAUSAL && x > y) {
      *o = neg_inf_half();
    } else {
      const half_t prev = Epilogue::needs_prev(a.store) ? *o : (half_t)0;
      *o = ep.apply(acc[v], prev, bias_x);
    }
  }
}
