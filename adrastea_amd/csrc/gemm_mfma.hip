// fp16 "NT" GEMM on the CDNA4 matrix cores: O[b,y,x] = store(sum_k L[b,y,k] * R[b,k,x]) for
// operands whose K dimension is contiguous in memory on BOTH sides (stride_lx == 1 and
// stride_ry == 1) and a row-major output (stride_ox == 1).  That covers every linear layer of
// the callers (weights arrive as W[N,K].permute([1,0]), adrastea_models/src/llama.rs:503-532)
// and the attention score product Q.K^T on the interleaved-head views of llama.rs:534-550.
// Row strides (stride_ly, stride_rx, stride_oy) and batch strides are free.
//
// Structure: one workgroup per BM x BN output tile, WM x WN wavefronts, each owning a
// (BM/WM) x (BN/WN) sub-tile as 32x32 fp32 accumulators of v_mfma_f32_32x32x16_f16.  A and B
// K-slices of depth BK are staged global -> registers -> LDS with 128-bit accesses, double
// buffered in LDS so that the global loads of slice t+1 are in flight while slice t feeds the
// MFMAs; one barrier per slice.  LDS rows are XOR-swizzled at 16-byte granularity so that the
// 128-bit fragment reads of 8 consecutive rows hit 8 different bank groups.
#include "adr_common.hpp"

namespace adr {

namespace {

constexpr int XCDS = 8;  // MI355X: 8 accelerator dies, workgroup i is dispatched to die i % 8

// Physical byte offset of 16-byte chunk `kc` of row `row` in a [rows][CPR chunks] LDS tile.
template <int CPR>
__device__ __forceinline__ int lds_chunk_off(int row, int kc) {
  int idx = row * CPR + kc;
  int line = idx >> 3, pos = idx & 7;  // 8 chunks = one 128-byte line = all 32 banks
  return ((line << 3) | (pos ^ (line & 7))) << 4;
}

// Work decomposition shared by host and device.
struct TileMap {
  int tiles_m, tiles_n, tiles_per_batch, total;
  int group_m;  // tile rows per L2-reuse group
};

template <int BM, int BN, int BK, int WM, int WN, int MINB, bool LOAD_SCALE, bool WQ>
__global__ __launch_bounds__(WM* WN * 64, MINB) void gemm_nt_kernel(MatmulArgs a, TileMap map) {
  constexpr int NT = WM * WN * 64;
  constexpr int CPR = BK / 8;                // 16-byte chunks per tile row
  constexpr int LA = BM * CPR / NT;          // chunks each thread stages for A
  constexpr int LB = BN * CPR / NT;
  constexpr int WTM = BM / WM, WTN = BN / WN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int KK = BK / 16;
  static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "staging must divide evenly");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 16 == 0, "MFMA 32x32x16 tiling");

  extern __shared__ __attribute__((aligned(128))) unsigned char smem[];
  unsigned char* const sA = smem;                         // [2][BM][BK] halves
  unsigned char* const sB = smem + 2 * BM * BK * 2;       // [2][BN][BK] halves

  // ---- which tile: XCD-aware remap, then grouped (tile-row-major inside groups of group_m)
  int id = blockIdx.x;
  {
    const int per = (map.total + XCDS - 1) / XCDS;
    const int tall = map.total % XCDS == 0 ? XCDS : map.total % XCDS;
    const int xcd = id % XCDS, local = id / XCDS;
    id = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
  }
  const int batch = id / map.tiles_per_batch;
  int t = id - batch * map.tiles_per_batch;
  const int group_span = map.group_m * map.tiles_n;
  const int g = t / group_span;
  const int gm0 = g * map.group_m;
  const int gsz = min(map.group_m, map.tiles_m - gm0);
  t -= g * group_span;
  const int tile_m = gm0 + t % gsz;
  const int tile_n = t / gsz;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;

  half_t* const out = a.output + (int64_t)batch * a.stride_oz;

  // ---- fully masked tile: every x > every y (matmul.cu:182-184) -> write -inf, no math
  if (a.mask == ADR_MASK_CAUSAL && n0 > m0 + BM - 1) {
    for (int e = tid; e < BM * BN; e += NT) {
      int y = m0 + e / BN, x = n0 + e % BN;
      if (y < a.m && x < a.n) out[(int64_t)y * a.stride_oy + x] = neg_inf_half();
    }
    return;
  }

  const half_t* const A = a.lhs + (int64_t)batch * a.stride_lz;
  const half_t* const B = a.rhs + (int64_t)batch * a.stride_rz;  // fp16 right operand (!WQ)

  // ---- staging assignment: chunk c = tid + i*NT -> (row, kc); out-of-range rows are clamped
  // to the last valid row (their products are discarded at the store)
  const half_t* gA[LA];
  const half_t* gB[LB];       // fp16 right operand
  const uint8_t* gQ[LB];      // u8 right operand: 8 weights per chunk ...
  const half_t* gS[LB];       // ... and the scale row of that weight row
  int offA[LA], offB[LB], kcA[LA], kcB[LB];
#pragma unroll
  for (int i = 0; i < LA; i++) {
    int c = tid + i * NT, row = c / CPR, kc = c % CPR;
    gA[i] = A + (int64_t)min(m0 + row, a.m - 1) * a.stride_ly + kc * 8;
    offA[i] = lds_chunk_off<CPR>(row, kc);
    kcA[i] = kc * 8;
  }
#pragma unroll
  for (int i = 0; i < LB; i++) {
    int c = tid + i * NT, row = c / CPR, kc = c % CPR;
    const int brow = min(n0 + row, a.n - 1);
    if (WQ) {
      gQ[i] = a.rhs_q + (int64_t)brow * a.k + kc * 8;
      gS[i] = a.scales + (int64_t)brow * (a.k / a.block_size);
    } else {
      gB[i] = B + (int64_t)brow * a.stride_rx + kc * 8;
    }
    offB[i] = lds_chunk_off<CPR>(row, kc);
    kcB[i] = kc * 8;
  }

  u32x4_t ra[LA], rb[LB];
  u32x2_t rq[LB];
  half_t rs[LB];
  const int K = a.k;
  const int KT = (K + BK - 1) / BK;
  const half_t hscale = (half_t)a.scale;

  auto load_slice = [&](int kt) {
    const int k0 = kt * BK;
    const bool full = k0 + BK <= K;
#pragma unroll
    for (int i = 0; i < LA; i++) {
      if (full || k0 + kcA[i] < K)
        ra[i] = *(const u32x4_t*)(gA[i] + k0);
      else
        ra[i] = u32x4_t{0, 0, 0, 0};
    }
#pragma unroll
    for (int i = 0; i < LB; i++) {
      if (WQ) {
        // a chunk of 8 weights never straddles a scale block (block_size % 8 == 0); chunks
        // beyond K get scale 0 with mid-range weights, i.e. exact zeros
        const bool in = full || k0 + kcB[i] < K;
        rq[i] = in ? *(const u32x2_t*)(gQ[i] + k0) : u32x2_t{0, 0};
        rs[i] = in ? gS[i][(k0 + kcB[i]) / a.block_size] : (half_t)0;
      } else if (full || k0 + kcB[i] < K) {
        rb[i] = *(const u32x4_t*)(gB[i] + k0);
      } else {
        rb[i] = u32x4_t{0, 0, 0, 0};
      }
    }
  };
  auto store_slice = [&](int buf) {
    unsigned char* dA = sA + buf * (BM * BK * 2);
    unsigned char* dB = sB + buf * (BN * BK * 2);
#pragma unroll
    for (int i = 0; i < LA; i++) {
      if (LOAD_SCALE) {  // operands are scaled in fp16 before the product (matmul.cu:439-443)
        half8_t v = __builtin_bit_cast(half8_t, ra[i]);
        v = v * hscale;
        ra[i] = __builtin_bit_cast(u32x4_t, v);
      }
      *(u32x4_t*)(dA + offA[i]) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < LB; i++) {
      if (WQ) {  // dequantisation fused into the staging of the weight tile
        const half2_t s2 = {rs[i], rs[i]};
        rb[i] = __builtin_bit_cast(u32x4_t, dequant8(rq[i][0], rq[i][1], s2));
      }
      if (LOAD_SCALE) {
        half8_t v = __builtin_bit_cast(half8_t, rb[i]);
        v = v * hscale;
        rb[i] = __builtin_bit_cast(u32x4_t, v);
      }
      *(u32x4_t*)(dB + offB[i]) = rb[i];
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  // fragment addressing: lane -> (row = lane % 32, k-group = lane / 32)
  const int frow = lane & 31, fkg = lane >> 5;

  load_slice(0);
  store_slice(0);
  __syncthreads();

  for (int kt = 0; kt < KT; kt++) {
    const int buf = kt & 1;
    if (kt + 1 < KT) load_slice(kt + 1);
    const unsigned char* cA = sA + buf * (BM * BK * 2);
    const unsigned char* cB = sB + buf * (BN * BK * 2);
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      half8_t fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        fa[i] = *(const half8_t*)(cA + lds_chunk_off<CPR>(wm * WTM + i * 32 + frow, kk * 2 + fkg));
#pragma unroll
      for (int j = 0; j < TN; j++)
        fb[j] = *(const half8_t*)(cB + lds_chunk_off<CPR>(wn * WTN + j * 32 + frow, kk * 2 + fkg));
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) store_slice(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue: accumulator element r of a 32x32 tile is row 8*(r/4) + 4*(lane/32) + r%4,
  // column lane % 32
  Epilogue ep{a.bias, a.beta, hscale, a.store};
  const bool need_prev = Epilogue::needs_prev(a.store);
  const bool need_bias = Epilogue::needs_bias(a.store);
  const bool causal = a.mask == ADR_MASK_CAUSAL;
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int x = n0 + wn * WTN + j * 32 + frow;
    if (x >= a.n) continue;
    const half_t bias_x = need_bias ? a.bias[x] : (half_t)0;
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int ybase = m0 + wm * WTM + i * 32 + 4 * fkg;
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const int y = ybase + 8 * (r / 4) + (r % 4);
        if (y >= a.m) continue;
        half_t* p = out + (int64_t)y * a.stride_oy + x;
        if (causal && x > y) {
          *p = neg_inf_half();
        } else {
          half_t prev = need_prev ? *p : (half_t)0;
          *p = ep.apply(acc[i][j][r], prev, bias_x);
        }
      }
    }
  }
}

struct GemmShape {
  int bm, bn, bk, threads, lds;
  const char* name;
};

template <int BM, int BN, int BK, int WM, int WN, int MINB>
hipError_t launch_cfg(hipStream_t stream, const MatmulArgs& a) {
  TileMap map;
  map.tiles_m = (a.m + BM - 1) / BM;
  map.tiles_n = (a.n + BN - 1) / BN;
  map.tiles_per_batch = map.tiles_m * map.tiles_n;
  const int64_t total = (int64_t)map.tiles_per_batch * a.batches;
  if (total > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  map.total = (int)total;
  map.group_m = map.tiles_m < 8 ? map.tiles_m : 8;
  constexpr int LDS = 2 * (BM + BN) * BK * 2;
  dim3 grid((unsigned)map.total, 1, 1), block(WM * WN * 64, 1, 1);
  static_assert(LDS <= 64 * 1024, "larger tiles need hipFuncSetAttribute per device");
  if (a.rhs_q)
    hipLaunchKernelGGL((gemm_nt_kernel<BM, BN, BK, WM, WN, MINB, false, true>), grid, block, LDS,
                       stream, a, map);
  else if (a.load == ADR_LOAD_SCALE)
    hipLaunchKernelGGL((gemm_nt_kernel<BM, BN, BK, WM, WN, MINB, true, false>), grid, block, LDS,
                       stream, a, map);
  else
    hipLaunchKernelGGL((gemm_nt_kernel<BM, BN, BK, WM, WN, MINB, false, false>), grid, block, LDS,
                       stream, a, map);
  return hipGetLastError();
}

enum GemmChoice { GEMM_NONE = 0, GEMM_256x128, GEMM_128x128, GEMM_64x64 };

// The MFMA family needs 16-byte aligned, K-contiguous rows on both operands.
GemmChoice choose(const MatmulArgs& a) {
  if (a.stride_lx != 1 || a.stride_ry != 1 || a.stride_ox != 1) return GEMM_NONE;
  if (a.k % 8 != 0 || a.k < 8) return GEMM_NONE;
  if ((a.stride_ly % 8) | (a.stride_rx % 8) | (a.stride_lz % 8) | (a.stride_rz % 8)) return GEMM_NONE;
  if (a.lhs && ((uintptr_t)a.lhs % 16 != 0 || (uintptr_t)a.rhs % 16 != 0 ||
                (uintptr_t)a.rhs_q % 8 != 0)) return GEMM_NONE;
  const int64_t t256 = (int64_t)((a.m + 255) / 256) * ((a.n + 127) / 128) * a.batches;
  const int64_t t128 = (int64_t)((a.m + 127) / 128) * ((a.n + 127) / 128) * a.batches;
  if (t256 >= 200) return GEMM_256x128;
  if (t128 >= 128) return GEMM_128x128;
  return GEMM_64x64;
}

}  // namespace

bool mfma_gemm_supported(const MatmulArgs& a, const char** name) {
  switch (choose(a)) {
    case GEMM_256x128: *name = "gemm_nt_mfma_256x128x32"; return true;
    case GEMM_128x128: *name = "gemm_nt_mfma_128x128x32"; return true;
    case GEMM_64x64: *name = "gemm_nt_mfma_64x64x64"; return true;
    default: return false;
  }
}

hipError_t launch_mfma_gemm(hipStream_t stream, const MatmulArgs& a) {
  switch (choose(a)) {
    case GEMM_256x128: return launch_cfg<256, 128, 32, 2, 2, 2>(stream, a);
    case GEMM_128x128: return launch_cfg<128, 128, 32, 2, 2, 2>(stream, a);
    case GEMM_64x64: return launch_cfg<64, 64, 64, 2, 2, 2>(stream, a);
    default: return hipErrorInvalidValue;
  }
}

hipError_t launch_gemm_u8_mfma(hipStream_t stream, half_t* out, const half_t* lhs,
                               const uint8_t* rhs, const half_t* scales, int m, int p, int n,
                               int block_size, float beta) {
  MatmulArgs a{};
  a.output = out;
  a.lhs = lhs;
  a.rhs = nullptr;
  a.batches = 1;
  a.m = m; a.k = p; a.n = n;
  a.stride_ox = 1; a.stride_oy = n;
  a.stride_lx = 1; a.stride_ly = p;
  a.stride_rx = p; a.stride_ry = 1;
  a.beta = beta;
  a.scale = 1.0f;
  a.store = STORE_ACC_BETA;
  a.rhs_q = rhs;
  a.scales = scales;
  a.block_size = block_size;
  return launch_mfma_gemm(stream, a);
}

}  // namespace adr
