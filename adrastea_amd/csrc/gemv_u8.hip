// u8-quantised-weight skinny GEMM / GEMV for decode (m <= 16):
//   out[r,c] = fp16( sum_i lhs[r,i] * w[c,i] + beta * out[r,c] ),
//   w[c,i]   = (float(q[c,i]) - 127.5f) * float(scales[c, i/block_size])
// (adrastea_kernels/cpp/matmul_nt_fp16u8.cu:4-24 and
// matmul_nt_wmma_16x128x256_fp16u8.cu:5-7, 43-83; format quantize.cu:3-56).
//
// The problem is bound by streaming the u8 weights from HBM once.  Two kernels:
//
//  gemv_u8_dot_kernel (m <= 2)   no matrix cores.  A wavefront streams whole 1 KiB segments of
//      one weight row per load instruction (lane l: 16 bytes at l*16, perfectly coalesced),
//      keeps its activation slices in registers for all rows of the workgroup, and evaluates
//        sum_k x_k (q_k - 127.5) s  =  s * ( sum_k x_k (1024 + q_k)  -  1151.5 * sum_k x_k )
//      per lane (16 weights of one scale block): the bytes are unpacked with one v_perm_b32
//      per pair into the fp16 numbers 1024 + q (bit pattern 0x6400 | q) and fed to
//      v_dot2_f32_f16 with fp32 accumulation; the second term is row independent and computed
//      once.  This is the arithmetic of the reference's naive kernel (unrounded weights,
//      matmul_nt_fp16u8.cu:17-21) in fp32.  Lane sums are reduced with DPP adds.
//
//  gemv_u8_kernel (m <= 16)      v_mfma_f32_16x16x32_f16 with the 16 weight rows of the
//      workgroup as the A operand and the activations as the B operand (rows beyond m are
//      zero).  Per 256-element macro step a lane (row r = lane % 16, group g = lane / 16)
//      loads 4 x 16 weight bytes such that the four lanes of a row cover 64 contiguous bytes
//      per instruction, dequantises them in registers to fp16 exactly as the stand-alone
//      dequantise kernel does (the WMMA kernel's arithmetic) and issues two MFMAs per load.
//      The k slots of an MFMA may hold any 32 distinct k as long as both operands agree,
//      which is what lets a lane use 16 contiguous bytes.  Wavefronts split K; partial sums
//      are reduced through LDS.
#include "adr_common.hpp"

namespace adr {

namespace {

constexpr int MACRO_K = 256;  // k elements per macro step
constexpr int ROWS = 16;      // weight rows per workgroup

struct Stage {
  u32x4_t w[4];   // 4 x 16 weight bytes of this lane's row
  u32x4_t sc;     // the eight fp16 scales (block_size 32) of the macro step
  u32x4_t x[8];   // 4 x 16 activation halves of this lane's activation row
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
  // load j of a macro step takes bytes j*64 + g*16 .. +16 of the row: the four lanes of a row
  // cover 64 contiguous bytes per instruction
  const uint8_t* wrow = rhs + (int64_t)row * p + g * 16;
  const half_t* srow = scales + (int64_t)row * nblk;
  const bool xvalid = r < m;
  const half_t* xrow = lhs + (int64_t)min(r, m - 1) * p + g * 16;
  const int steps = p / MACRO_K;

  auto load = [&](Stage& s, int ms) {
    const uint8_t* wp = wrow + (int64_t)ms * MACRO_K;
#pragma unroll
    for (int j = 0; j < 4; j++) s.w[j] = *(const u32x4_t*)(wp + j * 64);
    s.sc = *(const u32x4_t*)(srow + ms * (MACRO_K / 32));
    const half_t* xp = xrow + (int64_t)ms * MACRO_K;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      // (lanes beyond m load row m-1 again -- same addresses as its own lanes, no extra
      // traffic -- and are zeroed: a load under a branch would be waited for at the join)
      const u32x4_t x0 = *(const u32x4_t*)(xp + j * 64), x1 = *(const u32x4_t*)(xp + j * 64 + 8);
      s.x[2 * j] = xvalid ? x0 : u32x4_t{0, 0, 0, 0};
      s.x[2 * j + 1] = xvalid ? x1 : u32x4_t{0, 0, 0, 0};
    }
  };

  float4_t acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
  auto compute = [&](const Stage& s) {
    const half8_t sc = __builtin_bit_cast(half8_t, s.sc);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      // the lane's 16 weights of load j sit in scale block 2j (g < 2) or 2j + 1
      const half_t sv = g < 2 ? sc[2 * j] : sc[2 * j + 1];
      const half2_t s2 = {sv, sv};
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


// Variant for wide matrices: a workgroup covers RG groups of 16 weight rows, and a wavefront keeps
// the activation fragments of its macro step in registers while it walks the RG groups, so the
// activations are fetched once per 16*RG weight rows instead of once per 16.
struct WStage {
  u32x4_t w[4];  // 4 x 16 weight bytes of this lane's row
  u32x4_t sc;    // the eight fp16 scales (block_size 32) of the macro step
};

template <int NW, int RG>
__global__ __launch_bounds__(NW * 64) void gemv_u8_wide_kernel(half_t* __restrict__ out,
                                                               const half_t* __restrict__ lhs,
                                                               const uint8_t* __restrict__ rhs,
                                                               const half_t* __restrict__ scales,
                                                               int m, int p, int n, float beta) {
  __shared__ float partial[NW][RG][ROWS * 16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (ROWS * RG);
  const int nblk = p / 32;
  const bool xvalid = r < m;
  const half_t* xrow = lhs + (int64_t)min(r, m - 1) * p + g * 16;
  const int steps = p / MACRO_K;
  const uint8_t* wrow[RG];
  const half_t* srow[RG];
#pragma unroll
  for (int q = 0; q < RG; q++) {
    const int row = min(n0 + q * ROWS + r, n - 1);  // tail rows are clamped, never stored
    wrow[q] = rhs + (int64_t)row * p + g * 16;
    srow[q] = scales + (int64_t)row * nblk;
  }
  auto load_w = [&](WStage& s, int q, int ms) {
    const uint8_t* wp = wrow[q] + (int64_t)ms * MACRO_K;
#pragma unroll
    for (int j = 0; j < 4; j++) s.w[j] = *(const u32x4_t*)(wp + j * 64);
    s.sc = *(const u32x4_t*)(srow[q] + ms * (MACRO_K / 32));
  };
  auto load_x = [&](u32x4_t (&x)[8], int ms) {
    const half_t* xp = xrow + (int64_t)ms * MACRO_K;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      // (under the lane mask on purpose: measured faster here than unconditional loads of a
      // clamped row, which is what the 16-row kernel does)
      x[2 * j] = xvalid ? *(const u32x4_t*)(xp + j * 64) : u32x4_t{0, 0, 0, 0};
      x[2 * j + 1] = xvalid ? *(const u32x4_t*)(xp + j * 64 + 8) : u32x4_t{0, 0, 0, 0};
    }
  };
  float4_t acc[RG][2];
#pragma unroll
  for (int q = 0; q < RG; q++) acc[q][0] = acc[q][1] = float4_t{0, 0, 0, 0};
  auto compute = [&](const WStage& s, const u32x4_t (&x)[8], float4_t (&a)[2]) {
    const half8_t sc = __builtin_bit_cast(half8_t, s.sc);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const half_t sv = g < 2 ? sc[2 * j] : sc[2 * j + 1];
      const half2_t s2 = {sv, sv};
      half8_t a0 = dequant8(s.w[j][0], s.w[j][1], s2);
      half8_t a1 = dequant8(s.w[j][2], s.w[j][3], s2);
      a[0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, __builtin_bit_cast(half8_t, x[2 * j]), a[0], 0, 0, 0);
      a[1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, __builtin_bit_cast(half8_t, x[2 * j + 1]), a[1], 0, 0, 0);
    }
  };

  // all weight loads of a macro step are issued before its first use
  for (int ms = wave; ms < steps; ms += NW) {
    u32x4_t x[8];
    WStage s[RG];
    load_x(x, ms);
#pragma unroll
    for (int q = 0; q < RG; q++) load_w(s[q], q, ms);
#pragma unroll
    for (int q = 0; q < RG; q++) compute(s[q], x, acc[q]);
  }

#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int i = 0; i < 4; i++) partial[wave][q][(4 * g + i) * 16 + r] = acc[q][0][i] + acc[q][1][i];
  __syncthreads();
  for (int e = tid; e < RG * ROWS * 16; e += NW * 64) {
    const int mm = e / (RG * ROWS), nn = e % (RG * ROWS);  // consecutive threads -> consecutive columns
    if (mm < m && n0 + nn < n) {
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < NW; w++) sum += partial[w][nn / ROWS][(nn % ROWS) * 16 + mm];
      half_t* o = out + (int64_t)mm * n + n0 + nn;
      // the previous output is read even for beta == 0, as the reference does
      *o = (half_t)(sum + beta * (float)*o);
    }
  }
}

// K = 4096: weights and activations come in by global -> LDS DMA, four whole 256-byte row
// pieces per instruction (the register path touches sixteen rows with 64 bytes each per
// instruction, which moves the same bytes about a quarter slower).  A wavefront owns two macro
// steps x (2 activation tiles + RG weight row groups) tiles of 4 KiB ([16 rows][16 chunks of 16
// bytes], chunk c of row r at position c ^ r so that fragment reads spread over all banks) and
// streams them through a private ring of RING tiles: nothing but its own vmcnt orders the DMA
// against its reads.  The scales are loaded into registers before the first DMA, so the count of
// outstanding loads at any later point is a multiple of the four DMA instructions of a tile.
// (With the activations of both macro steps in registers, loaded in MFMA layout as 64-byte
// pieces: m=16 N4096 8.4 us against 7.1, N11008 15.2 against 13.9, N12288 15.9 against 14.7.)
#define ADR_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define ADR_GLB_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

template <int NW, int RG, int RING, int MB>
__global__ __launch_bounds__(NW * 64) void gemv_u8_ring_kernel(half_t* __restrict__ out,
                                                               const half_t* __restrict__ lhs,
                                                               const uint8_t* __restrict__ rhs,
                                                               const half_t* __restrict__ scales,
                                                               int m, int p, int n, float beta) {
  constexpr int TILE = ROWS * MACRO_K;  // 4096 bytes
  // a macro step: two tiles of activations per block of sixteen rows ([16 rows][128 halves]: k
  // 0..127 and 128..255 of the step), then its RG weight tiles
  constexpr int PER = RG + 2 * MB;
  constexpr int UNITS = 2 * PER;        // tiles per wavefront: macro steps wave, wave + NW
  static_assert(RING <= UNITS && NW * MB * RG * 256 * 4 <= NW * RING * TILE, "partials reuse the ring");
  __shared__ __attribute__((aligned(1024))) unsigned char ring[NW * RING * TILE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (ROWS * RG);
  const int nblk = p / 32;
  bool xvalid[MB];
#pragma unroll
  for (int b = 0; b < MB; b++) xvalid[b] = b * 16 + r < m;
  unsigned char* const mine = ring + wave * RING * TILE;

  // registers first: the scales of all tiles
  u32x4_t x[MB][8], sc[2][RG];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int ms = wave + h * NW;
#pragma unroll
    for (int q = 0; q < RG; q++)
      sc[h][q] = *(const u32x4_t*)(scales + (int64_t)min(n0 + q * ROWS + r, n - 1) * nblk +
                                   ms * (MACRO_K / 32));
  }
  // DMA instruction i of a tile fills its chunks [64 i, 64 i + 64): rows 4i .. 4i+3
  auto issue = [&](int u) {  // tile u: macro step half u / PER; q < 0: activation tile q + 2 MB
                             // (block (q + 2 MB) / 2, k half (q + 2 MB) % 2)
    const int h = u / PER, q = u % PER - 2 * MB;
    const int xb = q < 0 ? (q + 2 * MB) / 2 : 0, xh = q < 0 ? (q + 2 * MB) % 2 : 0;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = 4 * i + (lane >> 4), kc = (lane & 15) ^ row;
      // (rows beyond m read row m - 1 again and are zeroed when used)
      const void* src =
          q < 0 ? (const void*)(lhs + (int64_t)min(xb * 16 + row, m - 1) * p +
                                (int64_t)(wave + h * NW) * MACRO_K + xh * 128 + kc * 8)
                : (const void*)(rhs + (int64_t)min(n0 + q * ROWS + row, n - 1) * p +
                                (int64_t)(wave + h * NW) * MACRO_K + kc * 16);
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(src),
                                       ADR_LDS_PTR(mine + (u % RING) * TILE + i * 1024), 16, 0, 0);
    }
  };
  int roff[4];  // fragment read j of the lane: logical chunk 4j + g of row r
#pragma unroll
  for (int j = 0; j < 4; j++) roff[j] = r * 256 + (((4 * j + g) ^ r) << 4);
  int xoff[4];  // activation fragment 2 jj + e of a tile: logical chunk 8 jj + 2 g + e of row r
#pragma unroll
  for (int f = 0; f < 4; f++) xoff[f] = r * 256 + (((8 * (f >> 1) + 2 * g + (f & 1)) ^ r) << 4);

  float4_t acc[MB][RG][2];
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int q = 0; q < RG; q++) acc[b][q][0] = acc[b][q][1] = float4_t{0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < RING; u++) issue(u);
#pragma unroll
  for (int u = 0; u < UNITS; u++) {
    // tiles u+1 .. min(u+RING-1, UNITS-1) may still be in flight: four DMA instructions each
    constexpr int Z = 0;
    const int later = (u + RING - 1 < UNITS ? RING - 1 : UNITS - 1 - u) * 4 + Z;
    if (later == 8) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    else if (later == 4) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
    else if (later == 12) __builtin_amdgcn_s_waitcnt(0x0F70 | 12);
    else __builtin_amdgcn_s_waitcnt(0x0F70 | 0);
    const int h = u / PER, q = u % PER - 2 * MB;
    const unsigned char* tile = mine + (u % RING) * TILE;
    const half8_t s8 = __builtin_bit_cast(half8_t, sc[h][q < 0 ? 0 : q]);
    const u32x4_t z = {0, 0, 0, 0};
    u32x4_t w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) w[j] = *(const u32x4_t*)(tile + (q < 0 ? xoff[j] : roff[j]));
    // the tile is in registers before its slot is refilled
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    if (u + RING < UNITS) issue(u + RING);
    __builtin_amdgcn_sched_barrier(0);
    if (q < 0) {  // activations of one block of rows, one half of the step's k
      const int t = q < 0 ? q + 2 * MB : 0;
#pragma unroll
      for (int f = 0; f < 4; f++) x[t / 2][(t % 2) * 4 + f] = w[f];
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const half_t sv = g < 2 ? s8[2 * j] : s8[2 * j + 1];
      const half2_t s2 = {sv, sv};
      const half8_t a0 = dequant8(w[j][0], w[j][1], s2), a1 = dequant8(w[j][2], w[j][3], s2);
#pragma unroll
      for (int b = 0; b < MB; b++) {
        const half8_t b0 = __builtin_bit_cast(half8_t, xvalid[b] ? x[b][2 * j] : z);
        const half8_t b1 = __builtin_bit_cast(half8_t, xvalid[b] ? x[b][2 * j + 1] : z);
        acc[b][q][0] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, acc[b][q][0], 0, 0, 0);
        acc[b][q][1] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, acc[b][q][1], 0, 0, 0);
      }
    }
  }

  // the ring is dead: its memory takes the per-wavefront partial sums [NW][MB][RG][256]
  __syncthreads();
  float* partial = (float*)ring;
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int q = 0; q < RG; q++)
#pragma unroll
      for (int i = 0; i < 4; i++)
        partial[((wave * MB + b) * RG + q) * 256 + (4 * g + i) * 16 + r] =
            acc[b][q][0][i] + acc[b][q][1][i];
  __syncthreads();
  for (int e = tid; e < MB * RG * ROWS * 16; e += NW * 64) {
    const int mm = e / (RG * ROWS), nn = e % (RG * ROWS);  // consecutive threads -> consecutive columns
    if (mm < m && n0 + nn < n) {
      float sum = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < NW; w2++)
        sum += partial[((w2 * MB + mm / 16) * RG + nn / ROWS) * 256 + (nn % ROWS) * 16 + mm % 16];
      half_t* o = out + (int64_t)mm * n + n0 + nn;
      // the previous output is read even for beta == 0, as the reference does
      *o = (half_t)(sum + beta * (float)*o);
    }
  }
}

// Other K (multiples of 256), sixteen weight rows per workgroup: the same private ring, walked
// ROUNDS times.  Wavefront w owns macro steps w, w + NW, ...; every ring slot holds one macro step:
// its 4 KiB weight tile in LDS and its activations and scales in registers.  A slot is refilled
// right after it has been multiplied, and every refill issues the same 13 memory instructions
// whether or not the wavefront has a macro step left (the surplus ones read one 16-byte line and
// are multiplied with zero scales), so the wait before a slot's use is "all but the 13 (RING - 1)
// youngest" and no load sits under a branch.
// XR: the slot's activations come through LDS too, as two more tiles of the slot ([16 rows][128
// halves] each, same chunk swizzle) by eight DMA instructions in place of the eight loads, so
// the count per slot stays thirteen; a slot is then 12 KiB, which fits with four wavefronts.
template <int NW, int RING, int ROUNDS, bool XR>
__global__ __launch_bounds__(NW * 64) void gemv_u8_ring_loop_kernel(half_t* __restrict__ out,
                                                                    const half_t* __restrict__ lhs,
                                                                    const uint8_t* __restrict__ rhs,
                                                                    const half_t* __restrict__ scales,
                                                                    int m, int p, int n, float beta) {
  constexpr int TILE = ROWS * MACRO_K;
  constexpr int SLOT = XR ? 3 * TILE : TILE;  // weight tile, then the two activation tiles
  constexpr int PER = 8 + 1 + 4;  // activation loads, scale load, DMA instructions per slot
  static_assert(NW * RING * SLOT <= 160 * 1024 && NW * 256 * 4 <= NW * RING * SLOT, "LDS");
  __shared__ __attribute__((aligned(1024))) unsigned char ring[NW * RING * SLOT];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * ROWS;
  const int nblk = p / 32;
  const bool xvalid = r < m;
  const int steps = p / MACRO_K;
  const half_t* xrow = lhs + (int64_t)min(r, m - 1) * p + g * 16;
  const half_t* srow = scales + (int64_t)min(n0 + r, n - 1) * nblk;
  unsigned char* const mine = ring + wave * RING * SLOT;
  // DMA instruction i of a tile fills its chunks [64 i, 64 i + 64): rows 4i .. 4i+3
  const uint8_t* wsrc[4];
  const half_t* xsrc[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int row = 4 * i + (lane >> 4), kc = (lane & 15) ^ row;
    wsrc[i] = rhs + (int64_t)min(n0 + row, n - 1) * p + kc * 16;
    xsrc[i] = lhs + (int64_t)min(row, m - 1) * p + kc * 8;
  }
  int roff[4];  // fragment read j of the lane: logical chunk 4j + g of row r
#pragma unroll
  for (int j = 0; j < 4; j++) roff[j] = r * 256 + (((4 * j + g) ^ r) << 4);
  int xoff[4];  // activation fragment 2 jj + e of a tile: logical chunk 8 jj + 2 g + e of row r
#pragma unroll
  for (int f = 0; f < 4; f++) xoff[f] = r * 256 + (((8 * (f >> 1) + 2 * g + (f & 1)) ^ r) << 4);

  u32x4_t x[XR ? 1 : RING][8];
  u32x4_t sc[RING];
  auto issue = [&](int slot, int ms) {
    const bool live = ms < steps;  // wave-uniform
    const int64_t koff = live ? (int64_t)ms * MACRO_K : 0;
    const half_t* xp = xrow + koff;
    if constexpr (XR) {
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int i = 0; i < 4; i++) {
          // (rows beyond m read row m - 1 again and are zeroed when used)
          const half_t* src = live ? xsrc[i] + koff + t * 128 : lhs;
          __builtin_amdgcn_global_load_lds(
              ADR_GLB_PTR(src), ADR_LDS_PTR(mine + slot * SLOT + (1 + t) * TILE + i * 1024), 16, 0, 0);
        }
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        // lanes beyond m read row m-1 again (the same addresses as its own lanes) and are zeroed
        // when used: a load under a lane mask would be waited for where the lanes rejoin
        x[slot][2 * j] = *(const u32x4_t*)(xp + j * 64);
        x[slot][2 * j + 1] = *(const u32x4_t*)(xp + j * 64 + 8);
      }
    }
    sc[slot] = *(const u32x4_t*)(srow + (live ? ms * (MACRO_K / 32) : 0));
#pragma unroll
    for (int i = 0; i < 4; i++) {
      // a surplus slot fetches one 16-byte line (all lanes the same address)
      const uint8_t* src = live ? wsrc[i] + koff : rhs;
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(src),
                                       ADR_LDS_PTR(mine + slot * SLOT + i * 1024), 16, 0, 0);
    }
  };
  float4_t acc0 = {0, 0, 0, 0}, acc1 = {0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < RING; i++) issue(i, wave + i * NW);
  // ROUNDS = ceil(ceil(steps / NW) / RING), the same for every wavefront; unrolled, because the
  // compiler drains all loads at the head of a run-time loop that carries loads in registers
#pragma unroll
  for (int rd = 0; rd < ROUNDS; rd++) {
#pragma unroll
    for (int i = 0; i < RING; i++) {
      // slots issued after this one: RING - 1, fewer at the very end
      const int later = PER * (rd + 1 < ROUNDS ? RING - 1 : RING - 1 - i);
      static_assert(RING == 3, "the three wait immediates below");
      if (later == 2 * PER) __builtin_amdgcn_s_waitcnt(0x0F70 | ((2 * PER) & 0xF) | (((2 * PER) >> 4) << 14));
      else if (later == PER) __builtin_amdgcn_s_waitcnt(0x0F70 | (PER & 0xF) | ((PER >> 4) << 14));
      else __builtin_amdgcn_s_waitcnt(0x0F70);
      const unsigned char* tile = mine + i * SLOT;
      u32x4_t w[4];
#pragma unroll
      for (int j = 0; j < 4; j++) w[j] = *(const u32x4_t*)(tile + roff[j]);
      if constexpr (XR) {
#pragma unroll
        for (int f = 0; f < 8; f++) x[0][f] = *(const u32x4_t*)(tile + (1 + f / 4) * TILE + xoff[f % 4]);
        // tile and activations are in registers before the slot is refilled below
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      }
      // zero scales for a surplus slot: it adds nothing (selected here, not where the scales
      // are loaded: a use right behind the load would wait for it and everything before it)
      const u32x4_t z = {0, 0, 0, 0};
      const bool live = wave + (rd * RING + i) * NW < steps;
      const half8_t s8 = __builtin_bit_cast(half8_t, live ? sc[i] : z);
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const half_t sv = g < 2 ? s8[2 * j] : s8[2 * j + 1];
        const half2_t s2 = {sv, sv};
        const half8_t a0 = dequant8(w[j][0], w[j][1], s2), a1 = dequant8(w[j][2], w[j][3], s2);
        const half8_t b0 = __builtin_bit_cast(half8_t, xvalid ? x[XR ? 0 : i][2 * j] : z);
        const half8_t b1 = __builtin_bit_cast(half8_t, xvalid ? x[XR ? 0 : i][2 * j + 1] : z);
        acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, b0, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, b1, acc1, 0, 0, 0);
      }
      // the slot's tile and registers have been consumed: refill it
      __builtin_amdgcn_sched_barrier(0);
      if (rd + 1 < ROUNDS) issue(i, wave + ((rd + 1) * RING + i) * NW);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

  __syncthreads();
  float* partial = (float*)ring;  // [NW][256]
#pragma unroll
  for (int i = 0; i < 4; i++) partial[wave * 256 + (4 * g + i) * 16 + r] = acc0[i] + acc1[i];
  __syncthreads();
  for (int e = tid; e < ROWS * 16; e += NW * 64) {
    const int mm = e / ROWS, nn = e % ROWS;  // consecutive threads -> consecutive output columns
    if (mm < m && n0 + nn < n) {
      float sum = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < NW; w2++) sum += partial[w2 * 256 + nn * 16 + mm];
      half_t* o = out + (int64_t)mm * n + n0 + nn;
      // the previous output is read even for beta == 0, as the reference does
      *o = (half_t)(sum + beta * (float)*o);
    }
  }
}

// MR activation rows, NW wavefronts, RPB weight rows per workgroup, SEGW 1 KiB K segments per
// wavefront (wavefront w owns segments w, w+NW, ...).
template <int MR, int NW, int RPB, int SEGW>
__global__ __launch_bounds__(NW * 64) void gemv_u8_dot_kernel(half_t* __restrict__ out,
                                                              const half_t* __restrict__ lhs,
                                                              const uint8_t* __restrict__ rhs,
                                                              const half_t* __restrict__ scales,
                                                              int m, int p, int n, int block_size,
                                                              float beta) {
  __shared__ float partial[NW][RPB][MR];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * RPB;
  const int nblk = p / block_size;
  const int nseg = (p + 1023) / 1024;
  half8_t xr[SEGW][MR][2];  // this lane's 16 activations of each owned segment and row
  float xs[SEGW][MR];       // 1151.5 * their sum
  bool act[SEGW];
  int sidx[SEGW];           // scale block of the lane's 16 weights
  // All loads of the workgroup are issued up front and unconditionally (a load under a branch
  // would be waited for at the join): inactive segments and rows beyond m read a clamped address
  // and are zeroed afterwards.
  u32x4_t xraw[SEGW][MR][2];
#pragma unroll
  for (int j = 0; j < SEGW; j++) {
    const int seg = wave + j * NW;
    const int k = seg * 1024 + lane * 16;
    act[j] = seg < nseg && k < p;
    sidx[j] = k / block_size;
    const int kc = act[j] ? k : 0;
#pragma unroll
    for (int mm = 0; mm < MR; mm++) {
      const half_t* xp = lhs + (int64_t)min(mm, m - 1) * p + kc;
      xraw[j][mm][0] = *(const u32x4_t*)xp;
      xraw[j][mm][1] = *(const u32x4_t*)(xp + 8);
    }
  }
  u32x4_t wall[RPB][SEGW];
  half_t scall[RPB][SEGW];
#pragma unroll
  for (int r = 0; r < RPB; r++) {
    const int row = min(n0 + r, n - 1);  // rows beyond n are clamped; their sums are not stored
    const uint8_t* wp = rhs + (int64_t)row * p + lane * 16;
    const half_t* sp = scales + (int64_t)row * nblk;
#pragma unroll
    for (int j = 0; j < SEGW; j++) {
      // streaming load: a weight byte is read once per launch
      wall[r][j] = __builtin_nontemporal_load(
          (const u32x4_t*)(wp + (act[j] ? (wave + j * NW) * 1024 : -lane * 16)));
      const half_t sv = sp[act[j] ? sidx[j] : 0];
      scall[r][j] = act[j] ? sv : (half_t)0;
    }
  }
#pragma unroll
  for (int j = 0; j < SEGW; j++) {
#pragma unroll
    for (int mm = 0; mm < MR; mm++) {
      const bool v = act[j] && mm < m;
      const u32x4_t z = {0, 0, 0, 0};
      xr[j][mm][0] = __builtin_bit_cast(half8_t, v ? xraw[j][mm][0] : z);
      xr[j][mm][1] = __builtin_bit_cast(half8_t, v ? xraw[j][mm][1] : z);
      float sum = 0.0f;
#pragma unroll
      for (int e = 0; e < 8; e++) sum += (float)xr[j][mm][0][e] + (float)xr[j][mm][1][e];
      xs[j][mm] = 1151.5f * sum;
    }
  }
#pragma unroll
  for (int r = 0; r < RPB; r++) {
    const u32x4_t (&w)[SEGW] = wall[r];
    const half_t (&sc)[SEGW] = scall[r];
    float tot[MR];
#pragma unroll
    for (int mm = 0; mm < MR; mm++) tot[mm] = 0.0f;
#pragma unroll
    for (int j = 0; j < SEGW; j++) {
      float pp[MR];
#pragma unroll
      for (int mm = 0; mm < MR; mm++) pp[mm] = -xs[j][mm];
#pragma unroll
      for (int e = 0; e < 4; e++) {
        // bytes b0..b3 of the dword -> halves (1024+b0, 1024+b1) and (1024+b2, 1024+b3)
        const uint32_t lo = __builtin_amdgcn_perm(0x64646464u, w[j][e], 0x07010700u);
        const uint32_t hi = __builtin_amdgcn_perm(0x64646464u, w[j][e], 0x07030702u);
#pragma unroll
        for (int mm = 0; mm < MR; mm++) {
          const half8_t x8 = xr[j][mm][e >> 1];
          const h2_t x01 = {x8[(e & 1) * 4], x8[(e & 1) * 4 + 1]};
          const h2_t x23 = {x8[(e & 1) * 4 + 2], x8[(e & 1) * 4 + 3]};
          pp[mm] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, lo), x01, pp[mm], false);
          pp[mm] = __builtin_amdgcn_fdot2(__builtin_bit_cast(h2_t, hi), x23, pp[mm], false);
        }
      }
      const float s = (float)sc[j];
#pragma unroll
      for (int mm = 0; mm < MR; mm++) tot[mm] += s * pp[mm];
    }
#pragma unroll
    for (int mm = 0; mm < MR; mm++) {
      const float v = wave_sum_dpp(tot[mm]);
      if (lane == 63) partial[wave][r][mm] = v;
    }
  }
  __syncthreads();
  for (int e = tid; e < RPB * MR; e += NW * 64) {
    const int mm = e / RPB, r = e % RPB;  // consecutive threads -> consecutive output columns
    if (mm < m && n0 + r < n) {
      float sum = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < NW; w2++) sum += partial[w2][r][mm];
      half_t* o = out + (int64_t)mm * n + n0 + r;
      // the previous output is read even for beta == 0, as the reference does
      *o = (half_t)(sum + beta * (float)*o);
    }
  }
}

template <int MR, int NW, int RPB, int SEGW>
hipError_t launch_dot(hipStream_t stream, half_t* out, const half_t* lhs, const uint8_t* rhs,
                      const half_t* scales, int m, int p, int n, int block_size, float beta) {
  hipLaunchKernelGGL((gemv_u8_dot_kernel<MR, NW, RPB, SEGW>), dim3((n + RPB - 1) / RPB),
                     dim3(NW * 64), 0, stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
  return hipGetLastError();
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

enum U8Choice { U8_NAIVE = 0, U8_DOT, U8_GEMV, U8_GEMM };

U8Choice choose_u8(const void* lhs, const void* rhs, const void* scales, int m, int p, int n,
                   int block_size) {
  const bool aligned = ((uintptr_t)lhs % 16 == 0) && ((uintptr_t)rhs % 16 == 0) &&
                       ((uintptr_t)scales % 16 == 0);
  // (p == 0: the operands may be null pointers; the per-output kernel then never reads them)
  if (!aligned || p == 0) return U8_NAIVE;
  // dot-product kernel: 16 weights of a lane share one scale; at most 16 segments of 1 KiB.
  // It wins for one or two activation rows; from three on its VALU work (dot products and lane
  // reductions per activation row) costs more than the MFMA kernels' less coalesced loads.
  const bool dot_ok = block_size % 16 == 0 && p % 16 == 0 && p <= 16 * 1024;
  if (dot_ok && m <= 2) return U8_DOT;
  if (m <= 16 && block_size == 32 && p % MACRO_K == 0) return U8_GEMV;
  if (block_size % 8 == 0 && p % 8 == 0) return U8_GEMM;
  return U8_NAIVE;
}

// 17 to 64 activation rows (to 128 on matrices under 8192 rows) against at least 4 MiB of
// weights: the sixteen-row kernels once per block of sixteen rows.  The tiled GEMM walks K on
// N / 64 .. N / 128 CUs for these (K4096 N4096 m=17..32 42.9 us, m=64..128 58.5; N12288 53.4 ..
// 68.5; K11008 N4096 133 .. 171) where a sixteen-row launch takes 7.2 / 15.3 / 17.1 us (N12288
// m=96: 78.4 us in blocks against 68.3 tiled, hence the narrower bound there).
bool rows_in_blocks_of_16(int m, int p, int n, int block_size) {
  return m > 16 && m <= (n < 8192 ? 128 : 64) && (int64_t)n * p >= (1 << 22) &&
         choose_u8(nullptr, nullptr, nullptr, 16, p, n, block_size) == U8_GEMV;
}

}  // namespace

hipError_t launch_gemm_u8_mfma(hipStream_t stream, half_t* out, const half_t* lhs,
                               const uint8_t* rhs, const half_t* scales, int m, int p, int n,
                               int block_size, float beta);
const char* gemm_u8_mfma_plan(int m, int p, int n, int block_size);
bool gemm_u8_mfma_supported(const half_t* lhs, const uint8_t* rhs, const half_t* scales, int m, int p,
                            int n, int block_size);

const char* gemm_u8_plan(int m, int p, int n, int block_size) {
  if (rows_in_blocks_of_16(m, p, n, block_size)) m = 16;
  switch (choose_u8(nullptr, nullptr, nullptr, m, p, n, block_size)) {
    case U8_DOT: return "gemv_u8_dot2_stream";
    case U8_GEMV:
      if (p == 16 * MACRO_K) return n < 8192 ? "gemv_u8_mfma16_dma" : "gemv_u8_mfma16_wide_dma";
      if (n < 8192 && p > 16 * MACRO_K && p <= 72 * MACRO_K) return "gemv_u8_mfma16_dma";
      return n < 8192 ? "gemv_u8_mfma16_stream" : "gemv_u8_mfma16_wide";
    case U8_GEMM: {
      // the tile is part of the name: "gemm_nt_u8_mfma_256x192x64", "gemm_nt_u8_stage_128x128x32", ...
      const char* tiled = gemm_u8_mfma_plan(m, p, n, block_size);
      return tiled ? tiled : "gemm_u8_naive";
    }
    default: return "gemm_u8_naive";
  }
}

hipError_t launch_gemm_u8(hipStream_t stream, half_t* out, const half_t* lhs, const uint8_t* rhs,
                          const half_t* scales, int m, int p, int n, int block_size, float beta) {
  if (rows_in_blocks_of_16(m, p, n, block_size) &&
      choose_u8(lhs, rhs, scales, 16, p, n, block_size) == U8_GEMV) {
    // (p is a multiple of 256 here, so every block of rows starts 16-byte aligned)
    // K 4096: blocks of 32 rows on the ring kernel with two blocks of activations (m=32: N4096
    // 13.3 -> 8.8 us, N12288 27.5 -> 18.4; m=64: 25.1 -> 16.8, 52.9 -> 34.9)
    const int step = p == 16 * MACRO_K ? 32 : 16;
    for (int r0 = 0; r0 < m; r0 += step) {
      const int mb = min(step, m - r0);
      half_t* o = out + (int64_t)r0 * n;
      const half_t* l = lhs + (int64_t)r0 * p;
      hipError_t e;
      if (mb > 16) {
        if (n >= 8192)
          hipLaunchKernelGGL((gemv_u8_ring_kernel<8, 3, 4, 2>), dim3((n + 3 * ROWS - 1) / (3 * ROWS)),
                             dim3(512), 0, stream, o, l, rhs, scales, mb, p, n, beta);
        else
          hipLaunchKernelGGL((gemv_u8_ring_kernel<8, 1, 4, 2>), dim3((n + ROWS - 1) / ROWS), dim3(512),
                             0, stream, o, l, rhs, scales, mb, p, n, beta);
        e = hipGetLastError();
      } else {
        e = launch_gemm_u8(stream, o, l, rhs, scales, mb, p, n, block_size, beta);
      }
      if (e != hipSuccess) return e;
    }
    return hipSuccess;
  }
  switch (choose_u8(lhs, rhs, scales, m, p, n, block_size)) {
    case U8_DOT: {
      const bool wide = n > 6144;
      if (p <= 4096) {  // 4 wavefronts, one segment each
        if (m == 1) return wide ? launch_dot<1, 4, 4, 1>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta)
                                : launch_dot<1, 4, 2, 1>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
        return launch_dot<2, 4, 4, 1>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      }
      // up to 12 segments: 4 wavefronts, three segments each (K = 11008 has 11: one idle slot
      // instead of five with 8 x 2)
      if (m == 1 && p <= 12 * 1024)
        return launch_dot<1, 4, 4, 3>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      // up to 16 segments: 8 wavefronts, two segments each
      if (m == 1) return launch_dot<1, 8, 4, 2>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      return launch_dot<2, 8, 4, 2>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
    }
    case U8_GEMV: {
      const int blocks = (n + ROWS - 1) / ROWS;
      const int steps = p / MACRO_K;
      // enough wavefronts per workgroup to keep every macro step of a small problem in flight
      // wide matrices: 48 weight rows per workgroup share one fetch of the activations
      if (n >= 8192) {
        if (steps == 16)
          hipLaunchKernelGGL((gemv_u8_ring_kernel<8, 3, 4, 1>), dim3((n + 3 * ROWS - 1) / (3 * ROWS)),
                             dim3(512), 0, stream, out, lhs, rhs, scales, m, p, n, beta);
        else
          hipLaunchKernelGGL((gemv_u8_wide_kernel<8, 3>), dim3((n + 3 * ROWS - 1) / (3 * ROWS)),
                             dim3(512), 0, stream, out, lhs, rhs, scales, m, p, n, beta);
        return hipGetLastError();
      }
      if (steps == 16) {
        hipLaunchKernelGGL((gemv_u8_ring_kernel<8, 1, 4, 1>), dim3(blocks), dim3(512), 0, stream, out,
                           lhs, rhs, scales, m, p, n, beta);
        return hipGetLastError();
      }
      // ten rows and more, K 9472 .. 12288: four wavefronts, activations through LDS (K11008
      // N4096: m=16 19.7 -> 17.1 us, m=12 17.8 -> 16.5; m=8 16.3 -> 16.9, so not below ten)
      if (steps > 16 && m >= 10 && ((steps + 3) / 4 + 2) / 3 == 4) {
        hipLaunchKernelGGL((gemv_u8_ring_loop_kernel<4, 3, 4, true>), dim3(blocks), dim3(256), 0, stream,
                           out, lhs, rhs, scales, m, p, n, beta);
        return hipGetLastError();
      }
      if (steps > 16) {
        const int rounds = ((steps + 7) / 8 + 2) / 3;
        if (rounds == 1)
          hipLaunchKernelGGL((gemv_u8_ring_loop_kernel<8, 3, 1, false>), dim3(blocks), dim3(512), 0, stream,
                             out, lhs, rhs, scales, m, p, n, beta);
        else if (rounds == 2)
          hipLaunchKernelGGL((gemv_u8_ring_loop_kernel<8, 3, 2, false>), dim3(blocks), dim3(512), 0, stream,
                             out, lhs, rhs, scales, m, p, n, beta);
        else if (rounds == 3)
          hipLaunchKernelGGL((gemv_u8_ring_loop_kernel<8, 3, 3, false>), dim3(blocks), dim3(512), 0, stream,
                             out, lhs, rhs, scales, m, p, n, beta);
        if (rounds <= 3) return hipGetLastError();
      }
      if (steps >= 16 && blocks <= 1024)
        hipLaunchKernelGGL(gemv_u8_kernel<8>, dim3(blocks), dim3(512), 0, stream, out, lhs, rhs,
                           scales, m, p, n, beta);
      else
        hipLaunchKernelGGL(gemv_u8_kernel<4>, dim3(blocks), dim3(256), 0, stream, out, lhs, rhs,
                           scales, m, p, n, beta);
      return hipGetLastError();
    }
    case U8_GEMM:
      if (gemm_u8_mfma_supported(lhs, rhs, scales, m, p, n, block_size))
        return launch_gemm_u8_mfma(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      [[fallthrough]];  // no tiled kernel takes these operands: one thread per output
    default: {
      if ((m + 3) / 4 > 65535) return hipErrorInvalidConfiguration;
      hipLaunchKernelGGL(gemm_u8_naive_kernel, dim3((n + 63) / 64, (m + 3) / 4), dim3(256), 0,
                         stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      return hipGetLastError();
    }
  }
}

}  // namespace adr
