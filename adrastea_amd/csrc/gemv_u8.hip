// u8-quantised-weight skinny GEMM / GEMV for decode (m <= 16):
//   out[r,c] = fp16( sum_i lhs[r,i] * w[c,i] + beta * out[r,c] ),
//   w[c,i]   = (float(q[c,i]) - 127.5f) * float(scales[c, i/block_size])
// (adrastea_kernels/cpp/matmul_nt_fp16u8.cu:4-24 and
// matmul_nt_wmma_16x128x256_fp16u8.cu:5-7, 43-83; format quantize.cu:3-56).
//
// The problem is bound by streaming the u8 weights from HBM once.  Kernels:
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
//  gemv_u8_regstream_kernel (3 <= m <= 16, block size 32, K % 256 == 0)   the same arithmetic on
//      the matrix cores: one v_mfma_f32_16x16x32_f16 per scale block of 32 weights on the
//      integers 1024 + q, its accumulator input preset to -1151.5 * (sum of the block's
//      activations), the four results scaled in fp32.  Weights and activations are fetched in
//      pieces of 4 rows x 256 bytes per instruction (what DRAM serves at the streaming rate; the
//      matrix-core operand layout itself would ask for 16 rows x 64 bytes) into registers, and a
//      private 4 KiB LDS tile per wavefront turns them into operand layout.  Requests run a
//      fixed distance ahead of their use: a compute unit holds only some 64 KiB of requests in
//      flight whatever is asked, oldest wavefront first, so asking for everything up front
//      starves the younger wavefronts and leaves all arithmetic to the end.
//
//  gemv_u8_ring_kernel (17 .. 32 rows per pass, K = 4096)   v_mfma_f32_16x16x32_f16 on weights
//      dequantised to fp16 in registers exactly as the stand-alone dequantise kernel does (the
//      WMMA kernel's arithmetic), two blocks of sixteen activation rows per pass over the
//      weights, operands through a per-wavefront LDS ring filled by global -> LDS DMA.
#include "adr_common.hpp"

namespace adr {

// (gemm_mfma.hip) estimated time of the product on the tiled u8 kernel, us; negative: not covered
double gemm_u8_mfma_estimate_us(int m, int p, int n, int block_size);

namespace {

constexpr int MACRO_K = 256;  // k elements per macro step
constexpr int ROWS = 16;      // weight rows per workgroup

// K = 4096, 17 to 32 activation rows per pass (MB = 2 blocks of sixteen): weights and activations
// come in by global -> LDS DMA, four whole 256-byte row pieces per instruction, the weights are
// dequantised to fp16 in registers (the WMMA kernel's arithmetic).  A wavefront owns two macro
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

// 3 to 16 activation rows, any K % 256 == 0, block size 32.  A workgroup of eight wavefronts owns
// RG groups of sixteen weight rows; wavefront w owns the macro steps (256 k) w, w + 8, ...  Per
// macro step a wavefront handles PER = 2 + RG tiles of 4 KiB ([16 rows][256 bytes]): two of
// activations (k 0..127 and 128..255 of the step as fp16) and RG of weights.  Tile u of every
// step has its own four registers per lane; the request for a tile is issued three tiles before
// its use (two with one row group), as four instructions of 4 rows x 256 contiguous bytes (quarter a of the wavefront takes
// row 4i + a, lane x of the quarter the 16-byte chunk x).  On arrival the tile goes through the
// wavefront's private LDS tile (chunk c of row r at position c ^ r: both directions free of bank
// conflicts) and comes back in matrix-core operand layout: lane (r, g) gets, of row r, the 8
// weights g of a scale block, or the 8 activations g of its 32.
// Arithmetic per scale block b of a weight row (the naive kernel's formula, matmul_nt_fp16u8.cu:
// 17-21, in fp32):  sum_k x_k (q_k - 127.5) s_b = s_b (sum_k x_k (1024 + q_k) - 1151.5 sum_k x_k).
// The activations are the FIRST matrix-core operand, so a lane's four results are four
// activation rows of ONE weight row (lane % 16) and take one scale; sum_k x_k comes from a
// product with an all-ones operand once per step and enters the block's product as accumulator
// input, times -1151.5.  Every product x_k (1024 + q_k) is exact in fp32.
// MQ: groups of four activation rows that exist (requests for the others are left out at compile
// time; the LDS tile then holds stale rows there, which only reach results that are not stored).
template <int RG, int MQ>
__global__ __launch_bounds__(512) void gemv_u8_regstream_kernel(half_t* __restrict__ out,
                                                                const half_t* __restrict__ lhs,
                                                                const uint8_t* __restrict__ rhs,
                                                                const half_t* __restrict__ scales,
                                                                int m, int p, int n, float beta) {
  constexpr int NW = 8, TILE = ROWS * MACRO_K, RB = ROWS * RG, PER = 2 + RG;
  constexpr int DIST = PER - 1 < 3 ? PER - 1 : 3;  // tiles between a request and its use
  __shared__ __attribute__((aligned(1024))) unsigned char shuf[NW][TILE];
  __shared__ float partial[NW][RG][256];
  const int tid = threadIdx.x, lane = tid & 63;
  // (wave-uniform by construction; said so, the step's addresses live in scalar registers)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int a = lane >> 4, x = lane & 15;  // request role: quarter a takes row 4i + a, chunk x
  const int r = lane & 15, g = lane >> 4;  // operand role: row r, group g of 8 within a block of 32
  const int n0 = blockIdx.x * RB;
  const int nblk = p / 32, steps = p / MACRO_K, last = steps - 1;
  unsigned char* const mine = shuf[wave];
  // the previous output of the elements this thread will store, requested before anything else
  // (unconditionally, from a clamped address: a load under a lane mask is waited for where the
  // lanes rejoin); read even for beta == 0, as the reference does
  constexpr int EPT = (RB * 16 + NW * 64 - 1) / (NW * 64);
  half_t prev[EPT];
#pragma unroll
  for (int k = 0; k < EPT; k++) {
    const int e = tid + k * NW * 64, mm = e / RB, nn = e % RB;
    prev[k] = out[(int64_t)min(mm, m - 1) * n + min(n0 + nn, n - 1)];
  }
  // scales of a step: the eight blocks of row q * 16 + r (16 bytes), requested a whole step ahead
  uint32_t so[RG];
#pragma unroll
  for (int q = 0; q < RG; q++) so[q] = (uint32_t)min(q * ROWS + r, n - 1 - n0) * (uint32_t)nblk * 2u;
  const unsigned char* const sbase = (const unsigned char*)(scales + (int64_t)n0 * nblk);
  u32x4_t sc[RG], sc_next[RG];
#pragma unroll
  for (int q = 0; q < RG; q++) sc[q] = *(const u32x4_t*)(sbase + min(wave, last) * 16 + so[q]);
  // Request addresses: a uniform base per step (scalar registers) plus one 32-bit byte offset per
  // lane and instruction.  Rows beyond m read row m - 1 again and rows beyond n row n - 1 (their
  // products are never stored).
  uint32_t xo[MQ], wo[RG][4];
#pragma unroll
  for (int i = 0; i < MQ; i++) xo[i] = (uint32_t)min(4 * i + a, m - 1) * (uint32_t)p * 2u + x * 16;
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int i = 0; i < 4; i++)
      wo[q][i] = (uint32_t)min(q * ROWS + 4 * i + a, n - 1 - n0) * (uint32_t)p + x * 16;
  const unsigned char* const xbase = (const unsigned char*)lhs;
  const unsigned char* const wbase = rhs + (int64_t)n0 * p;
  u32x4_t ld[PER][4];
  auto request = [&](int ms, int u) {  // tile u of macro step ms into its registers
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (u < 2) {
        if (i < MQ) ld[u][i] = *(const u32x4_t*)(xbase + (int64_t)ms * (MACRO_K * 2) + u * 256 + xo[i]);
      } else {
        // streaming load: a weight byte is read once per launch
        ld[u][i] = __builtin_nontemporal_load(
            (const u32x4_t*)(wbase + (int64_t)ms * MACRO_K + wo[u - 2][i]));
      }
    }
  };
#pragma unroll
  for (int u = 0; u < DIST; u++) request(min(wave, last), u);

  int woff[4], roff[8], xoff[4];
#pragma unroll
  for (int i = 0; i < 4; i++) woff[i] = (4 * i + a) * 256 + ((x ^ (4 * i + a)) << 4);
  // weights of block b = bytes 32 b .. 32 b + 31 of the row: lane (r, g) takes bytes 8 g .. 8 g + 7
#pragma unroll
  for (int b = 0; b < 8; b++) roff[b] = r * 256 + (((2 * b + (g >> 1)) ^ r) << 4) + (g & 1) * 8;
  // activations of block b = chunks 4 b .. 4 b + 3 of the step: tile b / 4, chunk 4 (b % 4) + g
#pragma unroll
  for (int b = 0; b < 4; b++) xoff[b] = r * 256 + (((4 * b + g) ^ r) << 4);

  float4_t acc[RG];
#pragma unroll
  for (int q = 0; q < RG; q++) acc[q] = float4_t{0, 0, 0, 0};
  const half_t one = (half_t)1.0f;
  const half8_t ones = {one, one, one, one, one, one, one, one};
  half8_t xf[8];    // activation operands of the step's eight blocks
  float4_t c0[8];   // -1151.5 * their sums, in result layout

#pragma unroll 1
  for (int ms = wave; ms < steps; ms += NW) {
    const int ms_next = min(ms + NW, last);  // (past the end: the last step again, never used)
#pragma unroll
    for (int u = 0; u < PER; u++) {
      __builtin_amdgcn_sched_barrier(0);
      if (u + DIST < PER) request(ms, u + DIST); else request(ms_next, u + DIST - PER);
      if (u == 0) {
#pragma unroll
        for (int q = 0; q < RG; q++) sc_next[q] = *(const u32x4_t*)(sbase + ms_next * 16 + so[q]);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; i++)
        if (u >= 2 || i < MQ) *(u32x4_t*)(mine + woff[i]) = ld[u][i];
      if (u < 2) {
#pragma unroll
        for (int b = 0; b < 4; b++) xf[4 * u + b] = *(const half8_t*)(mine + xoff[b]);
#pragma unroll
        for (int b = 0; b < 4; b++) {
          const float4_t z = {0, 0, 0, 0};
          c0[4 * u + b] =
              __builtin_amdgcn_mfma_f32_16x16x32_f16(xf[4 * u + b], ones, z, 0, 0, 0) * -1151.5f;
        }
      } else {
        const int q = u - 2;
        const half8_t s8 = __builtin_bit_cast(half8_t, sc[q]);
#pragma unroll
        for (int h = 0; h < 2; h++) {
          u32x2_t w[4];
#pragma unroll
          for (int b = 0; b < 4; b++) w[b] = *(const u32x2_t*)(mine + roff[4 * h + b]);
#pragma unroll
          for (int b = 0; b < 4; b++) {
            // bytes b0..b3 of a dword -> halves (1024 + b0, 1024 + b1) and (1024 + b2, 1024 + b3)
            u32x4_t v;
            v[0] = __builtin_amdgcn_perm(0x64646464u, w[b][0], 0x07010700u);
            v[1] = __builtin_amdgcn_perm(0x64646464u, w[b][0], 0x07030702u);
            v[2] = __builtin_amdgcn_perm(0x64646464u, w[b][1], 0x07010700u);
            v[3] = __builtin_amdgcn_perm(0x64646464u, w[b][1], 0x07030702u);
            const float4_t d = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                xf[4 * h + b], __builtin_bit_cast(half8_t, v), c0[4 * h + b], 0, 0, 0);
            acc[q] += d * (float)s8[4 * h + b];
          }
        }
      }
    }
#pragma unroll
    for (int q = 0; q < RG; q++) sc[q] = sc_next[q];
  }

  // lane (weight row r, group g): acc[q][i] belongs to activation row 4 g + i
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int i = 0; i < 4; i++) partial[wave][q][r * 16 + 4 * g + i] = acc[q][i];
  // (not __syncthreads(): its fence would wait for the surplus requests of the last step)
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the partial sums are in LDS
  __builtin_amdgcn_s_barrier();
#pragma unroll
  for (int k = 0; k < EPT; k++) {
    const int e = tid + k * NW * 64, mm = e / RB, nn = e % RB;  // consecutive threads -> consecutive columns
    if (e < RB * 16 && mm < m && n0 + nn < n) {
      float sum = 0.0f;
#pragma unroll
      for (int w2 = 0; w2 < NW; w2++) sum += partial[w2][nn / ROWS][(nn % ROWS) * 16 + mm];
      out[(int64_t)mm * n + n0 + nn] = (half_t)(sum + beta * (float)prev[k]);
    }
  }
}

// 17 to 64 activation rows, block size 32, any K % 256 == 0: the request pipeline of the kernel
// above with MB blocks of sixteen activation rows per workgroup, so that the weights are read
// once for all of them.  With two blocks and more the per-block correction term of the kernel
// above would not fit the register file; the VALU work that trick saves is small beside the
// time the bytes take anyway, so here every weight is dequantised to fp16 exactly as
// dequantize_absmax_uint8 does (dequant8, the formula of the reference's WMMA kernel, as in the
// tiled u8 GEMM) and v_mfma_f32_16x16x32_f16 accumulates straight into the result.  A macro
// step is 256 k: two tiles of activations per block (k 0..127 and 128..255) and RG tiles of
// weights.  It is walked in two halves so that only one half's activation operands (16
// registers per block) are live: the weight tiles stay in the wavefront's LDS slots, one per
// row group, between the halves.  Request order per step = consumption order: the blocks' first
// tiles, the weight tiles, the blocks' second tiles.
template <int RG, int MB>
__global__ __launch_bounds__(512) void gemv_u8_blocks_kernel(half_t* __restrict__ out,
                                                             const half_t* __restrict__ lhs,
                                                             const uint8_t* __restrict__ rhs,
                                                             const half_t* __restrict__ scales,
                                                             int m, int p, int n, float beta) {
  constexpr int NW = 8, TILE = ROWS * MACRO_K, RB = ROWS * RG, PER = 2 * MB + RG;
  constexpr int DIST = 3;  // tiles between a request and its use
  static_assert(PER > DIST, "a step holds more tiles than are in flight");
  // per wavefront: slot 0 for activation tiles, slots 1 .. RG for the step's weight tiles
  __shared__ __attribute__((aligned(1024))) unsigned char shuf[NW][RG + 1][TILE];
  static_assert(NW * MB * RG * 256 * 4 <= NW * (RG + 1) * TILE, "the partial sums reuse the tiles");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int a = lane >> 4, x = lane & 15;  // request role: quarter a takes row 4i + a, chunk x
  const int r = lane & 15, g = lane >> 4;  // operand role: row r, k-group g of a block of 32
  const int n0 = blockIdx.x * RB;
  const int nblk = p / 32, steps = p / MACRO_K, last = steps - 1;
  unsigned char* const mine = shuf[wave][0];

  // scales of a step: the eight blocks of row q * 16 + r (16 bytes), requested a whole step ahead
  uint32_t so[RG];
#pragma unroll
  for (int q = 0; q < RG; q++) so[q] = (uint32_t)min(q * ROWS + r, n - 1 - n0) * (uint32_t)nblk * 2u;
  const unsigned char* const sbase = (const unsigned char*)(scales + (int64_t)n0 * nblk);
  u32x4_t sc[RG], sc_next[RG];
#pragma unroll
  for (int q = 0; q < RG; q++) sc[q] = *(const u32x4_t*)(sbase + min(wave, last) * 16 + so[q]);
  // request addresses: a uniform base per step plus a 32-bit byte offset per lane and instruction
  // (rows beyond m read row m - 1 again, rows beyond n row n - 1: their products are never stored)
  uint32_t xo[MB][4], wo[RG][4];
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int i = 0; i < 4; i++)
      xo[b][i] = (uint32_t)min(b * ROWS + 4 * i + a, m - 1) * (uint32_t)p * 2u + x * 16;
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int i = 0; i < 4; i++)
      wo[q][i] = (uint32_t)min(q * ROWS + 4 * i + a, n - 1 - n0) * (uint32_t)p + x * 16;
  const unsigned char* const xbase = (const unsigned char*)lhs;
  const unsigned char* const wbase = rhs + (int64_t)n0 * p;
  u32x4_t ld[PER][4];
  // tile u of a step: u < MB: first half of block u; u < MB + RG: weight group u - MB; else the
  // second half of block u - MB - RG
  auto request = [&](int ms, int u) {
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (u < MB)
        ld[u][i] = *(const u32x4_t*)(xbase + (int64_t)ms * (MACRO_K * 2) + xo[u][i]);
      else if (u < MB + RG)  // streaming load: a weight byte is read once per launch
        ld[u][i] = __builtin_nontemporal_load(
            (const u32x4_t*)(wbase + (int64_t)ms * MACRO_K + wo[u - MB][i]));
      else
        ld[u][i] = *(const u32x4_t*)(xbase + (int64_t)ms * (MACRO_K * 2) + 256 + xo[u - MB - RG][i]);
    }
  };
#pragma unroll
  for (int u = 0; u < DIST; u++) request(min(wave, last), u);

  int woff[4], roff[8], xoff[4];
#pragma unroll
  for (int i = 0; i < 4; i++) woff[i] = (4 * i + a) * 256 + ((x ^ (4 * i + a)) << 4);
  // weights of block b = bytes 32 b .. 32 b + 31 of the row: lane (r, g) takes bytes 8 g .. 8 g + 7
#pragma unroll
  for (int b = 0; b < 8; b++) roff[b] = r * 256 + (((2 * b + (g >> 1)) ^ r) << 4) + (g & 1) * 8;
  // activations of block b of a half = chunks 4 b .. 4 b + 3 of the tile: chunk 4 b + g
#pragma unroll
  for (int b = 0; b < 4; b++) xoff[b] = r * 256 + (((4 * b + g) ^ r) << 4);

  float4_t acc[MB][RG];
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int q = 0; q < RG; q++) acc[b][q] = float4_t{0, 0, 0, 0};
  half8_t xf[MB][4];  // activation operands of the current half: four blocks of 32 k

  // the weight operands of half h of row group q, from its LDS slot, against every block
  auto multiply = [&](int q, int h) {
    const unsigned char* slot = shuf[wave][1 + q];
    const half8_t s8 = __builtin_bit_cast(half8_t, sc[q]);
    u32x2_t w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) w[j] = *(const u32x2_t*)(slot + roff[4 * h + j]);
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const half2_t s2 = {s8[4 * h + j], s8[4 * h + j]};
      const half8_t wf = dequant8(w[j][0], w[j][1], s2);
#pragma unroll
      for (int b = 0; b < MB; b++)
        acc[b][q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf, xf[b][j], acc[b][q], 0, 0, 0);
    }
  };

#pragma unroll 1
  for (int ms = wave; ms < steps; ms += NW) {
    const int ms_next = min(ms + NW, last);  // (past the end: the last step again, never used)
#pragma unroll
    for (int u = 0; u < PER; u++) {
      __builtin_amdgcn_sched_barrier(0);
      if (u + DIST < PER) request(ms, u + DIST); else request(ms_next, u + DIST - PER);
      if (u == 0) {
#pragma unroll
        for (int q = 0; q < RG; q++) sc_next[q] = *(const u32x4_t*)(sbase + ms_next * 16 + so[q]);
      }
      __builtin_amdgcn_sched_barrier(0);
      const bool weights = u >= MB && u < MB + RG;
      unsigned char* dst = weights ? shuf[wave][1 + (u - MB)] : mine;
#pragma unroll
      for (int i = 0; i < 4; i++) *(u32x4_t*)(dst + woff[i]) = ld[u][i];
      if (!weights) {
        const int b = u < MB ? u : u - MB - RG;
#pragma unroll
        for (int j = 0; j < 4; j++) xf[b][j] = *(const half8_t*)(mine + xoff[j]);
      }
      if (u == MB + RG - 1) {  // all of the step's weights and the first halves are in: half 0
#pragma unroll
        for (int q = 0; q < RG; q++) multiply(q, 0);
      }
      if (u == PER - 1) {      // the second halves are in: half 1
#pragma unroll
        for (int q = 0; q < RG; q++) multiply(q, 1);
      }
    }
#pragma unroll
    for (int q = 0; q < RG; q++) sc[q] = sc_next[q];
  }

  // lane (r, g): acc[b][q][v] is weight row 4g + v of group q against activation row r of block b
  // (not __syncthreads(): its fence would wait for the surplus requests of the last step)
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): this wavefront's tiles are dead
  __builtin_amdgcn_s_barrier();        // ... and everybody else's
  float* const partial = (float*)&shuf[0][0][0];  // [NW][MB][RG][256]
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int q = 0; q < RG; q++)
#pragma unroll
      for (int v = 0; v < 4; v++)
        partial[((wave * MB + b) * RG + q) * 256 + (4 * g + v) * 16 + r] = acc[b][q][v];
  __builtin_amdgcn_s_waitcnt(0xC07F);
  __builtin_amdgcn_s_barrier();
  for (int e = tid; e < MB * RG * 256; e += NW * 64) {
    const int col = e % RB, y = e / RB;  // consecutive threads -> consecutive columns
    if (y >= m || n0 + col >= n) continue;
    float sum = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < NW; w2++)
      sum += partial[((w2 * MB + y / 16) * RG + col / 16) * 256 + (col % 16) * 16 + y % 16];
    half_t* o = out + (int64_t)y * n + n0 + col;
    // the previous output is read even for beta == 0, as the reference does
    *o = (half_t)(sum + beta * (float)*o);
  }
}

template <int RG, int MB>
hipError_t launch_blocks(hipStream_t stream, half_t* out, const half_t* lhs, const uint8_t* rhs,
                         const half_t* scales, int m, int p, int n, float beta) {
  hipLaunchKernelGGL((gemv_u8_blocks_kernel<RG, MB>), dim3((n + ROWS * RG - 1) / (ROWS * RG)), dim3(512), 0,
                     stream, out, lhs, rhs, scales, m, p, n, beta);
  return hipGetLastError();
}

template <int RG>
hipError_t launch_regstream(hipStream_t stream, half_t* out, const half_t* lhs, const uint8_t* rhs,
                            const half_t* scales, int m, int p, int n, float beta) {
  const dim3 grid((n + ROWS * RG - 1) / (ROWS * RG)), block(512);
  switch ((m + 3) / 4) {
    case 1: hipLaunchKernelGGL((gemv_u8_regstream_kernel<RG, 1>), grid, block, 0, stream, out, lhs, rhs, scales, m, p, n, beta); break;
    case 2: hipLaunchKernelGGL((gemv_u8_regstream_kernel<RG, 2>), grid, block, 0, stream, out, lhs, rhs, scales, m, p, n, beta); break;
    case 3: hipLaunchKernelGGL((gemv_u8_regstream_kernel<RG, 3>), grid, block, 0, stream, out, lhs, rhs, scales, m, p, n, beta); break;
    default: hipLaunchKernelGGL((gemv_u8_regstream_kernel<RG, 4>), grid, block, 0, stream, out, lhs, rhs, scales, m, p, n, beta); break;
  }
  return hipGetLastError();
}

// groups of sixteen weight rows per workgroup: as many as still give every compute unit a
// workgroup (at most three: 48 rows share one fetch of the activations), but never a count that
// leaves a second, nearly empty round of workgroups (N5120, 320 groups: two per workgroup, K13824
// m=32 39.3 -> 31.4 us; N13824, 288 workgroups of three: two, K5120 m=32 39.0 -> 29.7)
int regstream_row_groups(int n) {
  const int cus = device_info_for_plan().cus;
  const int groups = (n + ROWS - 1) / ROWS;
  if (groups <= cus) return 1;
  if (groups < 3 * cus - cus / 2) return 2;
  const int w3 = (groups + 2) / 3;
  return w3 > cus && w3 <= 2 * cus && w3 % cus <= cus / 4 ? 2 : 3;
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
  // (two rows over a long K: the matrix-core kernel, K11008 N4096 11.8 against 13.4 us; equal on K 4096)
  const bool gemv_ok = block_size == 32 && p % MACRO_K == 0;
  if (dot_ok && m <= 2 && !(m == 2 && p > 4096 && gemv_ok)) return U8_DOT;
  if (m <= 16 && gemv_ok) return U8_GEMV;
  if (block_size % 8 == 0 && p % 8 == 0) return U8_GEMM;
  return U8_NAIVE;
}

// 17 activation rows and more against at least 4 MiB of weights: passes of up to 64 rows on the
// matrix-core streaming kernels, each pass reading the weights once.  A pass of 64 rows is one
// workgroup per sixteen weight rows, 2 + 0.0023 K us per round of them over the CUs (K4096 N4096
// 13.1 us, N8192 23.5, N12288 33.9, K11008 N4096 26.4, K5120 N5120 25.7); a last pass of r rows
// costs 0.55 + 0.45 r / 64 of that.  Up to 32 rows the passes always win (K4096 N12288 m=32 18 us
// against 25 on 64 x 64 tiles); above, where this estimate is below the tiled kernel's own.
// Measured with weights that come from HBM: K11008 N4096 m=64 27 against 61 us (passes), m=96 45
// against 53, m=128 53 against 59, m=160 71 against 53 (tiled); K4096 N4096 m=96 22.4 against 23.2,
// m=128 a tie, m=160 36 against 23; wide matrices are tiled from 33 rows (K4096 N12288 m=40 29
// against 26, m=64 34 against 28, m=70 47 against 31; K5120 N13824 m=64 50 against 36), 13B-sized
// narrow ones from 65 (K13824 N5120 m=64 58 against 77, m=70 78 against 57).
bool rows_in_passes(int m, int p, int n, int block_size) {
  if (m <= 16 || m > 256 || (int64_t)n * p < (1 << 22) ||
      choose_u8(nullptr, nullptr, nullptr, 16, p, n, block_size) != U8_GEMV)
    return false;
  // (a test or benchmark forces a tile of the tiled kernel, or -- value 9 -- the passes)
  if (knob(KNOB_U8_TILE)) return knob(KNOB_U8_TILE) == 9;
  if (m <= 32) return true;
  const int cus = device_info_for_plan().cus;
  // one pass of up to three blocks of rows against a matrix so wide that the 64 x 64 tiles need a
  // second round: K6656 N17920 m=40 57.5 us against 73.6, K8192 N22016 m=48 74 against 89 (weights
  // from HBM; with four blocks the pass loses: m=64 104 against 92)
  if (m <= 48 && (n + 63) / 64 > cus) return true;
  const int rounds = ((n + ROWS - 1) / ROWS + cus - 1) / cus;
  const double t64 = fmax(12.0, rounds * (2.0 + 0.0023 * p));
  const int rem = m % 64;
  const double passes = (m / 64) * t64 + (rem ? t64 * (0.55 + 0.45 * rem / 64.0) : 0.0);
  const double tiled = gemm_u8_mfma_estimate_us(m, p, n, block_size);
  return tiled < 0.0 || passes < tiled;
}

}  // namespace

hipError_t launch_gemm_u8_mfma(hipStream_t stream, half_t* out, const half_t* lhs,
                               const uint8_t* rhs, const half_t* scales, int m, int p, int n,
                               int block_size, float beta);
const char* gemm_u8_mfma_plan(int m, int p, int n, int block_size);
bool gemm_u8_mfma_supported(const half_t* lhs, const uint8_t* rhs, const half_t* scales, int m, int p,
                            int n, int block_size);

const char* gemm_u8_plan(int m, int p, int n, int block_size) {
  if (rows_in_passes(m, p, n, block_size))
    return m <= 32 && p == 16 * MACRO_K ? "gemv_u8_mfma16_dma_32rows" : "gemv_u8_mfma16_blocks";
  switch (choose_u8(nullptr, nullptr, nullptr, m, p, n, block_size)) {
    case U8_DOT: return "gemv_u8_dot2_stream";
    case U8_GEMV: return "gemv_u8_mfma16_regstream";
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
  if (rows_in_passes(m, p, n, block_size) &&
      choose_u8(lhs, rhs, scales, 16, p, n, block_size) == U8_GEMV) {
    // 17 rows and more against 4 MiB of weights and more: passes of up to 64 rows, each reading
    // the weights once for two to four blocks of sixteen rows (p is a multiple of 256 here, so
    // every pass starts 16-byte aligned).  Row groups per workgroup as the register file allows:
    // two with two or three blocks, one with four.  K11008 N4096 m=32 / 64 / 128:
    // 28.5 / 55.1 / 112 us in passes of sixteen rows -> 19.0 / 26.4 / 53.
    const int rg = regstream_row_groups(n);
    for (int r0 = 0; r0 < m; r0 += 64) {
      const int mb = min(64, m - r0);
      half_t* o = out + (int64_t)r0 * n;
      const half_t* l = lhs + (int64_t)r0 * p;
      hipError_t e;
      if (mb <= 16 && r0 > 0) {
        // The last pass of a product of more than 64 rows: on the kernels of the other passes
        // (weights rounded to fp16 as dequantize_absmax_uint8 does), so that every row of one
        // product sees the same arithmetic; the sixteen-row kernels evaluate the naive kernel's
        // formula on unrounded weights.
        e = rg == 3 ? launch_blocks<3, 1>(stream, o, l, rhs, scales, mb, p, n, beta)
          : rg == 2 ? launch_blocks<2, 1>(stream, o, l, rhs, scales, mb, p, n, beta)
                    : launch_blocks<1, 2>(stream, o, l, rhs, scales, mb, p, n, beta);
      } else if (mb <= 16) {
        e = launch_gemm_u8(stream, o, l, rhs, scales, mb, p, n, block_size, beta);
      } else if (mb <= 32 && p == 16 * MACRO_K) {
        // K 4096, up to 32 rows: the DMA-ring kernel with two blocks is 4-10 % ahead (m=32: N4096
        // 9.6 against 10.0 us, N12288 18.9 against 21.0)
        if (n >= 8192)
          hipLaunchKernelGGL((gemv_u8_ring_kernel<8, 3, 4, 2>), dim3((n + 3 * ROWS - 1) / (3 * ROWS)),
                             dim3(512), 0, stream, o, l, rhs, scales, mb, p, n, beta);
        else
          hipLaunchKernelGGL((gemv_u8_ring_kernel<8, 1, 4, 2>), dim3((n + ROWS - 1) / ROWS), dim3(512),
                             0, stream, o, l, rhs, scales, mb, p, n, beta);
        e = hipGetLastError();
      } else if (mb <= 32) {
        // (three row groups with two blocks spill four registers and are no faster: K5120 N13824
        // m=32 29.8-31.7 against 29.7-30.1 us)
        e = rg >= 2 ? launch_blocks<2, 2>(stream, o, l, rhs, scales, mb, p, n, beta)
                    : launch_blocks<1, 2>(stream, o, l, rhs, scales, mb, p, n, beta);
      } else if (mb <= 48) {
        e = rg >= 2 ? launch_blocks<2, 3>(stream, o, l, rhs, scales, mb, p, n, beta)
                    : launch_blocks<1, 3>(stream, o, l, rhs, scales, mb, p, n, beta);
      } else {
        e = launch_blocks<1, 4>(stream, o, l, rhs, scales, mb, p, n, beta);
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
      // up to 8 segments: 8 wavefronts, one segment each.  A workgroup takes as long as its busiest
      // wavefront, and 4 x 3 gives one of them two of K = 5120's five segments (LLaMA-13B: N13824
      // 21.6 -> 14.1 us, N5120 9.3 -> 7.4; K6656 N17920 26.0 -> 21.2, K8192 N8192 15.1 -> 13.3)
      if (m == 1 && p <= 8 * 1024)
        return launch_dot<1, 8, 4, 1>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      // up to 12 segments: twelve wavefronts with one each (K11008 N4096 10.8 -> 10.4 us, K9216 N9216
      // 17.9 -> 17.0, K12288 N12288 26.8 -> 25.7; four wavefronts with three each before, and
      // 8 x 2 behind that: 11.2 and 19.5)
      if (m == 1 && p <= 12 * 1024)
        return launch_dot<1, 12, 4, 1>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      // up to 16 segments: 8 wavefronts, two segments each
      if (m == 1) return launch_dot<1, 8, 4, 2>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
      return launch_dot<2, 8, 4, 2>(stream, out, lhs, rhs, scales, m, p, n, block_size, beta);
    }
    case U8_GEMV:
      switch (regstream_row_groups(n)) {
        case 3: return launch_regstream<3>(stream, out, lhs, rhs, scales, m, p, n, beta);
        case 2: return launch_regstream<2>(stream, out, lhs, rhs, scales, m, p, n, beta);
        default: return launch_regstream<1>(stream, out, lhs, rhs, scales, m, p, n, beta);
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
