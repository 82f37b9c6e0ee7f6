// fp16 skinny matmul for decode, m <= 8 activation rows against a K-contiguous weight matrix:
// the shape GpuKernels::matmul_f16 is called with once per generated token
// (adrastea_models/src/llama.rs:485-591: W[N,K].permute([1,0]) on a [tokens, K] activation;
// kernel arguments adrastea_models/src/kernels.rs:864-887).  The tiled kernels need tens of
// microseconds for it -- a handful of 64 x 64 tiles walking K slice by slice -- while the job is
// to read N x K x 2 bytes once.
//
// No matrix cores: a wavefront streams whole 1 KiB segments (512 k) of one weight row per load
// instruction (lane l: 16 bytes at l * 16, streaming loads), keeps the activations of its
// segments in registers for all rows of the workgroup, and accumulates with v_dot2_f32_f16
// (exact fp16 products, fp32 sums); lane sums are reduced with DPP adds, the wavefronts of a
// workgroup through LDS.  Every store operator and the causal mask are applied to the m x RPB
// results of the workgroup.
#include "adr_common.hpp"

namespace adr {

namespace {

// MR activation rows, NW wavefronts, RPB weight rows per workgroup, SEGW segments per wavefront
// (wavefront w owns segments w, w + NW, ...).
template <int MR, int NW, int RPB, int SEGW>
__global__ __launch_bounds__(NW * 64) void gemv_f16_dot_kernel(MatmulArgs a) {
  __shared__ float partial[NW][RPB][MR];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * RPB;
  // All loads of the workgroup are issued up front and unconditionally (a load under a branch
  // would be waited for at the join): segments past K and rows past m read a valid address and
  // are zeroed afterwards.  K % 8 == 0, so a lane's eight values are all inside or all outside.
  bool act[SEGW];
  u32x4_t xraw[SEGW][MR];
#pragma unroll
  for (int j = 0; j < SEGW; j++) {
    const int k = (wave + j * NW) * 512 + lane * 8;
    act[j] = k < a.k;
    const int kc = act[j] ? k : 0;
#pragma unroll
    for (int mm = 0; mm < MR; mm++)
      xraw[j][mm] = *(const u32x4_t*)(a.lhs + (int64_t)min(mm, a.m - 1) * a.stride_ly + kc);
  }
  u32x4_t w[RPB][SEGW];
#pragma unroll
  for (int r = 0; r < RPB; r++) {
    const half_t* wp = a.rhs + (int64_t)min(n0 + r, a.n - 1) * a.stride_rx;  // clamped, not stored
#pragma unroll
    for (int j = 0; j < SEGW; j++) {
      const int k = (wave + j * NW) * 512 + lane * 8;
      // streaming load: a weight is read once per launch
      w[r][j] = __builtin_nontemporal_load((const u32x4_t*)(wp + (act[j] ? k : 0)));
    }
  }
  u32x4_t x[SEGW][MR];
#pragma unroll
  for (int j = 0; j < SEGW; j++)
#pragma unroll
    for (int mm = 0; mm < MR; mm++)
      x[j][mm] = (act[j] && mm < a.m) ? xraw[j][mm] : u32x4_t{0, 0, 0, 0};
#pragma unroll
  for (int r = 0; r < RPB; r++) {
    float tot[MR];
#pragma unroll
    for (int mm = 0; mm < MR; mm++) tot[mm] = 0.0f;
#pragma unroll
    for (int j = 0; j < SEGW; j++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        // (through scalars: a bit_cast applied to a vector element directly reads element 0)
        const uint32_t wv = w[r][j][e];
        const h2_t w2 = __builtin_bit_cast(h2_t, wv);
#pragma unroll
        for (int mm = 0; mm < MR; mm++) {
          const uint32_t xv = x[j][mm][e];
          tot[mm] = __builtin_amdgcn_fdot2(w2, __builtin_bit_cast(h2_t, xv), tot[mm], false);
        }
      }
#pragma unroll
    for (int mm = 0; mm < MR; mm++) {
      const float v = wave_sum_dpp(tot[mm]);
      if (lane == 63) partial[wave][r][mm] = v;
    }
  }
  __syncthreads();
  const Epilogue ep{a.bias, a.beta, (half_t)a.scale, a.store, true};
  for (int e = tid; e < RPB * MR; e += NW * 64) {
    const int y = e / RPB, r = e % RPB, xcol = n0 + r;  // consecutive threads -> consecutive columns
    if (y >= a.m || xcol >= a.n) continue;
    half_t* o = a.output + (int64_t)y * a.stride_oy + (int64_t)xcol * a.stride_ox;
    if (a.mask == ADR_MASK_CAUSAL && xcol > y) {  // matmul.cu:210-213
      *o = neg_inf_half();
      continue;
    }
    float sum = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < NW; w2++) sum += partial[w2][r][y];
    const half_t prev = Epilogue::needs_prev(a.store) ? *o : (half_t)0;
    const half_t bias_x = Epilogue::needs_bias(a.store) ? a.bias[xcol] : (half_t)0;
    *o = ep.apply(sum, prev, bias_x);
  }
}

// Nine to thirty-two activation rows: matrix cores.  A workgroup owns 16 * RG weight rows, its
// wavefronts split K (wavefront w takes the 128-k macro steps w, w + NW, ...) and their partial
// sums meet in LDS, so every CU has work however few rows there are -- the tiled kernels put a
// 64 x 64 tile on N / 64 CUs and walk the whole of K on each.  v_mfma_f32_16x16x32_f16 with the
// weight rows as the A operand and a block of 16 activation rows as the B operand; lane (r, g)
// holds 8 consecutive k of row r for k-group g of either operand (which 32 k an instruction sums
// over is free as long as both operands agree).  MB blocks of 16 activation rows reuse the
// weight fragments, U macro steps are loaded per trip.  K % 128 == 0.
template <int NW, int RG, int MB, int U>
__global__ __launch_bounds__(NW * 64) void skinny_f16_mfma_kernel(MatmulArgs a) {
  constexpr int MACRO = 128;
  __shared__ float partial[NW][RG][MB][256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * RG);
  const int steps = a.k / MACRO;
  const half_t* wrow[RG];
#pragma unroll
  for (int q = 0; q < RG; q++)  // rows past n are clamped, their sums never stored
    wrow[q] = a.rhs + (int64_t)min(n0 + q * 16 + r, a.n - 1) * a.stride_rx + g * 8;
  const half_t* xrow[MB];
  bool xvalid[MB];
#pragma unroll
  for (int b = 0; b < MB; b++) {
    xvalid[b] = b * 16 + r < a.m;
    xrow[b] = a.lhs + (int64_t)min(b * 16 + r, a.m - 1) * a.stride_ly + g * 8;
  }
  float4_t acc[RG][MB];
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int b = 0; b < MB; b++) acc[q][b] = float4_t{0, 0, 0, 0};
  for (int ms0 = wave; ms0 < steps; ms0 += NW * U) {
    // every load of the trip (U macro steps) is issued before the first multiply; rows past m
    // read row m - 1 again, steps past K the last step, and are zeroed (a load under a lane
    // mask or a branch would be waited for on the spot)
    u32x4_t w[U][RG][4], x[U][MB][4];
    bool live[U];
#pragma unroll
    for (int u = 0; u < U; u++) {
      live[u] = ms0 + u * NW < steps;
      const int ms = live[u] ? ms0 + u * NW : steps - 1;
#pragma unroll
      for (int q = 0; q < RG; q++)
#pragma unroll
        for (int j = 0; j < 4; j++)
          w[u][q][j] = __builtin_nontemporal_load((const u32x4_t*)(wrow[q] + ms * MACRO + j * 32));
#pragma unroll
      for (int b = 0; b < MB; b++)
#pragma unroll
        for (int j = 0; j < 4; j++) x[u][b][j] = *(const u32x4_t*)(xrow[b] + ms * MACRO + j * 32);
    }
#pragma unroll
    for (int u = 0; u < U; u++)
#pragma unroll
      for (int b = 0; b < MB; b++)
#pragma unroll
        for (int j = 0; j < 4; j++) {
          const u32x4_t xz = (xvalid[b] && live[u]) ? x[u][b][j] : u32x4_t{0, 0, 0, 0};
          const half8_t xb = __builtin_bit_cast(half8_t, xz);
#pragma unroll
          for (int q = 0; q < RG; q++) {
            const u32x4_t wv = w[u][q][j];
            acc[q][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, wv), xb,
                                                               acc[q][b], 0, 0, 0);
          }
        }
  }
  // lane (r, g) holds sums of weight rows 4g .. 4g+3 against activation row r of the block
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int b = 0; b < MB; b++)
#pragma unroll
      for (int v = 0; v < 4; v++) partial[wave][q][b][(4 * g + v) * 16 + r] = acc[q][b][v];
  __syncthreads();
  const Epilogue ep{a.bias, a.beta, (half_t)a.scale, a.store, true};
  for (int e = tid; e < RG * MB * 256; e += NW * 64) {
    // consecutive threads -> consecutive output columns (weight rows)
    const int col = e % (16 * RG), y = e / (16 * RG);
    const int xcol = n0 + col;
    if (y >= a.m || xcol >= a.n) continue;
    half_t* o = a.output + (int64_t)y * a.stride_oy + (int64_t)xcol * a.stride_ox;
    if (a.mask == ADR_MASK_CAUSAL && xcol > y) {
      *o = neg_inf_half();
      continue;
    }
    float sum = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < NW; w2++) sum += partial[w2][col / 16][y / 16][(col % 16) * 16 + (y % 16)];
    const half_t prev = Epilogue::needs_prev(a.store) ? *o : (half_t)0;
    const half_t bias_x = Epilogue::needs_bias(a.store) ? a.bias[xcol] : (half_t)0;
    *o = ep.apply(sum, prev, bias_x);
  }
}

// MB blocks of up to sixteen activation rows, K = 128 * pieces with NW * (HS - 1) < pieces <=
// NW * HS (the wavefronts that have no piece in the last round read the last piece again against
// zeroed activations).  Weights and activations come in by global -> LDS DMA, four whole 256-byte
// row pieces per instruction (the register path above touches sixteen rows with 64 bytes each per
// instruction, which DRAM serves a third slower).  A wavefront owns HS macro steps x (MB blocks
// of activations + RG groups of sixteen weight rows) tiles of 4 KiB ([16 rows][16 chunks of 16
// bytes], chunk c of row r at position c ^ r so that fragment reads spread over all banks) and
// streams them through a private ring of RING tiles: nothing but its own vmcnt orders the DMA
// against its reads, and every outstanding load is one of the four DMA instructions of a tile.
#define ADR_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define ADR_GLB_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

template <int NW, int RG, int HS, int RING, int MB>
__global__ __launch_bounds__(NW * 64) void skinny_f16_ring_kernel(MatmulArgs a) {
  constexpr int TILE = 16 * 256, MACRO = 128;
  // the activations of a macro step travel through the ring as MB more tiles ahead of the
  // step's weight tiles (loaded straight into registers in MFMA layout they came as 64-byte
  // pieces from L2 and took sixteen registers per block and macro step: m=16 K11008 N4096
  // 27.7 us against 23.5)
  constexpr int PER = RG + MB;
  constexpr int UNITS = HS * PER;
  static_assert(RING <= UNITS && NW * MB * RG * 256 * 4 <= NW * RING * TILE, "partials reuse the ring");
  __shared__ __attribute__((aligned(1024))) unsigned char ring[NW * RING * TILE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, g = lane >> 4;
  const int n0 = blockIdx.x * (16 * RG);
  bool xvalid[MB];  // MB blocks of sixteen activation rows
#pragma unroll
  for (int b = 0; b < MB; b++) xvalid[b] = b * 16 + r < a.m;
  unsigned char* const mine = ring + wave * RING * TILE;
  const int pieces = a.k / MACRO;
  const bool last_valid = wave + (HS - 1) * NW < pieces;
  const int last_piece = min(wave + (HS - 1) * NW, pieces - 1);
  u32x4_t x[MB][4];  // the activations of the current macro step (rows past m read row m - 1
                     // and are zeroed when used)
  // DMA instruction i of a tile fills its chunks [64 i, 64 i + 64): rows 4i .. 4i+3
  auto issue = [&](int u) {  // tile u: macro step u / PER of the wavefront, then MB activation
                             // blocks and RG weight row groups in turn
    const int h = u / PER, q = u % PER - MB;  // q < 0: activation block q + MB
    const int piece = h == HS - 1 ? last_piece : wave + h * NW;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = 4 * i + (lane >> 4), kc = (lane & 15) ^ row;
      const half_t* src = (q < 0 ? a.lhs + (int64_t)min((q + MB) * 16 + row, a.m - 1) * a.stride_ly
                                 : a.rhs + (int64_t)min(n0 + q * 16 + row, a.n - 1) * a.stride_rx) +
                          (int64_t)piece * MACRO + kc * 8;
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(src),
                                       ADR_LDS_PTR(mine + (u % RING) * TILE + i * 1024), 16, 0, 0);
    }
  };
  int roff[4];  // fragment read j of the lane: logical chunk 4j + g of row r
#pragma unroll
  for (int j = 0; j < 4; j++) roff[j] = r * 256 + (((4 * j + g) ^ r) << 4);
  float4_t acc[MB][RG];
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int q = 0; q < RG; q++) acc[b][q] = float4_t{0, 0, 0, 0};
#pragma unroll
  for (int u = 0; u < RING; u++) issue(u);
#pragma unroll
  for (int u = 0; u < UNITS; u++) {
    // tiles u+1 .. min(u+RING-1, UNITS-1) may still be in flight: four DMA instructions each
    const int later = (u + RING - 1 < UNITS ? RING - 1 : UNITS - 1 - u) * 4;
    if (later == 12) __builtin_amdgcn_s_waitcnt(0x0F70 | 12);
    else if (later == 8) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
    else if (later == 4) __builtin_amdgcn_s_waitcnt(0x0F70 | 4);
    else __builtin_amdgcn_s_waitcnt(0x0F70 | 0);
    const int h = u / PER, q = u % PER - MB;
    const unsigned char* tile = mine + (u % RING) * TILE;
    u32x4_t w[4];
#pragma unroll
    for (int j = 0; j < 4; j++) w[j] = *(const u32x4_t*)(tile + roff[j]);
    // the tile is in registers before its slot is refilled
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    __builtin_amdgcn_sched_barrier(0);
    if (u + RING < UNITS) issue(u + RING);
    __builtin_amdgcn_sched_barrier(0);
    const u32x4_t z = {0, 0, 0, 0};
    if (q < 0) {  // the step's activations
#pragma unroll
      for (int j = 0; j < 4; j++) x[q < 0 ? q + MB : 0][j] = (h == HS - 1 && !last_valid) ? z : w[j];
      continue;
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const u32x4_t wv = w[j];
#pragma unroll
      for (int b = 0; b < MB; b++) {
        const u32x4_t xv = xvalid[b] ? x[b][j] : z;
        acc[b][q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
            __builtin_bit_cast(half8_t, wv), __builtin_bit_cast(half8_t, xv), acc[b][q], 0, 0, 0);
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
      for (int v = 0; v < 4; v++)
        partial[((wave * MB + b) * RG + q) * 256 + (4 * g + v) * 16 + r] = acc[b][q][v];
  __syncthreads();
  const Epilogue ep{a.bias, a.beta, (half_t)a.scale, a.store, true};
  for (int e = tid; e < MB * RG * 256; e += NW * 64) {
    const int col = e % (16 * RG), y = e / (16 * RG);  // consecutive threads -> consecutive columns
    const int xcol = n0 + col;
    if (y >= a.m || xcol >= a.n) continue;
    half_t* o = a.output + (int64_t)y * a.stride_oy + (int64_t)xcol * a.stride_ox;
    if (a.mask == ADR_MASK_CAUSAL && xcol > y) {
      *o = neg_inf_half();
      continue;
    }
    float sum = 0.0f;
#pragma unroll
    for (int w2 = 0; w2 < NW; w2++)
      sum += partial[((w2 * MB + y / 16) * RG + col / 16) * 256 + (col % 16) * 16 + y % 16];
    const half_t prev = Epilogue::needs_prev(a.store) ? *o : (half_t)0;
    const half_t bias_x = Epilogue::needs_bias(a.store) ? a.bias[xcol] : (half_t)0;
    *o = ep.apply(sum, prev, bias_x);
  }
}

template <int NW, int RG, int HS, int RING, int MB>
hipError_t launch_ring(hipStream_t stream, const MatmulArgs& a) {
  hipLaunchKernelGGL((skinny_f16_ring_kernel<NW, RG, HS, RING, MB>), dim3((a.n + 16 * RG - 1) / (16 * RG)),
                     dim3(NW * 64), 0, stream, a);
  return hipGetLastError();
}

template <int NW, int RG, int MB, int U>
hipError_t launch_skinny(hipStream_t stream, const MatmulArgs& a) {
  hipLaunchKernelGGL((skinny_f16_mfma_kernel<NW, RG, MB, U>), dim3((a.n + 16 * RG - 1) / (16 * RG)),
                     dim3(NW * 64), 0, stream, a);
  return hipGetLastError();
}

template <int MR, int NW, int RPB, int SEGW>
hipError_t launch(hipStream_t stream, const MatmulArgs& a) {
  hipLaunchKernelGGL((gemv_f16_dot_kernel<MR, NW, RPB, SEGW>), dim3((a.n + RPB - 1) / RPB),
                     dim3(NW * 64), 0, stream, a);
  return hipGetLastError();
}

// rows of activations the instantiation for m rows is built for
int rows_class(int m) { return m <= 1 ? 1 : m <= 2 ? 2 : m <= 4 ? 4 : 8; }

}  // namespace

static bool layout_ok(const MatmulArgs& a) {
  if (a.rhs_q || a.load != ADR_LOAD_IDENTITY || a.batches != 1) return false;
  if (a.stride_lx != 1 || a.stride_ry != 1) return false;
  if ((a.stride_ly | a.stride_rx) & 7) return false;
  if (a.lhs && (((uintptr_t)a.lhs | (uintptr_t)a.rhs) & 15)) return false;
  return true;
}

static bool dot_ok(const MatmulArgs& a) {
  // (the matrix-core kernels below take five rows and more where K allows)
  if (a.m < 1 || a.m > 8 || a.k % 8 != 0 || a.k < 512) return false;
  // worth it where the weight matrix is the traffic: at least 1 MiB of it
  if ((int64_t)a.n * a.k < (1 << 19)) return false;
  // segments the instantiations hold: 4 wavefronts x 2 or 8 x 3
  return (a.k + 511) / 512 <= 24;
}

static bool skinny_ok(const MatmulArgs& a) {
  // measured against the tiled kernels for 9..32 rows on N 4096..12288, K 4096 and 11008: never
  // slower (K11008 N4096 m=16: 27.5 against 65.9 us; K4096 N12288 m=32: 30.8 against 32.8);
  // from five rows on also ahead of the dot-product kernel (m=8, K4096 N12288: 21 against 24.9)
  if (a.k % 128 != 0 || a.k < 1024 || (int64_t)a.n * a.k < (1 << 22)) return false;
  if (a.m >= 5 && a.m <= 32) return true;
  // 33 to 64 rows: only the ring kernel, for the K classes built with three and four blocks
  const int hs = (a.k + 1023) / 1024;
  return a.m > 32 && a.m <= 64 && (hs == 4 || hs == 11);
}

enum SkinnyChoice { SKINNY_NONE, SKINNY_DOT, SKINNY_MFMA };

static SkinnyChoice choose_skinny(const MatmulArgs& a) {
  if (!layout_ok(a)) return SKINNY_NONE;
  // three and four rows on a matrix of at most 256 groups of 16 weight rows (one workgroup per
  // CU) and K up to 4096: the ring kernel is ahead already (m=4: K4096 N4096 9.4 -> 7.8 us, K2048
  // N4096 6.9 -> 5.6, K3072 N3072 7.0 -> 5.3; with N 6000 12.3 -> 13.0 and with K 11008 19.3 ->
  // 22.2, so not there; two rows: 7.7 either way)
  const int cus = device_info_for_plan().cus;  // MI355X: 256
  const bool narrow = a.m >= 3 && a.m <= 4 && a.n <= 16 * cus && a.k <= 4096 && a.k > 1024 &&
                      a.k % 128 == 0 && (int64_t)a.n * a.k >= (1 << 22);
  if (narrow) return SKINNY_MFMA;
  if (a.m <= 4 && dot_ok(a)) return SKINNY_DOT;
  if (skinny_ok(a)) return SKINNY_MFMA;
  return dot_ok(a) ? SKINNY_DOT : SKINNY_NONE;
}

bool gemv_f16_supported(const MatmulArgs& a, const char** name) {
  switch (choose_skinny(a)) {
    case SKINNY_DOT: *name = "gemv_f16_dot2_stream"; return true;
    case SKINNY_MFMA: *name = "skinny_f16_mfma16_splitk_lds"; return true;
    default: return false;
  }
}

hipError_t launch_gemv_f16(hipStream_t stream, const MatmulArgs& a) {
  if (choose_skinny(a) == SKINNY_MFMA) {
    // (one macro step per trip: two or three in flight per wavefront measured slower)
    // weight rows per workgroup: as few as still give (nearly) every CU a workgroup (N4096: 16
    // rows, 256 workgroups, K11008 m=16 27.2 us against 39.5 with 32 rows; N12288: 48 rows,
    // 25.7 against 28.7 with 16; N11008: 48 rows 25.2 against 31.7 with 32)
    const int cus = device_info_for_plan().cus;  // MI355X: 256
    const int rg = a.n >= 40 * cus ? 3 : a.n >= 24 * cus ? 2 : 1;
    // K in (1024 * (HS - 1), 1024 * HS] for the values of HS built here: weights, and the
    // activations with them, through the per-wavefront LDS ring (m=16, weights alone: K4096
    // N4096 12.4 -> 9.7 us, N11008 24.8 -> 20.3, N12288 25.9 -> 22.1; activations too: 9.9 ->
    // 8.7, 21.2 -> 19.7, 23.2 -> 21.9, K11008 N4096 27.7 -> 23.5)
    if (a.m <= 16) {
      switch ((a.k + 1023) / 1024) {
#define ADR_RING_CASE(HS)                                                         \
        case HS:                                                                  \
          if (rg == 3) return launch_ring<8, 3, HS, 4, 1>(stream, a);             \
          if (rg == 2) return launch_ring<8, 2, HS, 3, 1>(stream, a);             \
          return launch_ring<8, 1, HS, 4, 1>(stream, a);      
        ADR_RING_CASE(2) ADR_RING_CASE(3) ADR_RING_CASE(4) ADR_RING_CASE(5) ADR_RING_CASE(8)
        ADR_RING_CASE(11)
#undef ADR_RING_CASE
        default: break;
      }
    }
    // 33 to 64 rows, three and four blocks of activations, against the tiled kernels: K11008
    // N4096 m=33 46.3 -> 27.7 us, m=64 53.0 -> 34.1; K4096 N4096 13.8 -> 11.3, 14.4 -> 13.3; N12288
    // 25.7 -> 25.0, 29.0 -> 29.3
    if (a.m > 64) return hipErrorInvalidValue;  // (never chosen)
    if (a.m > 32) {
      switch ((a.k + 1023) / 1024) {
#define ADR_RING_CASE(HS)                                                                          \
        case HS:                                                                                   \
          if (a.m <= 48) {                                                                         \
            if (rg == 3) return launch_ring<8, 3, HS, 4, 3>(stream, a);                            \
            if (rg == 2) return launch_ring<8, 2, HS, 4, 3>(stream, a);                            \
            return launch_ring<8, 1, HS, 4, 3>(stream, a);                                         \
          }                                                                                        \
          if (rg == 3) return launch_ring<8, 3, HS, 4, 4>(stream, a);                              \
          if (rg == 2) return launch_ring<8, 2, HS, 4, 4>(stream, a);                              \
          return launch_ring<8, 1, HS, 4, 4>(stream, a);
        ADR_RING_CASE(4) ADR_RING_CASE(11)
#undef ADR_RING_CASE
        default: return hipErrorInvalidValue;
      }
    }
    // 17 to 32 rows: two blocks of activations (m=32, K4096, in registers: N4096 15.0 -> 13.6 us,
    // N11008 29.1 -> 24.6, N12288 30.8 -> 26.3)
    if (a.m > 16) {
      switch ((a.k + 1023) / 1024) {
#define ADR_RING_CASE(HS)                                                         \
        case HS:                                                                  \
          if (rg == 3) return launch_ring<8, 3, HS, 4, 2>(stream, a);             \
          if (rg == 2) return launch_ring<8, 2, HS, 4, 2>(stream, a);             \
          return launch_ring<8, 1, HS, 3, 2>(stream, a);      
        ADR_RING_CASE(2) ADR_RING_CASE(3) ADR_RING_CASE(4) ADR_RING_CASE(5) ADR_RING_CASE(8)
        ADR_RING_CASE(11)
#undef ADR_RING_CASE
        default: break;
      }
    }
    if (a.m <= 16) {
      if (rg == 3) return launch_skinny<8, 3, 1, 1>(stream, a);
      if (rg == 2) return launch_skinny<8, 2, 1, 1>(stream, a);
      return launch_skinny<8, 1, 1, 1>(stream, a);
    }
    if (rg == 3) return launch_skinny<8, 3, 2, 1>(stream, a);
    if (rg == 2) return launch_skinny<8, 2, 2, 1>(stream, a);
    return launch_skinny<8, 1, 2, 1>(stream, a);
  }
  const int nseg = (a.k + 511) / 512;
  const bool small = nseg <= 8;
  // Weight rows per workgroup: every workgroup fetches the activations of all m rows again
  // (from L2), so with eight rows a workgroup has to cover more weight rows to keep that
  // traffic below the weights' own (m=8, K4096 N12288: 32.3 us with two rows, 25.0 with eight).
  switch (rows_class(a.m)) {
    case 1: return small ? launch<1, 4, 4, 2>(stream, a) : launch<1, 8, 4, 3>(stream, a);
    case 2: return small ? launch<2, 4, 4, 2>(stream, a) : launch<2, 8, 4, 3>(stream, a);
    case 4: return small ? launch<4, 4, 4, 2>(stream, a) : launch<4, 8, 4, 3>(stream, a);
    default:
      if (!small) return launch<8, 8, 8, 3>(stream, a);
      return a.n >= 8192 ? launch<8, 4, 8, 2>(stream, a) : launch<8, 4, 4, 2>(stream, a);
  }
}

}  // namespace adr
