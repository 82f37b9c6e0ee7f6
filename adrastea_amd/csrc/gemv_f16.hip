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

// Five to sixty-four activation rows (three and four on small matrices): matrix cores,
// v_mfma_f32_16x16x32_f16 with sixteen weight rows as the A operand and a block of sixteen
// activation rows as the B operand; lane (r, g) holds 8 consecutive k of row r for k-group g of
// either operand.  A workgroup owns 16 * RG weight rows and MB blocks of activation rows; its
// eight wavefronts split K -- wavefront w takes the 128-k macro steps w, w + 8, ... in a run-time
// loop, any K % 128 == 0 -- and their partial sums meet in LDS, so every CU has work however few
// rows there are (the tiled kernels put a 64 x 64 tile on N / 64 CUs and walk all of K on each).
// A step is MB tiles of activations and RG tiles of weights, 16 rows x 256 bytes each, requested
// into registers a fixed number of tiles ahead -- four instructions per tile, each bringing four
// whole 256-byte row pieces (a quarter of the wavefront per piece, which DRAM serves at its
// streaming rate; sixteen 64-byte pieces per instruction are served a third slower) -- then
// passed through a private 4 KiB LDS tile that turns the request layout into the operand layout
// (chunk c of row r at position c ^ r, conflict-free both ways).  Request addresses are a
// uniform base per step plus a 32-bit lane offset.  Activation rows past m read row m - 1 and
// weight rows past n row n - 1: every output depends on its own two rows only, and those outputs
// are not stored.  (Earlier forms: the same tiles by global -> LDS DMA through a per-wavefront
// ring, unrolled over the whole of K and built for six values of ceil(K / 1024) -- K11008 N4096
// m=16 22.7 us against 21.2 here, m=32 25.7 against 22.9 -- and fragments loaded straight into
// registers as sixteen 64-byte pieces per instruction, 27 us.)
template <int RG, int MB>
__global__ __launch_bounds__(512) void skinny_f16_regstream_kernel(MatmulArgs a) {
  constexpr int NW = 8, TILE = 16 * 256, MACRO = 128, PER = MB + RG;
  constexpr int DIST = PER - 1 < 3 ? PER - 1 : 3;  // tiles between a request and its use
  __shared__ __attribute__((aligned(1024))) unsigned char shuf[NW][TILE];
  __shared__ float partial[NW][MB][RG][256];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // (uniform: step addresses stay scalar)
  const int qa = lane >> 4, x = lane & 15;  // request role: quarter qa takes row 4i + qa, chunk x
  const int r = lane & 15, g = lane >> 4;   // operand role: row r, k-group g
  const int n0 = blockIdx.x * (16 * RG);
  const int steps = a.k / MACRO, last = steps - 1;
  unsigned char* const mine = shuf[wave];

  uint32_t xo[MB][4], wo[RG][4];
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int i = 0; i < 4; i++)
      xo[b][i] = (uint32_t)min(b * 16 + 4 * i + qa, a.m - 1) * (uint32_t)a.stride_ly * 2u + x * 16;
#pragma unroll
  for (int q = 0; q < RG; q++)
#pragma unroll
    for (int i = 0; i < 4; i++)
      wo[q][i] = (uint32_t)min(q * 16 + 4 * i + qa, a.n - 1 - n0) * (uint32_t)a.stride_rx * 2u + x * 16;
  const unsigned char* const xbase = (const unsigned char*)a.lhs;
  const unsigned char* const wbase = (const unsigned char*)(a.rhs + (int64_t)n0 * a.stride_rx);
  u32x4_t ld[PER][4];
  auto request = [&](int ms, int u) {  // tile u of macro step ms into its registers
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (u < MB)
        ld[u][i] = *(const u32x4_t*)(xbase + (int64_t)ms * (MACRO * 2) + xo[u][i]);
      else  // streaming load: a weight is read once per launch
        ld[u][i] = __builtin_nontemporal_load(
            (const u32x4_t*)(wbase + (int64_t)ms * (MACRO * 2) + wo[u - MB][i]));
    }
  };
#pragma unroll
  for (int u = 0; u < DIST; u++) request(min(wave, last), u);

  int woff[4], roff[4];
#pragma unroll
  for (int i = 0; i < 4; i++) woff[i] = (4 * i + qa) * 256 + ((x ^ (4 * i + qa)) << 4);
#pragma unroll
  for (int j = 0; j < 4; j++) roff[j] = r * 256 + (((4 * j + g) ^ r) << 4);  // chunk 4j + g of row r

  float4_t acc[MB][RG];
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int q = 0; q < RG; q++) acc[b][q] = float4_t{0, 0, 0, 0};
  half8_t xf[MB][4];  // activation operands of the step

#pragma unroll 1
  for (int ms = wave; ms < steps; ms += NW) {
    const int ms_next = min(ms + NW, last);  // (past the end: the last step again, never used)
#pragma unroll
    for (int u = 0; u < PER; u++) {
      __builtin_amdgcn_sched_barrier(0);
      if (u + DIST < PER) request(ms, u + DIST); else request(ms_next, u + DIST - PER);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 4; i++) *(u32x4_t*)(mine + woff[i]) = ld[u][i];
      if (u < MB) {
#pragma unroll
        for (int j = 0; j < 4; j++) xf[u][j] = *(const half8_t*)(mine + roff[j]);
      } else {
        const int q = u - MB;
        half8_t wf[4];
#pragma unroll
        for (int j = 0; j < 4; j++) wf[j] = *(const half8_t*)(mine + roff[j]);
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
          for (int b = 0; b < MB; b++)
            acc[b][q] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[j], xf[b][j], acc[b][q], 0, 0, 0);
      }
    }
  }

  // lane (r, g): acc[b][q][v] is weight row 4g + v of group q against activation row r of block b
#pragma unroll
  for (int b = 0; b < MB; b++)
#pragma unroll
    for (int q = 0; q < RG; q++)
#pragma unroll
      for (int v = 0; v < 4; v++) partial[wave][b][q][(4 * g + v) * 16 + r] = acc[b][q][v];
  // (not __syncthreads(): its fence would wait for the surplus requests of the last step)
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the partial sums are in LDS
  __builtin_amdgcn_s_barrier();
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
    for (int w2 = 0; w2 < NW; w2++) sum += partial[w2][y / 16][col / 16][(col % 16) * 16 + y % 16];
    const half_t prev = Epilogue::needs_prev(a.store) ? *o : (half_t)0;
    const half_t bias_x = Epilogue::needs_bias(a.store) ? a.bias[xcol] : (half_t)0;
    *o = ep.apply(sum, prev, bias_x);
  }
}

template <int RG, int MB>
hipError_t launch_regstream(hipStream_t stream, const MatmulArgs& a) {
  hipLaunchKernelGGL((skinny_f16_regstream_kernel<RG, MB>), dim3((a.n + 16 * RG - 1) / (16 * RG)),
                     dim3(512), 0, stream, a);
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
  // five to sixty-four rows, any K % 128 == 0: measured against the tiled kernels on N 1024..12288,
  // K 4096..13824, never slower (K11008 N4096 m=16: 21 against 66 us; K4096 N12288 m=32: 22.5
  // against 32.8); from five rows on also ahead of the dot-product kernel (m=8, K4096 N12288:
  // 20.5 against 24.9)
  if (a.k % 128 != 0 || a.k < 1024 || (int64_t)a.n * a.k < (1 << 22)) return false;
  // four blocks of activation rows leave room for two groups of weight rows per workgroup; on a
  // wide matrix every workgroup then re-reads more activations than weights and the tiled
  // kernels are ahead (K4096 N12288 m=64: 38.8 against 29 us; N8192 and narrower: 38.7 against
  // 42.4, 14.0 against 14.4, K11008 N4096 31.9 against 53)
  if (a.m > 48 && a.n >= 40 * device_info_for_plan().cus) return false;
  // the same from 33 rows on where K is short of 8192 (K5120 N13824 m=48: 31.4 against 42.9 us,
  // K4096 N32000: 57.5 against 66.1; K8192 N22016 stays: 78.2 against 82.1)
  if (a.m > 32 && a.n >= 40 * device_info_for_plan().cus && a.k < 8192) return false;
  // a short K splits badly over the eight wavefronts (ten steps: two rounds) and two blocks of
  // activation rows double what each step re-reads: from 17 rows on, K < 4096 and more than one
  // workgroup per CU the tiled kernels are ahead (weights from HBM; K1280 N51865 m=32: 43.3
  // against 29.9 us, K1024 N16384: 15.8 against 9.3, K2048 N8192 m=64: 15.9 against 13.4, m=32:
  // 12.3 against 12.0; N4096 stays: K1024 m=32 5.1 against 6.4)
  if (a.m > 16 && a.k < 4096 && a.n > 16 * device_info_for_plan().cus) return false;
  // (one to four rows: only where the dot-product kernel does not reach, K > 12288 --
  // K13824 N5120 m=4: 53 us on the tiled kernels, 33 here)
  return a.m >= 1 && a.m <= 64;
}

enum SkinnyChoice { SKINNY_NONE, SKINNY_DOT, SKINNY_MFMA };

static SkinnyChoice choose_skinny(const MatmulArgs& a) {
  if (!layout_ok(a)) return SKINNY_NONE;
  // One and two rows: dot products.  From three rows on the matrix cores wherever they apply: with
  // weights that come from HBM they are level with the dot products at K 4096, 8192 and 12288 and
  // well ahead where K fills the dot kernel's segments badly (m=4: K5120 N15360 41.5 -> 27.0 us,
  // K6656 N19968 57.0 -> 43.5, K5120 N5120 17.3 -> 12.4, K4096 N12288 20.4 -> 18.7, K11008 N4096
  // 19.4 -> 18.1).  (With the weights resident in the Infinity Cache the dot products had looked
  // ahead at three and four rows on wide matrices, 12.3 against 13.0 us at N 6000.)
  if (a.m <= 2 && dot_ok(a)) return SKINNY_DOT;
  if (skinny_ok(a)) return SKINNY_MFMA;
  return dot_ok(a) ? SKINNY_DOT : SKINNY_NONE;
}

bool gemv_f16_supported(const MatmulArgs& a, const char** name) {
  switch (choose_skinny(a)) {
    case SKINNY_DOT: *name = "gemv_f16_dot2_stream"; return true;
    case SKINNY_MFMA: *name = "skinny_f16_mfma16_regstream"; return true;
    default: return false;
  }
}

hipError_t launch_gemv_f16(hipStream_t stream, const MatmulArgs& a) {
  if (choose_skinny(a) == SKINNY_MFMA) {
    // Groups of 16 weight rows per workgroup (measured over K 4096 .. 22016, N 4096 .. 32000):
    // one where that gives at most one workgroup per CU (N4096: K11008 m=16 27.2 us against 39.5
    // with two); two where one would leave a second, mostly empty round (N5120: K13824 m=64 52
    // against 68 us); beyond that, with up to 16 activation rows, one again -- two workgroups fit a
    // CU then and many short ones balance best (N8192 m=16 27 against 34 us, N17920 m=8 44
    // against 52); with more activation rows a workgroup re-reads more activations than it
    // reads weights unless it owns three groups (N12288 m=32: 23.2 against 25.1 with one), or
    // two where three would leave a nearly empty last round (N13824: 288 workgroups).
    const int cus = device_info_for_plan().cus;  // MI355X: 256
    const int groups = (a.n + 15) / 16;
    int rg;
    if (groups <= cus) {
      rg = 1;
    } else if (groups <= 28 * cus / 16) {
      rg = 2;
    } else if (a.m <= 16) {
      rg = 1;
    } else {
      rg = a.n >= 40 * cus ? 3 : 2;
      const int w3 = (a.n + 47) / 48;
      if (rg == 3 && w3 > cus && w3 <= 2 * cus && w3 % cus <= cus / 4) rg = 2;
    }
    switch ((a.m + 15) / 16) {  // blocks of sixteen activation rows
#define ADR_REG_CASE(MB, RG3)                                            \
      case MB:                                                           \
        if (rg == 3) return launch_regstream<RG3, MB>(stream, a);        \
        if (rg == 2) return launch_regstream<2, MB>(stream, a);          \
        return launch_regstream<1, MB>(stream, a);
      // (four blocks against three row groups would not fit the register file)
      ADR_REG_CASE(1, 3) ADR_REG_CASE(2, 3) ADR_REG_CASE(3, 3) ADR_REG_CASE(4, 2)
#undef ADR_REG_CASE
      default: return hipErrorInvalidValue;  // (never chosen)
    }
  }
  const int nseg = (a.k + 511) / 512;
  const bool small = nseg <= 8;
  // Weight rows per workgroup: every workgroup fetches the activations of all m rows again
  // (from L2), so with eight rows a workgroup has to cover more weight rows to keep that
  // traffic below the weights' own (m=8, K4096 N12288: 32.3 us with two rows, 25.0 with eight).
  // One and two rows: a workgroup takes as long as its busiest wavefront, so five to sixteen
  // segments go to eight wavefronts with one or two each instead of 4 x 2 and 8 x 3 (weights from
  // HBM, m=1 / m=2: K5120 N13824 25.1 -> 22.8 / 28.4 -> 24.1 us, K5120 N5120 12.0 -> 10.5 / 13.4 ->
  // 11.8, K6656 N17920 37.2 -> 36.0 / 40.7 -> 37.3, K4096 N12288 17.0 -> 16.8 / 17.9 -> 17.1; up to
  // four segments the four wavefronts stay: K1280 N51864 27.4 against 27.7)
  if (a.m <= 2 && nseg > 4 && nseg <= 16) {
    if (a.m == 1) return small ? launch<1, 8, 4, 1>(stream, a) : launch<1, 8, 4, 2>(stream, a);
    return small ? launch<2, 8, 4, 1>(stream, a) : launch<2, 8, 4, 2>(stream, a);
  }
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
