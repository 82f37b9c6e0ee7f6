// Fused attention for one layer: out = softmax(mask(scale * Q K^T) / temp) V per head, without
// the [heads, m, n] score tensor ever reaching memory.  It stands for the three launches at
// adrastea_models/src/llama.rs:541-554 (matmul_f16 with Scale + Causal, softmax_rows_inplace,
// matmul_f16), clip.rs:372-388 and whisper.rs:424-436, whose time on this part is the write and
// two reads of that tensor.  Scores and probabilities stay in fp32 registers (the three-launch
// path rounds both to fp16 in between), so results agree with that path to fp16 rounding, not
// bit for bit.
//
// One workgroup of four wavefronts takes 128 query rows of one head; each wavefront owns 32 of
// them.  Key and value rows stream through LDS in tiles of 64 by global -> LDS DMA, double
// buffered.  Per tile a wavefront computes S^T = K Q^T (MFMA 32x32x16, Q fragments resident in
// registers), so that every lane holds scores of ONE query row: the running maximum and sum are
// in-lane reductions plus one exchange with lane ^ 32.  The probabilities, narrowed to fp16,
// are already in the operand layout of the second product O^T = V^T P^T; its V^T fragments come
// from the row-major V tile by transposing LDS reads (ds_read_b64_tr_b16).
#include "adr_common.hpp"

namespace adr {

namespace {

#define ADR_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define ADR_GLB_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

struct AttnArgs {
  half_t* out;
  const half_t* q;
  const half_t* k;
  const half_t* v;
  int heads, m, n;  // query rows, key/value rows
  int so_y, so_z, sq_y, sq_z, sk_y, sk_z, sv_y, sv_z;  // element strides; the x strides are 1
  float c;          // scale * log2(e) / temperature
  uint32_t mask;
  int qblocks;      // ceil(m / 128)
};

// K tile: [64 rows][CPR 16-byte chunks]; chunk kc of row r sits at position kc ^ (line & 15)
// of its 256-byte line (16 lanes reading the same chunk of 16 consecutive rows hit 16
// different bank groups).
template <int CPR>
__device__ __forceinline__ int k_chunk_off(int row, int kc) {
  const int idx = row * CPR + kc, line = idx >> 4, pos = idx & 15;
  return ((line << 4) | (pos ^ (line & (CPR - 1)))) << 4;
}
template <int CPR>
__device__ __forceinline__ void k_chunk_inv(int phys, int& row, int& kc) {
  const int line = phys >> 4, pos = (phys & 15) ^ (line & (CPR - 1));
  const int idx = (line << 4) | pos;
  row = idx / CPR;
  kc = idx % CPR;
}
// V tile: [64 rows][CPR chunks], chunk c of row r at position c ^ v_swz(r): a transposing read
// touches 4 consecutive rows x 4 consecutive chunks per 32 lanes, and the XOR spreads those 16
// chunks over the 16 bank groups (rows of 128 bytes share a 256-byte line in pairs).
template <int CPR>
__device__ __forceinline__ int v_swz(int row) {
  return CPR == 16 ? ((row & 3) << 2) : (((row >> 1) & 1) << 2);
}

// Reductions over the lane pair (l, l ^ 32): v_permlane32_swap exchanges the upper half of one
// register with the lower half of the other, so with the same value in both its two results
// hold the pair's two values in every lane, without a trip through LDS.  The second result
// passes through an empty asm statement: without it the compiler folds a floating-point
// operation on the two results as if they were the same register.
__device__ __forceinline__ void pair_values(float v, float& x, float& y) {
  const uint32_t b = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  uint32_t r0 = r[0], r1 = r[1];
  asm volatile("" : "+v"(r1));
  x = __builtin_bit_cast(float, r0);
  y = __builtin_bit_cast(float, r1);
}
__device__ __forceinline__ float pair_max(float v) {
  float x, y;
  pair_values(v, x, y);
  return fmaxf(x, y);
}
__device__ __forceinline__ float pair_sum(float v) {
  float x, y;
  pair_values(v, x, y);
  return x + y;
}

template <int HD>
__global__ __launch_bounds__(256, 2) void attention_fwd_kernel(AttnArgs a) {
  constexpr int BM = 128, BN = 64, CPR = HD / 8;
  constexpr int TILE = BN * HD * 2;   // bytes of one K or V tile
  constexpr int NI = TILE / 1024 / 4; // DMA instructions per wavefront and tile
  constexpr int DS = HD / 16;         // MFMA k-steps over the head dimension
  constexpr int DT = HD / 32;         // 32-wide output column tiles
  constexpr int ROWB = HD * 2;        // bytes per tile row
  __shared__ __attribute__((aligned(1024))) unsigned char sK0[TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char sK1[TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char sV0[TILE];
  __shared__ __attribute__((aligned(1024))) unsigned char sV1[TILE];

  // (the wavefront index as a scalar: everything derived from it -- LDS stage addresses of the
  // transfers, role branches -- then stays out of the vector registers and the vector ALU)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 31, g = lane >> 5;
  const bool causal = a.mask == ADR_MASK_CAUSAL;

  // Workgroup -> (head, query block).  Consecutive workgroup ids go to different dies; die x takes
  // the heads [x * heads/8, (x+1) * heads/8), so that the query blocks of a head (which share K
  // and V) meet in one L2.  Under the causal mask block b has 2b + 2 key tiles.  A die's own
  // sequence runs through the upper half of the blocks downwards, then through the lower half
  // upwards: with 32 heads and 16 blocks all 64 workgroups of a die are resident at once, the
  // i-th and the (i+32)-th share a compute unit, and this order gives every unit a block b and
  // its complement 15 - b of the same head; with more work than fits, the heavy blocks start first.
  int head, qb;
  if (a.heads % 8 == 0 && a.qblocks % 2 == 0) {
    const int hx = a.heads >> 3, half = hx * (a.qblocks >> 1);
    const int x = blockIdx.x & 7, sq = blockIdx.x >> 3;
    const int j = sq < half ? sq : sq - half;
    head = x * hx + j % hx;
    qb = sq < half ? a.qblocks - 1 - j / hx : j / hx;
  } else {
    head = blockIdx.x / a.qblocks;
    qb = a.qblocks - 1 - blockIdx.x % a.qblocks;
  }
  const int q0 = qb * BM, q0w = q0 + wave * 32;

  const half_t* const Q = a.q + (int64_t)head * a.sq_z;
  const half_t* const K = a.k + (int64_t)head * a.sk_z;
  const half_t* const V = a.v + (int64_t)head * a.sv_z;

  int ntiles = (a.n + BN - 1) / BN;
  if (causal) ntiles = min(ntiles, (min(q0 + BM, a.m) - 1) / BN + 1);

  // DMA instruction i of this wavefront fills LDS chunks [(i*4 + wave)*64, +64) of a tile, lane
  // l the l-th of them; the lane fetches whatever (row, chunk) the swizzle puts there.
  int krow[NI], kcol[NI], vrow[NI], vcol[NI];
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int phys = (i * 4 + wave) * 64 + lane;
    int kc;
    k_chunk_inv<CPR>(phys, krow[i], kc);
    kcol[i] = kc * 8;
    vrow[i] = phys / CPR;
    vcol[i] = ((phys % CPR) ^ v_swz<CPR>(vrow[i])) * 8;
  }
  auto dma = [&](int tile, unsigned char* dK, unsigned char* dV) {
    const int kv0 = tile * BN;
#pragma unroll
    for (int i = 0; i < NI; i++) {
      // rows beyond the last are clamped to it; their scores are masked below
      const half_t* gk = K + (int64_t)min(kv0 + krow[i], a.n - 1) * a.sk_y + kcol[i];
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(gk), ADR_LDS_PTR(dK + (i * 4 + wave) * 1024),
                                       16, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < NI; i++) {
      const half_t* gv = V + (int64_t)min(kv0 + vrow[i], a.n - 1) * a.sv_y + vcol[i];
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(gv), ADR_LDS_PTR(dV + (i * 4 + wave) * 1024),
                                       16, 0, 0);
    }
  };

  // Q fragments (operand B of S^T = K Q^T): lane -> query row frow, head-dim group g
  half8_t qf[DS];
  {
    const half_t* qrow = Q + (int64_t)min(q0w + frow, a.m - 1) * a.sq_y + g * 8;
#pragma unroll
    for (int ds = 0; ds < DS; ds++) qf[ds] = *(const half8_t*)(qrow + ds * 16);
  }

  // LDS fragment offsets.  K: lane -> tile row frow (+32), chunk 2*ds + g.
  int offK[DS];
#pragma unroll
  for (int ds = 0; ds < DS; ds++) offK[ds] = k_chunk_off<CPR>(frow, ds * 2 + g);
  // V (transposing read): in each group of 16 lanes, lanes 4r..4r+3 address 16 consecutive
  // halves of tile row r, and lane i of the group receives column i of that 4 x 16 block.
  // Group b = (lane / 16) % 2 takes columns 16b.. of the 32-column tile, g the rows 4g..4g+3.
  int offV[DT];
  {
    const int s = lane & 15, b = (lane >> 4) & 1, r = s >> 2;
    const int row = 4 * g + r;  // + 32*kt + 16*t + 8*h, all multiples of 8: row & 3 == r
#pragma unroll
    for (int dt = 0; dt < DT; dt++) {
      const int chunk = 4 * dt + 2 * b + ((s & 3) >> 1);
      offV[dt] = row * ROWB + ((chunk ^ v_swz<CPR>(row)) << 4) + (s & 1) * 8;
    }
  }
  static_assert(CPR == 16 || CPR == 8, "head dimension 128 or 64");

  float16_t o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; dt++)
#pragma unroll
    for (int r = 0; r < 16; r++) o[dt][r] = 0.0f;
  float m_run = -1.0e30f, l_run = 0.0f;  // running maximum (log2 units) and this lane's sum

  auto tile_body = [&](int tile, const unsigned char* cK, const unsigned char* cV) {
    const int kv0 = tile * BN;
    if (causal && kv0 > q0w + 31) return;  // every score of this wavefront is masked
    // S^T tile: s[kt][4i+j] = score(query q0w + frow, key kv0 + 32kt + 8i + 4g + j)
    float16_t s[2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++) {
#pragma unroll
      for (int r = 0; r < 16; r++) s[kt][r] = 0.0f;
#pragma unroll
      for (int ds = 0; ds < DS; ds++) {
        const half8_t kf = *(const half8_t*)(cK + offK[ds] + kt * 32 * ROWB);
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[ds], s[kt], 0, 0, 0);
      }
    }
    const bool edge = (causal && kv0 + BN - 1 > q0w) || kv0 + BN > a.n;
    if (edge) {
      const int qi = q0w + frow;
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int r = 0; r < 16; r++) {
          const int kv = kv0 + 32 * kt + 8 * (r >> 2) + 4 * g + (r & 3);
          if (kv >= a.n || (causal && kv > qi)) s[kt][r] = -INFINITY;
        }
    }
    float mx = -1.0e30f;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) mx = fmaxf(mx, s[kt][r]);
    mx = pair_max(mx) * a.c;  // the row's maximum in log2 units (c > 0)
    // The exponent reference m_run follows the row maximum lazily: it moves only when some row
    // of the wavefront outgrew it by more than 2^8 (probabilities up to 256 are as exact in fp16
    // as those below 1), which after the first tiles is rare; the accumulator is rescaled only then.
    if (__builtin_amdgcn_ballot_w64(mx > m_run + 8.0f) != 0) {
      const float m_new = fmaxf(m_run, mx);
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      m_run = m_new;
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; dt++)
#pragma unroll
        for (int r = 0; r < 16; r++) o[dt][r] *= alpha;
    }
    float sum = 0.0f;
    half8_t pf[2][2];
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int r = 0; r < 16; r++) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[kt][r], a.c, -m_run));
        sum += p;
        pf[kt][r >> 3][r & 7] = (half_t)p;
      }
    l_run += sum;
    // O^T += V^T P^T: k-step (kt, t) covers keys 32kt + 16t + {4g + j, 8 + 4g + j}
    typedef short short4_t __attribute__((ext_vector_type(4)));
    typedef __attribute__((address_space(3))) short4_t lds_short4_t;
#pragma unroll
    for (int kt = 0; kt < 2; kt++)
#pragma unroll
      for (int t = 0; t < 2; t++)
#pragma unroll
        for (int dt = 0; dt < DT; dt++) {
          const unsigned char* p0 = cV + offV[dt] + (32 * kt + 16 * t) * ROWB;
          const short4_t lo =
              __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t*)ADR_LDS_PTR(p0));
          const short4_t hi =
              __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_t*)ADR_LDS_PTR(p0 + 8 * ROWB));
          const half8_t vf =
              __builtin_shufflevector(__builtin_bit_cast(half4_t, lo),
                                      __builtin_bit_cast(half4_t, hi), 0, 1, 2, 3, 4, 5, 6, 7);
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[kt][t], o[dt], 0, 0, 0);
        }
  };

  dma(0, sK0, sV0);
  for (int j = 0; j < ntiles; j += 2) {
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): tile j has landed
    __builtin_amdgcn_s_barrier();        // ... for every wavefront, and tile j-1 has been read
    if (j + 1 < ntiles) dma(j + 1, sK1, sV1);
    tile_body(j, sK0, sV0);
    if (j + 1 < ntiles) {
      __builtin_amdgcn_s_waitcnt(0x0070);
      __builtin_amdgcn_s_barrier();
      if (j + 2 < ntiles) dma(j + 2, sK0, sV0);
      tile_body(j + 1, sK1, sV1);
    }
  }

  // out[q][32dt + 8i + 4g + j] = o[dt][4i + j] / l
  const float l_tot = pair_sum(l_run);
  const float inv = 1.0f / l_tot;
  const int qi = q0w + frow;
  if (qi < a.m) {
    half_t* orow = a.out + (int64_t)head * a.so_z + (int64_t)qi * a.so_y + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; dt++)
#pragma unroll
      for (int i = 0; i < 4; i++) {
        half4_t r;
#pragma unroll
        for (int j = 0; j < 4; j++) r[j] = (half_t)(o[dt][4 * i + j] * inv);
        *(half4_t*)(orow + 32 * dt + 8 * i) = r;
      }
  }
}

}  // namespace

const char* attention_plan(int d) {
  return d == 128 ? "attention_fwd_mfma_128x64_d128" : d == 64 ? "attention_fwd_mfma_128x64_d64" : nullptr;
}

hipError_t launch_attention(hipStream_t stream, half_t* out, const half_t* q, const half_t* k,
                            const half_t* v, int heads, int m, int n, int d, int so_y, int so_z,
                            int sq_y, int sq_z, int sk_y, int sk_z, int sv_y, int sv_z, float scale,
                            float temp, uint32_t mask) {
  AttnArgs a;
  a.out = out; a.q = q; a.k = k; a.v = v;
  a.heads = heads; a.m = m; a.n = n;
  a.so_y = so_y; a.so_z = so_z; a.sq_y = sq_y; a.sq_z = sq_z;
  a.sk_y = sk_y; a.sk_z = sk_z; a.sv_y = sv_y; a.sv_z = sv_z;
  // the three-call sequence multiplies by the scale rounded to fp16 (matmul.cu:60-74)
  a.c = (float)(half_t)scale * 1.44269504088896340736f / temp;
  a.mask = mask;
  a.qblocks = (m + 127) / 128;
  const int64_t blocks = (int64_t)heads * a.qblocks;
  if (blocks > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  const dim3 grid((unsigned)blocks), block(256);
  if (d == 128)
    hipLaunchKernelGGL(attention_fwd_kernel<128>, grid, block, 0, stream, a);
  else
    hipLaunchKernelGGL(attention_fwd_kernel<64>, grid, block, 0, stream, a);
  return hipGetLastError();
}

}  // namespace adr
