// fp16 "NT" GEMM on the CDNA4 matrix cores: O[b,y,x] = store(sum_k L[b,y,k] * R[b,k,x]) for
// operands whose K dimension is contiguous in memory on BOTH sides (stride_lx == 1 and
// stride_ry == 1) and a row-major output (stride_ox == 1).  That covers every linear layer of
// the callers (weights arrive as W[N,K].permute([1,0]), adrastea_models/src/llama.rs:503-532)
// and the attention score product Q.K^T on the interleaved-head views of llama.rs:534-550.
// Row strides (stride_ly, stride_rx, stride_oy) and batch strides are free.
//
// The kernels share the tiling, the LDS layout and the epilogue:
//
//  gemm_nt_dma_kernel   K % 64 == 0, plain fp16 operands.  K slices of depth 64 go from global
//                       memory straight into LDS (global_load_lds_dwordx4, no register round
//                       trip) into statically separate LDS stages (three per operand, or two /
//                       three of the left and four of the right operand with the transfers split
//                       by wavefront role), so the loads of the next slices are in flight while
//                       the current slice feeds the MFMAs; one barrier per slice.  MFMA
//                       fragments are prefetched one k-step ahead and interleaved with the
//                       MFMAs by scheduling-group barriers.
//  gemm_nt_u8_kernel    the same with u8 weights dequantised on their way into LDS; its two small
//                       tiles can split K over groups of wavefronts inside the workgroup.
//  gemm_nt_shortk_kernel  K = 64 / 128 (the attention score product): persistent workgroups;
//                       also with the Load Scale operator (both operands scaled in fp16 on the
//                       way into the MFMAs) and for score rows that are not 16-byte aligned.
//  gemm_nn_anyrow_kernel  row-major x row-major products (P.V) whose left rows start at any even
//                       address and whose K is no multiple of 64 (sequence lengths like 77, 257,
//                       1500): left operand through registers, shifted into place.
//  gemm_nt_stage_kernel any K % 8 == 0, and the variants that must touch the data on the way
//                       in: u8 weights dequantised while staging (a K that is no multiple of 64,
//                       block sizes that are no power of two), and the Load Scale operator on
//                       other K.  Global -> registers -> LDS, two LDS stages.
//
// One workgroup owns a BM x BN output tile, WM x WN wavefronts each own a (BM/WM) x (BN/WN)
// sub-tile as fp32 accumulator blocks: 16 x 16 blocks of v_mfma_f32_16x16x32_f16 in the tiles
// with 256 rows or columns and the 128 x 128 tile (more flops within the part's power limit),
// 32 x 32 blocks of v_mfma_f32_32x32x16_f16 in the smaller ones.  LDS rows are XOR-swizzled at 16-byte granularity
// over 256-byte lines (64 banks) so that the 128-bit fragment reads of 16 consecutive rows are
// conflict-free (SQ_LDS_BANK_CONFLICT reads 0).  Accumulators are kept TRANSPOSED (the weight
// fragment is the first MFMA operand) so that a lane owns 4 consecutive output columns; the
// epilogue narrows them to fp16, transposes through a per-wavefront LDS slot and writes whole
// 16-byte chunks of output rows, applying the store operator, the bias and the causal mask on
// the way.
#include <stdint.h>
#include <type_traits>

#include "adr_common.hpp"

namespace adr {

namespace {

// MI355X has 8 accelerator dies (XCDs), each with its own L2; workgroup i is dispatched to die
// i % 8.  The count comes from the device query (TileMap::xcds).

#define ADR_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))
#define ADR_GLB_PTR(p) ((const __attribute__((address_space(1))) void*)(p))

// Physical byte offset of 16-byte chunk `kc` of row `row` in a [rows][CPR chunks] LDS tile.
// 16 chunks = one 256-byte line = all 64 banks; the chunk position inside a line is XORed
// with the line number.
template <int CPR>
__device__ __forceinline__ int lds_chunk_off(int row, int kc) {
  int idx = row * CPR + kc;
  int line = idx >> 4, pos = idx & 15;
  return ((line << 4) | (pos ^ (line & (CPR - 1)))) << 4;
}
// Inverse: which (row, kc) lives at physical chunk `phys`.
template <int CPR>
__device__ __forceinline__ void lds_chunk_inv(int phys, int& row, int& kc) {
  int line = phys >> 4, pos = (phys & 15) ^ (line & (CPR - 1));
  int idx = (line << 4) | pos;
  row = idx / CPR;
  kc = idx % CPR;
}

struct TileMap {
  int tiles_m, tiles_n, tiles_per_batch, total;
  int group_m;  // tile rows per L2-reuse group
  int xcds;     // dies of the device: workgroup i runs on die i % xcds
  int splits;   // K is cut into this many pieces, one workgroup each (1: no split)
};

// blockIdx.x -> (batch, tile_m, tile_n).  Consecutive ids land on different dies, so ids are
// first regrouped per die; inside a batch, tiles are walked column by column within groups of
// `group_m` tile rows so that the tiles resident on one die share A and B panels in its L2.
__device__ __forceinline__ void map_tile(const TileMap& map, int& batch, int& tile_m,
                                         int& tile_n, int id = blockIdx.x) {
  const int XCDS = map.xcds;
  const int per = (map.total + XCDS - 1) / XCDS;
  const int tall = map.total % XCDS == 0 ? XCDS : map.total % XCDS;
  const int xcd = id % XCDS, local = id / XCDS;
  id = xcd < tall ? xcd * per + local : tall * per + (xcd - tall) * (per - 1) + local;
  batch = id / map.tiles_per_batch;
  int t = id - batch * map.tiles_per_batch;
  const int group_span = map.group_m * map.tiles_n;
  const int g = t / group_span;
  const int gm0 = g * map.group_m;
  const int gsz = min(map.group_m, map.tiles_m - gm0);
  t -= g * group_span;
  tile_m = gm0 + t % gsz;
  tile_n = t / gsz;
}

__device__ __forceinline__ bool out_vectorizable(const MatmulArgs& a, const half_t* out) {
  // 16-byte row chunks need aligned rows; STORE_ACC_BETA with beta != 0 works on the fp32
  // accumulator and therefore stays on the element-wise path
  if ((a.stride_oy & 7) || ((uintptr_t)out & 15)) return false;
  if (Epilogue::needs_bias(a.store) && ((uintptr_t)a.bias & 15)) return false;
  if (a.store == STORE_ACC_BETA && a.beta != 0.0f) return false;
  return true;
}

// The store operator on 8 narrowed accumulators at once; the switch is taken once per chunk.
__device__ __forceinline__ half8_t apply_chunk(const MatmulArgs& a, const Epilogue& ep, half8_t v,
                                               half8_t prev, half8_t bias) {
  half8_t r = v;
  switch (a.store) {
    default:
    case ADR_STORE_IDENTITY:
      break;
    case ADR_STORE_SCALE:
      r = v * ep.hscale;
      break;
    case ADR_STORE_ADD:
      r = v + prev;
      break;
    case STORE_ACC_BETA:
      // beta == 0 on this path: acc + 0 * prev.  Non-finite garbage in the output poisons the
      // result exactly as in the reference; a finite one leaves the accumulator.
#pragma unroll
      for (int e = 0; e < 8; e++) {
        float t = 0.0f * (float)prev[e];
        r[e] = (t == t) ? v[e] : (half_t)t;
      }
      break;
    case ADR_STORE_BETA_BIAS:
    case ADR_STORE_QUICK_GELU_BIAS:
    case ADR_STORE_BETA_GELU_BIAS:
#pragma unroll
      for (int e = 0; e < 8; e++) r[e] = ep.apply_s16(v[e], prev[e], bias[e]);
      break;
  }
  return r;
}

// One chunk of 8 consecutive columns x..x+7 of output row y through the store operator, read and
// written W halves at a time: 8 where rows are 16-byte aligned, 4 or 2 where they are aligned to
// that many halves only (a score tensor whose row length is not a multiple of 8).
template <int W = 8>
__device__ __forceinline__ void store_chunk(const MatmulArgs& a, const Epilogue& ep, half_t* out,
                                            int y, int x, half8_t v) {
  typedef half_t piece_t __attribute__((ext_vector_type(W)));
  half_t* p = out + (int64_t)y * a.stride_oy + x;
  const bool full = x + 8 <= a.n;
  half8_t prev = {0, 0, 0, 0, 0, 0, 0, 0}, bias = {0, 0, 0, 0, 0, 0, 0, 0};
  if (full) {
    if (Epilogue::needs_prev(a.store)) {
#pragma unroll
      for (int q = 0; q < 8 / W; q++) {
        const piece_t t = *(const piece_t*)(p + q * W);
#pragma unroll
        for (int e = 0; e < W; e++) prev[q * W + e] = t[e];
      }
    }
    if (Epilogue::needs_bias(a.store)) bias = *(const half8_t*)(a.bias + x);
  } else {
#pragma unroll
    for (int e = 0; e < 8; e++) {
      if (x + e < a.n) {
        if (Epilogue::needs_prev(a.store)) prev[e] = p[e];
        if (Epilogue::needs_bias(a.store)) bias[e] = a.bias[x + e];
      }
    }
  }
  half8_t r = apply_chunk(a, ep, v, prev, bias);
  if (a.mask == ADR_MASK_CAUSAL && x + 7 > y) {
#pragma unroll
    for (int e = 0; e < 8; e++)
      if (x + e > y) r[e] = neg_inf_half();
  }
  if (full) {
#pragma unroll
    for (int q = 0; q < 8 / W; q++) {
      piece_t t;
#pragma unroll
      for (int e = 0; e < W; e++) t[e] = r[q * W + e];
      __builtin_nontemporal_store(t, (piece_t*)(p + q * W));
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; e++)
      if (x + e < a.n) p[e] = r[e];
  }
}

// store_chunk for output rows that start at any even address (a dense [M, N] result with an odd N,
// e.g. the 51865 logits of whisper.rs's decoder), for the store operators that do not read the
// output: the chunk goes out as a half, three dwords and a half (store8_any) instead of eight halves.
__device__ __forceinline__ void store_chunk_any(const MatmulArgs& a, const Epilogue& ep, half_t* out,
                                                int y, int x, half8_t v) {
  half_t* p = out + (int64_t)y * a.stride_oy + x;
  const bool full = x + 8 <= a.n;
  const half8_t prev = {0, 0, 0, 0, 0, 0, 0, 0};
  half8_t bias = {0, 0, 0, 0, 0, 0, 0, 0};
  if (Epilogue::needs_bias(a.store)) {
#pragma unroll
    for (int e = 0; e < 8; e++)
      if (x + e < a.n) bias[e] = a.bias[x + e];
  }
  half8_t r = apply_chunk(a, ep, v, prev, bias);
  if (a.mask == ADR_MASK_CAUSAL && x + 7 > y) {
#pragma unroll
    for (int e = 0; e < 8; e++)
      if (x + e > y) r[e] = neg_inf_half();
  }
  if (full) {
    store8_any(p, r);
  } else {
#pragma unroll
    for (int e = 0; e < 8; e++)
      if (x + e < a.n) p[e] = r[e];
  }
}

// Halves per access that every row chunk of the output (8 columns from a column that is a multiple
// of 8) is aligned to: 8, 4, 2, or 1 (element by element).  As out_vectorizable() for 8.
__device__ __forceinline__ int out_chunk_alignment(const MatmulArgs& a, const half_t* out) {
  if (Epilogue::needs_bias(a.store) && ((uintptr_t)a.bias & 15)) return 1;
  if (a.store == STORE_ACC_BETA && a.beta != 0.0f) return 1;
  const uintptr_t bits = (uintptr_t)a.stride_oy | (uintptr_t)a.stride_oz | ((uintptr_t)out >> 1);
  return (bits & 7) == 0 ? 8 : (bits & 3) == 0 ? 4 : (bits & 1) == 0 ? 2 : 1;
}

// Epilogue of one wavefront.  acc[i][j] is the TRANSPOSED 32x32 accumulator of row block i,
// column block j: lane l holds output row l % 32 and, in element r, column
// 8*(r/4) + 4*(l/32) + r%4.  (y0, x0) is the origin of the wavefront's sub-tile; `slot` is an
// LDS region private to this wavefront of at least 32 * (TN2*32 + 16) bytes.  TN2: the sub-tile's
// width in blocks of 16 columns (even for the 32x32x16 layout).
// The straight-line epilogue applies: the sub-tile begins inside the matrix and every 16-byte chunk
// of its rows lies wholly inside or wholly outside (all of them inside, or n a multiple of 8; rows
// and chunks past the matrix are read from the last row / chunk and not stored), it is on or below
// the diagonal of a causal product, rows are 16-byte aligned.
template <int TM, int TN2>
__device__ __forceinline__ bool epilogue_is_straight(const MatmulArgs& a, const half_t* out, int y0,
                                                     int x0) {
  const bool inside = y0 < a.m && x0 < a.n && (x0 + TN2 * 16 <= a.n || (a.n & 7) == 0);
  const bool unmasked = a.mask != ADR_MASK_CAUSAL || x0 + TN2 * 16 - 1 <= y0;
  return inside && unmasked && out_vectorizable(a, out);
}

// Accumulators of a wavefront's sub-tile come in two register layouts.  32x32x16 MFMA
// (float16_t acc[TM][TN2/2]): see above.  16x16x32 MFMA (float4_t acc[2*TM][TN2], transposed the
// same way): acc[i][j] is the 16 x 16 block of rows 16*i.., columns 16*j..; lane l holds output
// row l % 16 and, in element e, column 4*(l/16) + e.  The epilogues see both through these two
// helpers, which put 32-row block i of the sub-tile into the wavefront's LDS slot.
template <class T> struct is_mi16 { static constexpr bool value = false; };
template <int A, int B> struct is_mi16<float4_t[A][B]> { static constexpr bool value = true; };

// [32 rows][TN2*16 halves], PITCH bytes per row; `mul` multiplies when `scaled`
template <int TM, int TN2, class Acc>
__device__ __forceinline__ void stage_block_f16(Acc& acc, int i, unsigned char* slot, int lane,
                                                bool scaled, half_t mul) {
  constexpr int PITCH = TN2 * 32 + 16;
  if constexpr (is_mi16<Acc>::value) {
    const int lrow = lane & 15, g = lane >> 4;
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
      for (int j = 0; j < TN2; j++) {
        half4_t h;
#pragma unroll
        for (int e = 0; e < 4; e++) h[e] = (half_t)acc[2 * i + h2][j][e];
        *(half4_t*)(slot + (h2 * 16 + lrow) * PITCH + (j * 16 + 4 * g) * 2) = scaled ? h * mul : h;
      }
  } else {
    const int lrow = lane & 31, g = lane >> 5;
#pragma unroll
    for (int j = 0; j < TN2 / 2; j++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        half4_t h;
#pragma unroll
        for (int e = 0; e < 4; e++) h[e] = (half_t)acc[i][j][4 * q + e];
        *(half4_t*)(slot + lrow * PITCH + (j * 32 + 8 * q + 4 * g) * 2) = scaled ? h * mul : h;
      }
  }
}

// fp32: columns [qh*8*QN, +8*QN) of 32 x 32 block (i, j) as [32 rows][8*QN floats], FP bytes per row
template <int QN, class Acc>
__device__ __forceinline__ void stage_block_f32(Acc& acc, int i, int j, int qh, unsigned char* slot,
                                                int lane) {
  constexpr int FP = QN * 32 + 16;
  if constexpr (is_mi16<Acc>::value) {
    const int lrow = lane & 15, g = lane >> 4;
#pragma unroll
    for (int h2 = 0; h2 < 2; h2++)
#pragma unroll
      for (int jj = 0; jj < QN / 2; jj++)   // 16-column blocks staged at once: 2 (QN 4) or 1 (QN 2)
        *(float4_t*)(slot + (h2 * 16 + lrow) * FP + (jj * 16 + 4 * g) * 4) =
            acc[2 * i + h2][2 * j + (QN == 4 ? jj : qh)];
  } else {
    const int lrow = lane & 31, g = lane >> 5;
#pragma unroll
    for (int qq = 0; qq < QN; qq++) {
      const int q = qh * QN + qq;
      const float4_t v = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                          acc[i][j][4 * q + 3]};
      *(float4_t*)(slot + lrow * FP + (qq * 8 + 4 * g) * 4) = v;
    }
  }
}

// The straight-line epilogue for ONE store operator (OP is a compile-time constant: every
// operator gets its own compact instruction stream; with the operator switch inside the chunk
// loop the code of all of them, exp and tanh included, sat between any two stores, and the
// operators that are not Identity paid for it in instruction fetch).
template <int TM, int TN2, uint32_t OP, class Acc>
__device__ __forceinline__ void straight_epilogue(const MatmulArgs& a, half_t* out, Acc& acc, int y0,
                                                  int x0, unsigned char* slot, half_t hscale,
                                                  int lane) {
  constexpr bool plain_op = OP == ADR_STORE_IDENTITY || OP == ADR_STORE_SCALE;
  constexpr bool np = OP == ADR_STORE_ADD || OP == ADR_STORE_BETA_BIAS ||
                      OP == ADR_STORE_BETA_GELU_BIAS || OP == STORE_ACC_BETA;
  constexpr bool nb = OP == ADR_STORE_BETA_BIAS || OP == ADR_STORE_BETA_GELU_BIAS ||
                      OP == ADR_STORE_QUICK_GELU_BIAS;
  const Epilogue ep{a.bias, a.beta, hscale, OP, true};
  constexpr int PITCH = TN2 * 32 + 16;  // bytes per staged row (TN2*16 halves + pad)
  constexpr int CPW = TN2 * 2;          // 16-byte chunks per staged row
  const half_t mul = OP == ADR_STORE_SCALE ? hscale : (half_t)1.0f;
  // store round `it` of a 32-row block: lane -> 16-byte chunk it*64 + lane of the staged block
  // (scol: the chunk's first column, clamped to the last chunk of the matrix for the loads;
  // colin: the chunk lies inside the matrix)
  int rd[TN2], srow[TN2], scol[TN2];
  bool colin[TN2];
  const int cmax = a.n - 8 - x0;  // first column of the matrix's last chunk, relative to the sub-tile
#pragma unroll
  for (int it = 0; it < TN2; it++) {
    const int idx = it * 64 + lane, row = idx / CPW, c = idx % CPW;
    rd[it] = row * PITCH + c * 16;
    srow[it] = row;
    colin[it] = c * 8 <= cmax;
    scol[it] = min(c * 8, cmax);
  }
  half8_t bias[TN2];
  if (nb) {
#pragma unroll
    for (int it = 0; it < TN2; it++) bias[it] = *(const half8_t*)(a.bias + x0 + scol[it]);
  }
  half_t* const p0 = out + (int64_t)y0 * a.stride_oy + x0;
  const int last = a.m - y0 - 1;  // last row of the matrix, relative to the sub-tile
  // rows and chunks past the matrix are clamped for loads (so that no load sits under a lane
  // mask) and skipped for stores
  auto at = [&](int i, int it) {
    return p0 + (int64_t)min(i * 32 + srow[it], last) * a.stride_oy + scol[it];
  };
  // all of the sub-tile's previous output in one burst: with one workgroup per compute unit
  // nothing else hides this latency
  half8_t prev[TM][TN2];
  if (np) {
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int it = 0; it < TN2; it++) prev[i][it] = *(const half8_t*)at(i, it);
  }
#pragma unroll
  for (int i = 0; i < TM; i++) {
    // x * 1 is exact, so one multiply serves Identity and Scale (matmul.cu Scale: fp16
    // product); the other operators take the narrowed sum as it is
    stage_block_f16<TM, TN2>(acc, i, slot, lane, plain_op, mul);
#pragma unroll
    for (int it = 0; it < TN2; it++) {
      half8_t v = *(const half8_t*)(slot + rd[it]);
      if (OP == ADR_STORE_ADD) {
        v = v + prev[i][it];
      } else if (OP == STORE_ACC_BETA) {
        // beta == 0 on this path: acc + 0 * prev.  Non-finite garbage in the output poisons the
        // result exactly as in the reference; a finite one leaves the accumulator.
#pragma unroll
        for (int e = 0; e < 8; e++) {
          const float t = 0.0f * (float)prev[i][it][e];
          v[e] = (t == t) ? v[e] : (half_t)t;
        }
      } else if (!plain_op) {
#pragma unroll
        for (int e = 0; e < 8; e++)
          v[e] = ep.apply_s16(v[e], np ? prev[i][it][e] : (half_t)0, bias[it][e]);
      }
      // streaming store: the output is not read again by this launch and should not evict
      // operand panels from L2
      if (i * 32 + srow[it] <= last && colin[it]) __builtin_nontemporal_store(v, (half8_t*)at(i, it));
    }
  }
}

// acc + beta * out with beta != 0 (matmul_nt_wmma_16x128x256.cu:8-68 and its u8 twin: one rounding,
// of the fp32 sum): the straight-line form.  The fp32 accumulators pass through the wavefront's
// LDS slot, QN groups of eight columns of a 32 x 32 block at a time; a lane then owns whole
// 16-byte chunks of the output, whose previous values were all requested up front.  Same
// conditions as epilogue_is_straight, minus the restriction to beta == 0.
template <int TM, int TN2>
__device__ __forceinline__ bool acc_beta_is_straight(const MatmulArgs& a, const half_t* out, int y0,
                                                     int x0) {
  return a.store == STORE_ACC_BETA && a.beta != 0.0f && a.mask == ADR_MASK_NONE && y0 < a.m &&
         x0 < a.n && (x0 + TN2 * 16 <= a.n || (a.n & 7) == 0) && !(a.stride_oy & 7) &&
         !((uintptr_t)out & 15);
}

template <int TM, int TN2, class Acc>
__device__ __forceinline__ void straight_epilogue_acc_beta(const MatmulArgs& a, half_t* out, Acc& acc,
                                                           int y0, int x0, unsigned char* slot,
                                                           int lane) {
  // QN groups of eight columns at a time: a whole 32 x 32 block, or 16 columns where the sub-tile
  // is narrow or an odd number of 16-column blocks wide
  constexpr int QN = (TN2 >= 4 && TN2 % 2 == 0) ? 4 : 2;  // 32 rows x (QN * 32 + 16) bytes fit the slot
  constexpr int FP = QN * 32 + 16;        // bytes per staged row
  constexpr int G = TN2 * 2 / QN;         // column groups of the sub-tile
  constexpr int H = QN * 32 / 64;         // chunks per lane and group
  static_assert(32 * FP <= 32 * (TN2 * 32 + 16), "fp32 staging must fit the wavefront's slot");
  const int cmax = a.n - 8 - x0;          // first column of the matrix's last chunk, relative to the sub-tile
  const int last = a.m - y0 - 1;          // last row of the matrix, relative to the sub-tile
  half_t* const p0 = out + (int64_t)y0 * a.stride_oy + x0;
  int rrow[H], rcol[H];
#pragma unroll
  for (int h = 0; h < H; h++) {
    const int idx = h * 64 + lane;
    rrow[h] = idx / QN;
    rcol[h] = (idx % QN) * 8;
  }
  // rows and chunks past the matrix are clamped for the loads and skipped for the stores
  auto at = [&](int i, int g, int h) {
    return p0 + (int64_t)min(i * 32 + rrow[h], last) * a.stride_oy + min(g * QN * 8 + rcol[h], cmax);
  };
  half8_t prev[TM][G][H];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int g = 0; g < G; g++)
#pragma unroll
      for (int h = 0; h < H; h++) prev[i][g][h] = *(const half8_t*)at(i, g, h);
  const float beta = a.beta;
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int g = 0; g < G; g++) {
      stage_block_f32<QN>(acc, i, QN == 4 ? g : g >> 1, QN == 4 ? 0 : g & 1, slot, lane);
#pragma unroll
      for (int h = 0; h < H; h++) {
        const float4_t lo = *(const float4_t*)(slot + rrow[h] * FP + rcol[h] * 4);
        const float4_t hi = *(const float4_t*)(slot + rrow[h] * FP + rcol[h] * 4 + 16);
        half8_t v;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          v[e] = (half_t)(lo[e] + beta * (float)prev[i][g][h][e]);
          v[4 + e] = (half_t)(hi[e] + beta * (float)prev[i][g][h][4 + e]);
        }
        if (i * 32 + rrow[h] <= last && g * QN * 8 + rcol[h] <= cmax)
          __builtin_nontemporal_store(v, (half8_t*)at(i, g, h));
      }
    }
}

template <int TM, int TN2, class Acc>
__device__ __forceinline__ void wave_epilogue(const MatmulArgs& a, half_t* out, Acc& acc, int y0,
                                              int x0, unsigned char* slot, half_t hscale, int lane) {
  Epilogue ep{a.bias, a.beta, hscale, a.store, true};
  constexpr int PITCH = TN2 * 32 + 16;  // bytes per staged row (TN2*16 halves + pad)
  constexpr int CPW = TN2 * 2;          // 16-byte chunks per staged row
  if (acc_beta_is_straight<TM, TN2>(a, out, y0, x0))
    return straight_epilogue_acc_beta<TM, TN2>(a, out, acc, y0, x0, slot, lane);
  // Common case, straight-line: the sub-tile's columns lie inside the matrix, it is (for a
  // causal product) on or below the diagonal, rows are 16-byte aligned.
  if (epilogue_is_straight<TM, TN2>(a, out, y0, x0)) {
    switch (a.store) {
      case ADR_STORE_SCALE:
        return straight_epilogue<TM, TN2, ADR_STORE_SCALE>(a, out, acc, y0, x0, slot, hscale, lane);
      case ADR_STORE_ADD:
        return straight_epilogue<TM, TN2, ADR_STORE_ADD>(a, out, acc, y0, x0, slot, hscale, lane);
      case ADR_STORE_BETA_BIAS:
        return straight_epilogue<TM, TN2, ADR_STORE_BETA_BIAS>(a, out, acc, y0, x0, slot, hscale, lane);
      case ADR_STORE_QUICK_GELU_BIAS:
        return straight_epilogue<TM, TN2, ADR_STORE_QUICK_GELU_BIAS>(a, out, acc, y0, x0, slot, hscale, lane);
      case ADR_STORE_BETA_GELU_BIAS:
        return straight_epilogue<TM, TN2, ADR_STORE_BETA_GELU_BIAS>(a, out, acc, y0, x0, slot, hscale, lane);
      case STORE_ACC_BETA:
        return straight_epilogue<TM, TN2, STORE_ACC_BETA>(a, out, acc, y0, x0, slot, hscale, lane);
      default:
        return straight_epilogue<TM, TN2, ADR_STORE_IDENTITY>(a, out, acc, y0, x0, slot, hscale, lane);
    }
  }
  if (out_vectorizable(a, out)) {
#pragma unroll
    for (int i = 0; i < TM; i++) {
      stage_block_f16<TM, TN2>(acc, i, slot, lane, false, (half_t)1.0f);
#pragma unroll 1
      for (int it = 0; it < TN2; it++) {
        const int idx = it * 64 + lane;
        const int row = idx / CPW, c = idx % CPW;
        const half8_t v = *(const half8_t*)(slot + row * PITCH + c * 16);
        const int y = y0 + i * 32 + row, x = x0 + c * 8;
        if (y < a.m && x < a.n) store_chunk(a, ep, out, y, x, v);
      }
    }
  } else if (!Epilogue::needs_prev(a.store) && a.store != STORE_ACC_BETA) {
    // rows at any even address, nothing to read back: the same chunks, stored piecewise
#pragma unroll
    for (int i = 0; i < TM; i++) {
      stage_block_f16<TM, TN2>(acc, i, slot, lane, false, (half_t)1.0f);
#pragma unroll 1
      for (int it = 0; it < TN2; it++) {
        const int idx = it * 64 + lane;
        const int row = idx / CPW, c = idx % CPW;
        const half8_t v = *(const half8_t*)(slot + row * PITCH + c * 16);
        const int y = y0 + i * 32 + row, x = x0 + c * 8;
        if (y < a.m && x < a.n) store_chunk_any(a, ep, out, y, x, v);
      }
    }
  } else {
    // Element by element (unaligned or strided rows, or the fp32 form of acc + beta * out): the
    // fp32 accumulators pass through the wavefront's LDS slot, QN groups of eight columns of a
    // 32 x 32 block at a time, so that consecutive lanes store consecutive columns and the loop
    // over the elements needs no unrolling (a run-time index into the accumulator registers
    // would put them in scratch memory).
    const bool need_prev = Epilogue::needs_prev(a.store);
    const bool need_bias = Epilogue::needs_bias(a.store);
    const bool causal = a.mask == ADR_MASK_CAUSAL;
    constexpr int QN = (TN2 >= 4 && TN2 % 2 == 0) ? 4 : 2;  // 32 rows x (QN * 32 + 16) bytes fit the slot
    constexpr int FP = QN * 32 + 16;        // bytes per staged row
    static_assert(32 * FP <= 32 * PITCH, "fp32 staging must fit the wavefront's slot");
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int g = 0; g < TN2 * 2 / QN; g++) {
        stage_block_f32<QN>(acc, i, QN == 4 ? g : g >> 1, QN == 4 ? 0 : g & 1, slot, lane);
#pragma unroll 1
        for (int e = lane; e < 32 * 8 * QN; e += 64) {
          const int row = e / (8 * QN), c = e % (8 * QN);
          const int y = y0 + i * 32 + row, x = x0 + g * QN * 8 + c;
          if (y >= a.m || x >= a.n) continue;
          const float sum = *(const float*)(slot + row * FP + c * 4);
          half_t* p = out + (int64_t)y * a.stride_oy + x;
          if (causal && x > y) {
            *p = neg_inf_half();
          } else {
            half_t prev = need_prev ? *p : (half_t)0;
            half_t bias = need_bias ? a.bias[x] : (half_t)0;
            *p = ep.apply(sum, prev, bias);
          }
        }
      }
  }
}

// A tile that lies entirely above the diagonal of a causal product (every x > every y,
// matmul.cu:182-184) is -inf: written without any math.
template <int BM, int BN, int NT>
__device__ __forceinline__ void fill_masked_tile(const MatmulArgs& a, half_t* out, int m0, int n0,
                                                 int tid) {
  if (out_vectorizable(a, out)) {
    const half_t ninf = neg_inf_half();
    const half8_t v = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
    for (int e = tid; e < BM * BN / 8; e += NT) {
      const int y = m0 + e / (BN / 8), x = n0 + (e % (BN / 8)) * 8;
      if (y >= a.m || x >= a.n) continue;
      half_t* p = out + (int64_t)y * a.stride_oy + x;
      if (x + 8 <= a.n) {
        __builtin_nontemporal_store(v, (half8_t*)p);
      } else {
        for (int q = 0; x + q < a.n; q++) p[q] = ninf;
      }
    }
  } else {
    for (int e = tid; e < BM * BN; e += NT) {
      const int y = m0 + e / BN, x = n0 + e % BN;
      if (y < a.m && x < a.n) out[(int64_t)y * a.stride_oy + x] = neg_inf_half();
    }
  }
}

// =============================================================================================
// Direct-to-LDS kernel
// =============================================================================================
// SPLIT: the grid holds map.splits workgroups per tile, each multiplying its own piece of K and
// leaving the fp32 accumulators in a.workspace ([piece][tile][register chunk][thread] float4, so
// that consecutive threads store consecutive 16 bytes); splitk_reduce_kernel sums the pieces in
// a fixed order and runs the epilogue.
// MI16: v_mfma_f32_16x16x32_f16 instead of 32x32x16.  Same flops per clock, but on data that is
// not constant the part sustains 16 % more of them within its power limit (a bare loop on a
// 128 x 128 wavefront tile: 2070 against 1780 TFLOP/s; both 2460 on zeros).
template <int BM, int BN, int WM, int WN, int NSTAGE, int MINB, bool NN, int BK = 64, bool SPLIT = false,
          bool MI16 = false>
__global__ __launch_bounds__(WM* WN * 64, MINB) void gemm_nt_dma_kernel(MatmulArgs a,
                                                                         TileMap map) {
  // K slices of 64 (128 bytes of a row per slice and DMA request), or of 128 for the small tiles
  // of few-row products, which are bound by how DRAM serves those requests
  constexpr int MI = MI16 ? 16 : 32;           // rows (and columns) of one MFMA block
  constexpr int KG = 64 / MI;                  // 16-byte k-groups per k-step: lane / MI
  constexpr int CPR = BK / 8, KK = CPR / KG;   // k-steps per slice: of 16 k (32x32x16) or 32 k
  static_assert(BK == 64 || (BK == 128 && !NN && NSTAGE == 3), "slices of 64, or 128 with three stages");
  constexpr int NW = WM * WN, NT = NW * 64;
  // DMA instructions per thread and slice.  NSTAGE == 6 (two left + four right stages) and
  // NSTAGE == 7 (three left + four right): the first half of the wavefronts issues all transfers
  // of the left operand, the second half all of the right one (NWD each)
  constexpr int NWD = NSTAGE >= 6 ? NW / 2 : NW;
  constexpr int IA = BM * CPR / (NWD * 64), IB = BN * CPR / (NWD * 64);
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  constexpr int FM = WTM / MI, FN = WTN / MI;  // MFMA blocks of the wavefront's sub-tile
  constexpr int TN2 = WTN / 16;                // the sub-tile's width in 16-column blocks
  constexpr int SLOT = 32 * (TN2 * 32 + 16);
  static_assert(!MI16 || (!NN && !SPLIT), "16x16x32: plain NT products");
  static_assert(BM * CPR % (NWD * 64) == 0 && BN * CPR % (NWD * 64) == 0,
                "slices must split evenly over lanes");
  static_assert(WTM % 32 == 0 && WTN % (MI16 ? 16 : 32) == 0,
                "whole MFMA blocks (with 16x16x32 the sub-tile may be an odd number of them wide)");
  // epilogue slots: half of the wavefronts in each of the first two stages of the larger operand
  constexpr bool SLOTS_IN_B = BN > BM;
  // (per stage: half the wavefronts where they fit, else as many as fit, over three stages)
  constexpr int SLOT_STAGE = (SLOTS_IN_B ? BN : BM) * BK * 2;
  constexpr int SLOTS = (NW / 2) * SLOT <= SLOT_STAGE ? NW / 2 : SLOT_STAGE / SLOT;
  static_assert(SLOTS >= 1 && (NW + SLOTS - 1) / SLOTS <= (NSTAGE == 3 || (NSTAGE == 7 && !SLOTS_IN_B) ? 3 : 2),
                "epilogue slots must fit in the stage buffers");
  static_assert(NSTAGE == 2 || NSTAGE == 3 || NSTAGE == 6 || NSTAGE == 7,
                "2 or 3 LDS stages, or 6: two stages of the left and four of the right operand");
  static_assert(NSTAGE < 6 || (!NN && !SPLIT && NW % 2 == 0), "role split: plain NT products");
  static_assert(!NN || BN == 128, "the N-contiguous right operand is staged as [64][128] tiles");
  // Separate objects per stage: the compiler's alias analysis then knows that the asynchronous
  // LDS writes of one stage cannot touch the stage being read, and does not serialise them.
  __shared__ __attribute__((aligned(1024))) unsigned char sA0[BM * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sA1[BM * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sA2[NSTAGE == 3 || NSTAGE == 7 ? BM * BK * 2 : 1024];
  __shared__ __attribute__((aligned(1024))) unsigned char sB0[BN * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sB1[BN * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sB2[NSTAGE >= 3 ? BN * BK * 2 : 1024];
  __shared__ __attribute__((aligned(1024))) unsigned char sB3[NSTAGE >= 6 ? BN * BK * 2 : 1024];

  // Diagnostic build only (-DADR_PHASE_STAMPS, adrastea_amd.build.build_stamps_library, read by
  // bench.py --phase-stamps): every wavefront leaves the shader-clock and 100 MHz real-time
  // counters at its start, behind its prologue, behind its K loop and behind its stores in the
  // buffer passed as workspace ([workgroup][wavefront][10] 64-bit words).
#ifdef ADR_PHASE_STAMPS
  const uint64_t st_c0 = __builtin_readcyclecounter(), st_r0 = __builtin_amdgcn_s_memrealtime();
  uint64_t st_c1 = 0, st_r1 = 0, st_c2 = 0, st_r2 = 0;
#endif
  int batch, tile_m, tile_n;
  const int tile_id = SPLIT ? (int)(blockIdx.x % (unsigned)map.total) : (int)blockIdx.x;
  const int piece = SPLIT ? (int)(blockIdx.x / (unsigned)map.total) : 0;
  map_tile(map, batch, tile_m, tile_n, tile_id);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  // (the wavefront index as a scalar: everything derived from it -- LDS stage addresses of the
  // transfers, role branches -- then stays out of the vector registers and the vector ALU)
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  half_t* const out = a.output + (int64_t)batch * a.stride_oz;

  if (a.mask == ADR_MASK_CAUSAL && n0 > m0 + BM - 1) {
    // (split: the reduction kernel fills the tile; nothing is left in the workspace for it)
    if (!SPLIT) fill_masked_tile<BM, BN, NT>(a, out, m0, n0, tid);
    return;
  }

  // K slices of this workgroup: all of them, or piece `piece` of map.splits nearly equal ones
  const int KT_all = a.k / BK;
  const int kt_begin = SPLIT ? (int)((int64_t)KT_all * piece / map.splits) : 0;
  const int kt_end = SPLIT ? (int)((int64_t)KT_all * (piece + 1) / map.splits) : KT_all;
  const half_t* const A = a.lhs + (int64_t)batch * a.stride_lz + (int64_t)kt_begin * BK;
  const half_t* const B = a.rhs + (int64_t)batch * a.stride_rz +
                          (int64_t)kt_begin * (NN ? (int64_t)BK * a.stride_ry : BK);

  // DMA instruction i of this wavefront fills LDS chunks [(i*NW + wave)*64, +64) of a stage,
  // lane l the l-th of them; the lane fetches whatever (row, k-chunk) the swizzle puts there.
  // Rows beyond the matrix are clamped to the last row (their results are never stored).
  const int dwave = NSTAGE >= 6 ? wave % NWD : wave;  // index among the wavefronts issuing an operand
  const half_t* gA[IA];
  const half_t* gB[IB];
#pragma unroll
  for (int i = 0; i < IA; i++) {
    int row, kc;
    lds_chunk_inv<CPR>((i * NWD + dwave) * 64 + lane, row, kc);
    gA[i] = A + (int64_t)min(m0 + row, a.m - 1) * a.stride_ly + kc * 8;
  }
#pragma unroll
  for (int i = 0; i < IB; i++) {
    if (NN) {
      // right operand stored [k][n] (n contiguous): the stage is a [64 k][128 n] tile, one DMA
      // instruction brings 4 k-rows of 256 bytes; 16-byte chunk c of row k sits at position
      // c ^ ((k & 3) << 2) so that the transposing fragment reads spread over all banks
      const int krow = (i * NW + wave) * 4 + (lane >> 4);
      const int c = (lane & 15) ^ ((krow & 3) << 2);
      gB[i] = B + (int64_t)krow * a.stride_ry + min(n0 + c * 8, a.n - 8);
    } else {
      int row, kc;
      lds_chunk_inv<CPR>((i * NWD + dwave) * 64 + lane, row, kc);
      gB[i] = B + (int64_t)min(n0 + row, a.n - 1) * a.stride_rx + kc * 8;
    }
  }
  const int64_t b_slice = NN ? (int64_t)BK * a.stride_ry : BK;  // elements per K slice
  const int KT = kt_end - kt_begin;
  int kload = 0;  // next slice to fetch; past the end the last slice is fetched again (unused)
  auto dmaA = [&](int ks, unsigned char* dA) {
#pragma unroll
    for (int i = 0; i < IA; i++)
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(gA[i] + ks * BK),
                                       ADR_LDS_PTR(dA + (i * NWD + dwave) * 1024), 16, 0, 0);
  };
  auto dmaB = [&](int ks, unsigned char* dB) {
#pragma unroll
    for (int i = 0; i < IB; i++)
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(gB[i] + ks * b_slice),
                                       ADR_LDS_PTR(dB + (i * NWD + dwave) * 1024), 16, 0, 0);
  };
  auto dma = [&](unsigned char* dA, unsigned char* dB) {
    const int ks = min(kload, KT - 1);
    kload++;
    dmaA(ks, dA);
    dmaB(ks, dB);
  };

  typedef typename std::conditional<MI16, float4_t, float16_t>::type acc_t;
  acc_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < (MI16 ? 4 : 16); r++) acc[i][j][r] = 0.0f;

  // fragment addressing: lane -> (row = lane % MI, k-group = lane / MI), 8 halves = one chunk.
  // MI rows further down the chunk sits MI * CPR * 16 bytes further (a whole number of 256-byte
  // lines times 8: the swizzle does not change), so one offset per k-step serves all blocks.
  const int frow = lane & (MI - 1), fkg = lane / MI;
  constexpr int FSTEP = MI * CPR * 16;
  int offA[KK], offB[NN ? TN : 1][KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    offA[kk] = lds_chunk_off<CPR>(wm * WTM + frow, kk * KG + fkg);
#pragma unroll
    for (int j = 0; j < (NN ? TN : 1); j++) {
      if (NN) {
        // transposing read (ds_read_b64_tr_b16): inside each group of 16 lanes, lanes 4r..4r+3
        // address 16 consecutive halves of k-row r and lane i receives column i of that 4 x 16
        // block.  Group q = lane / 16 takes columns 16*(q%2).. of the 32-column block and
        // k-rows 8*(q/2).. of the k-step, so that lane l ends up with column l % 32 and
        // k-group l / 32, the MFMA operand layout.
        const int q = lane >> 4, r = (lane >> 2) & 3, jj = lane & 3;
        const int krow = kk * 16 + (q >> 1) * 8 + r;
        const int col = wn * WTN + j * 32 + 16 * (q & 1) + 4 * jj;
        offB[j][kk] = krow * 256 + ((((col >> 3) ^ ((krow & 3) << 2))) << 4) + (jj & 1) * 8;
      } else {
        offB[0][kk] = lds_chunk_off<CPR>(wn * WTN + frow, kk * KG + fkg);
      }
    }
  }

  half8_t fa[2][FM], fb[2][FN];
  auto load_frags = [&](int slot, const unsigned char* cA, const unsigned char* cB, int kk) {
#pragma unroll
    for (int i = 0; i < FM; i++) fa[slot][i] = *(const half8_t*)(cA + offA[kk] + i * FSTEP);
#pragma unroll
    for (int j = 0; j < FN; j++) {
      if (NN) {
        typedef short short4_t __attribute__((ext_vector_type(4)));
        typedef __attribute__((address_space(3))) short4_t lds_short4_t;
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4_t*)ADR_LDS_PTR(cB + offB[j][kk]));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4_t*)ADR_LDS_PTR(cB + offB[j][kk] + 4 * 256));  // k-rows + 4
        fb[slot][j] = __builtin_shufflevector(__builtin_bit_cast(half4_t, lo),
                                              __builtin_bit_cast(half4_t, hi), 0, 1, 2, 3, 4, 5, 6, 7);
      } else {
        fb[slot][j] = *(const half8_t*)(cB + offB[0][kk] + j * FSTEP);
      }
    }
  };
  auto mfmas = [&](int slot) {
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
      for (int j = 0; j < FN; j++) {
        if constexpr (MI16)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[slot][j], fa[slot][i], acc[i][j],
                                                             0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[slot][j], fa[slot][i], acc[i][j],
                                                             0, 0, 0);
      }
  };
  // MFMAs [lo, hi) of a k-step, in the order of mfmas()
  auto mfmas_range = [&](int slot, auto lo_tag, auto hi_tag) {
    constexpr int lo = decltype(lo_tag)::value, hi = decltype(hi_tag)::value;
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
      for (int j = 0; j < FN; j++) {
        if (i * FN + j < lo || i * FN + j >= hi) continue;
        if constexpr (MI16)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[slot][j], fa[slot][i], acc[i][j],
                                                             0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[slot][j], fa[slot][i], acc[i][j],
                                                             0, 0, 0);
      }
  };
  // s_waitcnt vmcnt(n) lgkmcnt(0): n outstanding DMA instructions may remain in flight
  auto wait_dma_barrier = [&](auto n_tag) {
    constexpr int n = decltype(n_tag)::value;
    __builtin_amdgcn_s_waitcnt(0x0070 | (n & 0xF) | ((n >> 4) << 14));
    __builtin_amdgcn_s_barrier();
  };
  constexpr int INFLIGHT = NSTAGE == 3 ? IA + IB : 0;
  // One K slice.  cur: stage being consumed (its k-step 0 fragments already sit in fragment
  // slot 0); nxt: the stage consumed next; (dA, dB): the stage the DMA issued here refills.
  auto slice = [&](const unsigned char* cA, const unsigned char* cB, const unsigned char* nA,
                   const unsigned char* nB, unsigned char* dA, unsigned char* dB) {
    // the DMA is issued in the first k-steps, one instruction per MFMA: sunk towards the wait
    // below, the whole global -> LDS latency would be exposed; issued as one burst, it would
    // hold up the MFMAs behind it
    dma(dA, dB);
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      if (kk + 1 < KK) {
        load_frags((kk + 1) & 1, cA, cB, kk + 1);
        mfmas(kk & 1);
        // interleave: LDS reads behind the first MFMAs of this k-step
        constexpr int READS = FM + (NN ? 2 * FN : FN);
        constexpr int PER = (READS + FM * FN - 1) / (FM * FN);
#pragma unroll
        for (int q = 0; q < FM * FN; q++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, PER, 0);
          if (kk * FM * FN + q < IA + IB) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
        }
      } else {
        mfmas(kk & 1);
      }
    }
    // the next stage has landed (only the DMA issued in this slice may still be in flight)
    // and every wavefront has left the current one
    wait_dma_barrier(std::integral_constant<int, INFLIGHT>{});
    load_frags(0, nA, nB, 0);
    __builtin_amdgcn_sched_barrier(0);
  };

  if constexpr (NSTAGE >= 6) {
    // Two (NSTAGE 6) or three (NSTAGE 7) stages of the left and four of the right operand, and two roles.  A wavefront's
    // transfers complete in the order it issued them, so a wavefront that issues both operands
    // cannot leave a right-operand slice in flight across the wait for the next left-operand
    // slice.  Here wavefronts 0 .. NW/2-1 issue every transfer of the left operand (slice kt+1 at
    // the head of slice kt, landed at its end) and the others every transfer of the right operand
    // (slice kt+3 at the head of slice kt; at its end slices kt+2 and kt+3 may still be in
    // flight): weights that no cache holds get three slices to arrive.  Each role has its own
    // instruction stream; both pass the same barriers.
    constexpr int SA = NSTAGE == 6 ? 2 : 3, SB = 4, P = NSTAGE == 6 ? 4 : 12;  // P: the stages' common period
    auto stA = [&](int i) -> unsigned char* { return i == 0 ? sA0 : i == 1 ? sA1 : sA2; };
    auto stB = [&](int i) -> unsigned char* { return i == 0 ? sB0 : i == 1 ? sB1 : i == 2 ? sB2 : sB3; };
    auto run = [&](auto role_tag) {
      constexpr bool LEFT = decltype(role_tag)::value;
      // (measured on the qkv product, same box, us with the weights rewritten by other launches in
      // between / multiplied again and again: the compiler's own choice, 38 of 48 behind the
      // barrier, 173 / 165; 4 or 8: 167 / 167; 12: 159 / 161; 16: 162 / 160; 20, 24: 162-164 / 162)
      // (the 256 x 128 tile with three left and four right stages: 4 behind the barrier o 58.6 us, 8
      // 57.2, 12 and 16 55.8; with three stages of both operands and every wavefront issuing both 57.4)
      constexpr int KEEP = 12;

      int kA = 0, kB = 0;
      auto slice6 = [&](const unsigned char* cA, const unsigned char* cB, const unsigned char* nA,
                        const unsigned char* nB, unsigned char* dA, unsigned char* dB) {
        if (LEFT) dmaA(min(kA++, KT - 1), dA); else dmaB(min(kB++, KT - 1), dB);
#pragma unroll
        for (int kk = 0; kk < KK; kk++) {
          if (kk + 1 < KK) {
            load_frags((kk + 1) & 1, cA, cB, kk + 1);
            mfmas(kk & 1);
#pragma unroll
            for (int q = 0; q < FM * FN; q++) {
              __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
              __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
              if (kk * FM * FN + q < (LEFT ? IA : IB)) __builtin_amdgcn_sched_group_barrier(0x010, 1, 0);
            }
          } else {
            // The slice's last MFMAs: all but KEEP of them in front of the wait and the barrier
            // (pinned: left to itself the compiler sinks most of the k-step behind the barrier,
            // and the wait for the left operand's transfers, issued at the head of this very
            // slice, then comes a few MFMAs after their issue), KEEP behind it, where they cover
            // the latency of the next slice's first fragment reads.
            mfmas_range(kk & 1, std::integral_constant<int, 0>{}, std::integral_constant<int, FM * FN - KEEP>{});
            __builtin_amdgcn_sched_barrier(0);
          }
        }
        wait_dma_barrier(std::integral_constant<int, LEFT ? (SA - 2) * IA : (SB - 2) * IB>{});
        load_frags(0, nA, nB, 0);
        mfmas_range((KK - 1) & 1, std::integral_constant<int, FM * FN - KEEP>{}, std::integral_constant<int, FM * FN>{});
#pragma unroll
        for (int q = 0; q < KEEP; q++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, (FM + FN + KEEP - 1) / KEEP, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      // slice kt (kt % P == p) reads stages p % SA and p % SB; the transfers issued at its head
      // refill the stages read one slice earlier: left slice kt + SA - 1, right slice kt + SB - 1
      auto slice_p = [&](int p) {
        slice6(stA(p % SA), stB(p % SB), stA((p + 1) % SA), stB((p + 1) % SB), stA((p + SA - 1) % SA),
               stB((p + SB - 1) % SB));
      };
      if (LEFT) {
#pragma unroll
        for (int i = 0; i < SA - 1; i++) dmaA(min(kA++, KT - 1), stA(i));
      } else {
#pragma unroll
        for (int i = 0; i < SB - 1; i++) dmaB(min(kB++, KT - 1), stB(i));
      }
      wait_dma_barrier(std::integral_constant<int, LEFT ? (SA - 2) * IA : (SB - 2) * IB>{});
      load_frags(0, sA0, sB0, 0);
#ifdef ADR_PHASE_STAMPS
      st_c1 = __builtin_readcyclecounter(); st_r1 = __builtin_amdgcn_s_memrealtime();
#endif
      int kt = 0;
      for (; kt + P <= KT; kt += P) {
#pragma unroll
        for (int p = 0; p < P; p++) slice_p(p);
      }
#pragma unroll
      for (int p = 0; p < P - 1; p++)
        if (kt < KT) { slice_p(p); kt++; }
    };
    if (__builtin_amdgcn_readfirstlane(wave) < NW / 2) run(std::true_type{}); else run(std::false_type{});
  } else if (NSTAGE == 3) {
    dma(sA0, sB0);
    dma(sA1, sB1);
    wait_dma_barrier(std::integral_constant<int, INFLIGHT>{});
    load_frags(0, sA0, sB0, 0);
#ifdef ADR_PHASE_STAMPS
    st_c1 = __builtin_readcyclecounter(); st_r1 = __builtin_amdgcn_s_memrealtime();
#endif
    int kt = 0;
    for (; kt + 3 <= KT; kt += 3) {
      slice(sA0, sB0, sA1, sB1, sA2, sB2);
      slice(sA1, sB1, sA2, sB2, sA0, sB0);
      slice(sA2, sB2, sA0, sB0, sA1, sB1);
    }
    if (kt < KT) { slice(sA0, sB0, sA1, sB1, sA2, sB2); kt++; }
    if (kt < KT) { slice(sA1, sB1, sA2, sB2, sA0, sB0); kt++; }
  } else {
    dma(sA0, sB0);
    wait_dma_barrier(std::integral_constant<int, 0>{});
    load_frags(0, sA0, sB0, 0);
    int kt = 0;
    for (; kt + 2 <= KT; kt += 2) {
      slice(sA0, sB0, sA1, sB1, sA1, sB1);
      slice(sA1, sB1, sA0, sB0, sA0, sB0);
    }
    if (kt < KT) slice(sA0, sB0, sA1, sB1, sA1, sB1);
  }
#ifdef ADR_PHASE_STAMPS
  st_c2 = __builtin_readcyclecounter(); st_r2 = __builtin_amdgcn_s_memrealtime();
#endif
  // drain the trailing (redundant) DMA before the stages are reused by the epilogue
  wait_dma_barrier(std::integral_constant<int, 0>{});

  if constexpr (SPLIT) {
    float4_t* const ws = (float4_t*)a.workspace +
                         ((int64_t)piece * map.total + tile_id) * (TM * TN * 4) * NT + tid;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const float4_t v = {acc[i][j][4 * c], acc[i][j][4 * c + 1], acc[i][j][4 * c + 2],
                              acc[i][j][4 * c + 3]};
          ws[(int64_t)((i * TN + j) * 4 + c) * NT] = v;
        }
    return;
  }
  unsigned char* slot;
  if constexpr ((NW + SLOTS - 1) / SLOTS <= 2)
    slot = SLOTS_IN_B ? (wave < SLOTS ? sB0 : sB1) : (wave < SLOTS ? sA0 : sA1);
  else
    slot = SLOTS_IN_B ? (wave < SLOTS ? sB0 : wave < 2 * SLOTS ? sB1 : sB2)
                      : (wave < SLOTS ? sA0 : wave < 2 * SLOTS ? sA1 : sA2);
  slot += (wave % SLOTS) * SLOT;
  wave_epilogue<TM, TN2>(a, out, acc, m0 + wm * WTM, n0 + wn * WTN, slot, (half_t)a.scale, lane);
#ifdef ADR_PHASE_STAMPS
  if (a.workspace && !SPLIT) {
    __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0): the tile is written
    const uint64_t st_c3 = __builtin_readcyclecounter(), st_r3 = __builtin_amdgcn_s_memrealtime();
    if (lane == 0) {
      uint64_t* st = (uint64_t*)a.workspace + ((int64_t)blockIdx.x * NW + wave) * 10;
      st[0] = st_c0; st[1] = st_c1; st[2] = st_c2; st[3] = st_c3;
      st[4] = st_r0; st[5] = st_r1; st[6] = st_r2; st[7] = st_r3;
      st[8] = __builtin_amdgcn_s_getreg((4 << 0) | (0 << 6) | (31 << 11));   // HW_ID
      st[9] = __builtin_amdgcn_s_getreg((20 << 0) | (0 << 6) | (31 << 11));  // XCC_ID
    }
  }
#endif
}

// Second launch of a split product: one workgroup per tile, with the geometry of the kernel that
// wrote the pieces.  Every thread sums its accumulator registers over the pieces (always in the
// order 0, 1, 2, ...: the result does not depend on which workgroup finished first) and the
// epilogue of the unsplit kernel stores the tile.
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(WM* WN * 64) void splitk_reduce_kernel(MatmulArgs a, TileMap map) {
  constexpr int NW = WM * WN, NT = NW * 64;
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  constexpr int SLOT = 32 * (TN * 64 + 16);
  __shared__ __attribute__((aligned(1024))) unsigned char slots[NW * SLOT];
  int batch, tile_m, tile_n;
  map_tile(map, batch, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  half_t* const out = a.output + (int64_t)batch * a.stride_oz;
  if (a.mask == ADR_MASK_CAUSAL && n0 > m0 + BM - 1) {
    fill_masked_tile<BM, BN, NT>(a, out, m0, n0, tid);
    return;
  }
  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;
  for (int piece = 0; piece < map.splits; piece++) {
    const float4_t* const ws = (const float4_t*)a.workspace +
                               ((int64_t)piece * map.total + blockIdx.x) * (TM * TN * 4) * NT + tid;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++)
#pragma unroll
        for (int c = 0; c < 4; c++) {
          const float4_t v = ws[(int64_t)((i * TN + j) * 4 + c) * NT];
#pragma unroll
          for (int e = 0; e < 4; e++) acc[i][j][4 * c + e] += v[e];
        }
  }
  wave_epilogue<TM, 2 * TN>(a, out, acc, m0 + wm * WTM, n0 + wn * WTN, slots + wave * SLOT,
                        (half_t)a.scale, lane);
}

// =============================================================================================
// Short-K persistent kernel (K == 64 or K == 128): QK^T-shaped products
// =============================================================================================
// With one or two K slices a tile is all load latency and epilogue, and the job is bound by the
// output writes.  One workgroup per CU walks segments of tile rows (128 x 128 tiles).  The left
// panel of a segment is copied from LDS into registers once, the right panels stream through a
// ring of three LDS buffers, and the twelve wavefronts have four roles:
//   0..3   upper group: rows 0..63 of every tile, 32 columns each;
//   4..7   lower group: rows 64..127.  A group alternates between multiplying its half of a tile
//          (32 MFMAs of 16x16x32 per wavefront, eight independent accumulators) and narrowing the result into its half of a 128 x 128 fp16
//          staging tile in LDS; the two groups run half a tile apart, so that while one
//          multiplies the other narrows, and the matrix pipes see a multiplying wavefront all the time;
//   8..9   write: read a staged half tile as whole 256-byte rows, apply the store operator,
//          issue the global stores.  Output writes stall the wavefront that issues them, so
//          they come from wavefronts that feed nothing else;
//   10..11 load: keep the DMA two tiles ahead and wait for it.  A wavefront's memory counter
//          covers its loads and stores alike, which is why loading and writing are not combined.
// One barrier per half tile.  Between barrier p and barrier p+1 (phase p), with tile j = p / 2:
//   even p: upper multiplies tile j        | lower narrows tile j-1 | writers: upper half of j-1
//   odd p:  upper narrows tile j           | lower multiplies tile j | writers: lower half of j-1
// A workgroup with T tiles passes 2T + 2 barriers in every role.  The right panel of tile j is read
// in phases 2j and 2j+1 and its buffer refilled (tile j+3) in phase 2j+2.  Both groups copy the
// left panel of a new segment in the even phase of its first tile (the lower group's registers
// are free by then), and the loader refills that buffer for the next segment one phase later.
struct ShortKMap {
  int tiles_m, tiles_n, rows;   // rows = batches * tiles_m
  int seg, segs_per_row, units; // a unit is `seg` consecutive tiles of one tile row
  int xcds;                     // dies of the device
  int prefilled;                // the tiles above the diagonal of a causal product are written
};

// The 128-column tiles that lie entirely above the diagonal of a causal product, as whole runs
// of a row (one wavefront per row): -inf without any arithmetic (matmul.cu:182-184).  Runs of up
// to a whole row are what the memory likes best; the same bytes written tile by tile from inside
// the persistent kernel hold up its barriers.
__global__ __launch_bounds__(256) void fill_causal_rows_kernel(MatmulArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);  // row, over all batches
  if (r >= (int64_t)a.batches * a.m) return;
  const int batch = (int)(r / a.m), y = (int)(r - (int64_t)batch * a.m);
  const int x0 = (y / 128 + 1) * 128;  // first column right of the tile that holds the diagonal
  half_t* const out = a.output + (int64_t)batch * a.stride_oz;
  half_t* const row = out + (int64_t)y * a.stride_oy;
  const half_t ninf = neg_inf_half();
  const half8_t v = {ninf, ninf, ninf, ninf, ninf, ninf, ninf, ninf};
  const bool aligned = out_vectorizable(a, out);
  for (int x = x0 + lane * 8; x < a.n; x += 512) {
    if (x + 8 <= a.n) {
      if (aligned) __builtin_nontemporal_store(v, (half8_t*)(row + x));
      else store8_any(row + x, v);
    } else {
      for (int q = 0; x + q < a.n; q++) row[x + q] = ninf;
    }
  }
}

// (four writers instead of two leave the multiplying wavefronts 128 registers, nine short, and
// measure the same: the stores wait for the memory, not for wavefronts to issue them)
constexpr int SHORTK_WRITERS = 2, SHORTK_LOADERS = 2;
constexpr int SHORTK_THREADS = (8 + SHORTK_WRITERS + SHORTK_LOADERS) * 64;

template <int N>
__device__ __forceinline__ void wait_vmcnt_at_most() {
  static_assert(N >= 0 && N < 64, "vmcnt is a six-bit counter");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

template <int CPR>  // 16-byte chunks per row: 8 (K = 64) or 16 (K = 128)
__global__ __launch_bounds__(SHORTK_THREADS, 1) void gemm_nt_shortk_kernel(MatmulArgs a,
                                                                           ShortKMap map) {
  constexpr int BM = 128, BN = 128, NWL = SHORTK_LOADERS, NWW = SHORTK_WRITERS;
  constexpr int WROWS = 64 / NWW, WIT = WROWS / 4;  // rows and read rounds of a writer per half tile
  constexpr int RING = 3;
  constexpr int IT = BM * CPR / (NWL * 64);    // DMA instructions per loader lane and panel
  constexpr int ROWS_PER_I = NWL * 64 / CPR;   // rows between a lane's successive instructions
  constexpr int PANEL = BM * CPR * 16;         // bytes of one 128-row panel
  static_assert(3 * IT < 64, "three panels in flight must fit the memory counter");
  __shared__ __attribute__((aligned(1024))) unsigned char sA[PANEL];
  __shared__ __attribute__((aligned(1024))) unsigned char sB[RING * PANEL];
  // staging tile: row r = 256 bytes, 16-byte chunk c at position c ^ (r & 15)
  __shared__ __attribute__((aligned(1024))) unsigned char sC[BM * BN * 2];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int G = gridDim.x;
  // Workgroup g runs on die g % 8: the workgroups of a die take neighbouring units (they share
  // right panels in the die's L2).  Odd rounds walk the workgroups backwards, which pairs long
  // and short rows of a causal product.
  const int XCDS = map.xcds;
  const int gl = G % XCDS == 0 ? (blockIdx.x % XCDS) * (G / XCDS) + blockIdx.x / XCDS : blockIdx.x;

  // Cursor over this workgroup's units and the tiles in them, in processing order.
  struct Cursor {
    int t, unit, batch, m0, n, n_end, n_vis_end;  // tiles [n, n_vis_end) computed, [.., n_end) filled
    bool valid, first;                            // first: no earlier computed tile in this unit
  };
  auto load_unit = [&](Cursor& c) {
    c.unit = c.t * G + ((c.t & 1) ? G - 1 - gl : gl);
    if (c.unit >= map.units) { c.valid = false; return; }
    const int row = c.unit / map.segs_per_row, sg = c.unit - row * map.segs_per_row;
    c.batch = row / map.tiles_m;
    c.m0 = (row - c.batch * map.tiles_m) * BM;
    c.n = sg * map.seg;
    c.n_end = min(c.n + map.seg, map.tiles_n);
    // tiles with n0 > m0 + BM - 1 of a causal product are all -inf
    const int vis = a.mask == ADR_MASK_CAUSAL ? (c.m0 + BM - 1) / BN + 1 : map.tiles_n;
    c.n_vis_end = min(c.n_end, vis);
    c.valid = true;
  };
  // first / next tile that is computed (units without one are skipped)
  auto first_item = [&](Cursor& c) {
    c.t = 0;
    load_unit(c);
    while (c.valid && c.n >= c.n_vis_end) { c.t++; load_unit(c); }
    c.first = true;
  };
  auto next_item = [&](Cursor& c) {
    c.n++;
    c.first = false;
    while (c.valid && c.n >= c.n_vis_end) { c.t++; load_unit(c); c.first = true; }
  };

  if (wave >= 8 + NWW) {
    // ---------------------------------------------------------------- loader wavefronts
    const int lw = wave - 8 - NWW;
    // The lane's place in DMA instruction 0.  Instruction i fills the 256-byte lines 4 * NWL * i
    // further down: the row moves with it, and the chunk by what those lines add to the swizzle.
    int drow, dkc;
    lds_chunk_inv<CPR>(lw * 64 + lane, drow, dkc);
    auto panel = [&](const half_t* base, int64_t row_stride, int r0, int rmax, unsigned char* dst) {
#pragma unroll
      for (int i = 0; i < IT; i++) {
        const int row = drow + i * ROWS_PER_I;
        const int kc = dkc ^ ((i * NWL * 4) & (CPR - 1));
        __builtin_amdgcn_global_load_lds(
            ADR_GLB_PTR(base + (int64_t)min(r0 + row, rmax) * row_stride + kc * 8),
            ADR_LDS_PTR(dst + (i * NWL + lw) * 1024), 16, 0, 0);
      }
    };
    Cursor cur;  // tile of the current phase
    first_item(cur);
    if (!cur.valid) return;
    // Panels are issued as groups of IT instructions; a group has landed once at most the
    // groups issued after it are outstanding.  `age` counts, one byte each, the groups issued
    // after the right panel in ring buffer 0, 1, 2 and after the youngest left panel (a buffer
    // is refilled every third right panel, so the counts stay small).  Kept in one register on
    // purpose: three variables picked by the buffer number end up in scratch memory, and a load
    // from there waits for every DMA in flight.
    uint32_t age = 0;
    int right_issued = 0;
    Cursor is = cur;  // next right panel to issue
    auto issued_into = [&](int byte) { age = (age + 0x01010101u) & ~(0xFFu << (8 * byte)); };
    auto younger_than = [&](int byte) { return (int)((age >> (8 * byte)) & 0xFFu); };
    auto issue_left = [&](const Cursor& c) {
      panel(a.lhs + (int64_t)c.batch * a.stride_lz, a.stride_ly, c.m0, a.m - 1, sA);
      issued_into(3);
    };
    auto issue_right = [&]() {
      if (!is.valid) return;
      const int slot = right_issued % RING;
      panel(a.rhs + (int64_t)is.batch * a.stride_rz, a.stride_rx, is.n * BN, a.n - 1,
            sB + slot * PANEL);
      issued_into(slot);
      right_issued++;
      next_item(is);
    };
    auto wait_landed = [&](int younger) {
      if (younger <= 0) wait_vmcnt_at_most<0>();
      else if (younger == 1) wait_vmcnt_at_most<IT>();
      else if (younger == 2) wait_vmcnt_at_most<2 * IT>();
      else wait_vmcnt_at_most<3 * IT>();
    };
    issue_left(cur);
    for (int k = 0; k < RING; k++) issue_right();
    wait_landed(min(younger_than(3), younger_than(0)));
    __builtin_amdgcn_s_barrier();  // barrier 0
    for (int p = 0;; p++) {
      const int j = p >> 1;
      if (p & 1) {
        // both groups copied the left panel of this unit in phase 2j: the next unit's may come
        if (cur.first) {
          Cursor nu = cur;
          do { next_item(nu); } while (nu.valid && !nu.first);
          if (nu.valid) issue_left(nu);
        }
        next_item(cur);  // tile j+1 starts after the next barrier
        if (cur.valid) {
          const int y = younger_than((j + 1) % RING);
          wait_landed(cur.first ? min(y, younger_than(3)) : y);
        }
        __builtin_amdgcn_s_barrier();  // barrier 2j+2
      } else {
        if (j >= 1) issue_right();  // tile j+2, into the buffer of tile j-1
        __builtin_amdgcn_s_barrier();  // barrier 2j+1
        if (!cur.valid) break;         // that was barrier 2T+1
      }
    }
    return;
  }

  if (wave >= 8) {
    // ---------------------------------------------------------------- writer wavefronts
    const int sw = wave - 8;                       // rows sw*WROWS .. of a half tile
    const int rrow = lane >> 4, rc = lane & 15;    // read round it: row it*4 + rrow, chunk rc
    const half_t hscale = (half_t)a.scale;
    Epilogue ep{a.bias, a.beta, hscale, a.store, true};
    const int walign = out_chunk_alignment(a, a.output);
    const bool vec = walign >= 2;
    // (Identity and Scale need neither the previous output nor the bias: any alignment)
    const bool plain = a.store == ADR_STORE_IDENTITY || a.store == ADR_STORE_SCALE;
    const half_t mul = a.store == ADR_STORE_SCALE ? hscale : (half_t)1.0f;
    auto write_half = [&](int batch, int m0, int n0, int half) {
      const int r0 = half * 64 + sw * WROWS;  // first of this wavefront's rows in the tile
      auto staged = [&](int it) {
        const int row = r0 + it * 4 + rrow;
        return *(const half8_t*)(sC + row * 256 + ((rc ^ (row & 15)) << 4));
      };
      half_t* const out = a.output + (int64_t)batch * a.stride_oz;
      const int y0 = m0 + r0 + rrow, x = n0 + rc * 8;
      const bool inside = m0 + r0 + WROWS <= a.m && n0 + BN <= a.n;
      const bool unmasked = a.mask != ADR_MASK_CAUSAL || n0 + BN - 1 <= m0 + r0;
      if (plain && unmasked) {
        half8_t v[WIT];
#pragma unroll
        for (int it = 0; it < WIT; it++) v[it] = staged(it);
        // x * 1 is exact: one multiply serves Identity and Scale (fp16 product, matmul.cu)
        half_t* const p = out + (int64_t)y0 * a.stride_oy + x;
        if (inside && walign == 8) {
#pragma unroll
          for (int it = 0; it < WIT; it++)
            __builtin_nontemporal_store(v[it] * mul, (half8_t*)(p + (int64_t)(it * 4) * a.stride_oy));
        } else {
          // a ragged tile (rows or chunks past the matrix are skipped, a chunk across its last
          // column goes element by element), or rows that are not 16-byte aligned (a row length
          // that is no multiple of 8: store8_any)
          const bool whole = x + 8 <= a.n, part = !whole && x < a.n;
#pragma unroll
          for (int it = 0; it < WIT; it++) {
            if (y0 + it * 4 >= a.m) continue;
            const half8_t r = v[it] * mul;
            half_t* const q = p + (int64_t)(it * 4) * a.stride_oy;
            if (whole) {
              if (walign == 8) __builtin_nontemporal_store(r, (half8_t*)q);
              else store8_any(q, r);
            } else if (part) {
#pragma unroll
              for (int e = 0; e < 8; e++)
                if (x + e < a.n) q[e] = r[e];
            }
          }
        }
      } else if (vec) {
        // (the rolled loops read the staging tile round by round: an array of rounds indexed by
        // the loop counter would live in scratch memory)
#pragma unroll 1
        for (int it = 0; it < WIT; it++) {
          const int y = y0 + it * 4;
          const half8_t v = staged(it);
          if (y < a.m && x < a.n) {
            if (walign == 8) store_chunk<8>(a, ep, out, y, x, v);
            else if (walign == 4) store_chunk<4>(a, ep, out, y, x, v);
            else store_chunk<2>(a, ep, out, y, x, v);
          }
        }
      } else {
        const bool need_prev = Epilogue::needs_prev(a.store);
        const bool need_bias = Epilogue::needs_bias(a.store);
#pragma unroll 1
        for (int it = 0; it < WIT; it++) {
          const int y = y0 + it * 4;
          const half8_t v = staged(it);
          if (y >= a.m) continue;
#pragma unroll
          for (int e = 0; e < 8; e++) {
            if (x + e >= a.n) continue;
            half_t* p = out + (int64_t)y * a.stride_oy + x + e;
            if (a.mask == ADR_MASK_CAUSAL && x + e > y) {
              *p = neg_inf_half();
            } else {
              const half_t prev = need_prev ? *p : (half_t)0;
              const half_t bias = need_bias ? a.bias[x + e] : (half_t)0;
              *p = ep.apply_s16(v[e], prev, bias);
            }
          }
        }
      }
    };
    Cursor c;
    c.t = 0;
    load_unit(c);
    bool started = false;
    while (c.valid) {
      const int first = c.n;
      for (; c.n < c.n_vis_end; c.n++) {
        if (!started) {
          __builtin_amdgcn_s_barrier();  // barrier 0
          __builtin_amdgcn_s_barrier();  // barrier 1
          started = true;
        }
        __builtin_amdgcn_s_barrier();  // barrier 2j+2: the upper half of tile j is staged
        write_half(c.batch, c.m0, c.n * BN, 0);
        __builtin_amdgcn_s_barrier();  // barrier 2j+3: the lower half
        write_half(c.batch, c.m0, c.n * BN, 1);
      }
      // fully masked tiles of this unit, unless fill_causal_rows_kernel wrote them already
      if (!map.prefilled)
        for (int n = max(first, c.n_vis_end); n < c.n_end; n++)
          fill_masked_tile<BM, BN, NWW * 64>(a, a.output + (int64_t)c.batch * a.stride_oz, c.m0, n * BN,
                                        tid - 512);
      c.t++;
      load_unit(c);
    }
    return;
  }

  // ------------------------------------------------------------------ multiplying wavefronts
  // 16x16x32 MFMAs: the 64 x 32 block of a wavefront is 4 x 2 independent accumulators, so that
  // no MFMA waits for the one before it
  constexpr int KS = CPR / 4;                // k-steps of 32
  const int grp = wave >> 2, wn = wave & 3;  // rows grp*64 .. +63, columns wn*32 .. +31 of a tile
  const int frow = lane & 15, fkg = lane >> 4;
  // k-step 0 of the first block; k-step kk is at (off ^ (kk << 6)), and sixteen rows further down
  // the swizzle repeats: block i is R16 bytes times i further on
  constexpr int R16 = 16 * CPR * 16;
  const int offQ = lds_chunk_off<CPR>(grp * 64 + frow, fkg);
  const int offB = lds_chunk_off<CPR>(wn * 32 + frow, fkg);
  half8_t qa[KS][4];   // this wavefront's rows of the left panel
  float4_t acc[4][2];
  // Load Scale (matmul.cu:439-443): both operands are multiplied by the scale, in fp16, before the
  // product -- the left panel once per segment, the right fragments as they are read
  const bool load_scale = a.load == ADR_LOAD_SCALE;
  const half_t ls = (half_t)a.scale;
  auto copy_left = [&]() {
#pragma unroll
    for (int kk = 0; kk < KS; kk++)
#pragma unroll
      for (int i = 0; i < 4; i++) qa[kk][i] = *(const half8_t*)(sA + (offQ ^ (kk << 6)) + i * R16);
    if (load_scale) {
#pragma unroll
      for (int kk = 0; kk < KS; kk++)
#pragma unroll
        for (int i = 0; i < 4; i++) qa[kk][i] = qa[kk][i] * ls;
    }
  };
  auto multiply = [&](const unsigned char* cB) {
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
      for (int jj = 0; jj < 2; jj++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[i][jj][r] = 0.0f;
    half8_t fb[2][2];
#pragma unroll
    for (int jj = 0; jj < 2; jj++) fb[0][jj] = *(const half8_t*)(cB + offB + jj * R16);
#pragma unroll
    for (int kk = 0; kk < KS; kk++) {
      if (kk + 1 < KS) {
#pragma unroll
        for (int jj = 0; jj < 2; jj++)
          fb[(kk + 1) & 1][jj] = *(const half8_t*)(cB + (offB ^ ((kk + 1) << 6)) + jj * R16);
      }
      if (load_scale) {
#pragma unroll
        for (int jj = 0; jj < 2; jj++) fb[kk & 1][jj] = fb[kk & 1][jj] * ls;
      }
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int jj = 0; jj < 2; jj++)
          acc[i][jj] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[kk & 1][jj], qa[kk][i], acc[i][jj],
                                                              0, 0, 0);
    }
    // a barrier orders memory operations only: without this the compiler sinks MFMAs below the
    // barrier that ends the phase, into the time that belongs to the other group's
    __builtin_amdgcn_sched_barrier(0);
  };
  // narrow and write the wavefront's 64 x 32 block: lane l of block (i, jj) holds row l % 16,
  // columns 4 * (l / 16) .. +3 of the block
  auto narrow = [&]() {
    const int lrow = lane & 15, cg = lane >> 4;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int row = grp * 64 + i * 16 + lrow;
#pragma unroll
      for (int jj = 0; jj < 2; jj++) {
        half4_t h;
#pragma unroll
        for (int e = 0; e < 4; e++) h[e] = (half_t)acc[i][jj][e];
        const int cc = wn * 4 + jj * 2 + (cg >> 1);
        *(half4_t*)(sC + row * 256 + ((cc ^ (row & 15)) << 4) + (cg & 1) * 8) = h;
      }
    }
  };

  Cursor c;
  first_item(c);
  if (!c.valid) return;
  if (grp == 0) {
    for (int j = 0; c.valid; j++) {
      __builtin_amdgcn_s_barrier();  // barrier 2j: the panels of tile j have landed
      if (c.first) copy_left();
      multiply(sB + (j % RING) * PANEL);
      __builtin_amdgcn_s_waitcnt(0xC07F);  // the panel has been read (lgkmcnt 0)
      __builtin_amdgcn_s_barrier();  // barrier 2j+1: this half of the staging tile is free
      narrow();
      __builtin_amdgcn_s_waitcnt(0xC07F);  // staged
      next_item(c);
    }
    __builtin_amdgcn_s_barrier();  // barrier 2T
    __builtin_amdgcn_s_barrier();  // barrier 2T+1
  } else {
    __builtin_amdgcn_s_barrier();  // barrier 0
    copy_left();
    for (int j = 0; c.valid; j++) {
      __builtin_amdgcn_s_waitcnt(0xC07F);
      __builtin_amdgcn_s_barrier();  // barrier 2j+1
      multiply(sB + (j % RING) * PANEL);
      __builtin_amdgcn_s_waitcnt(0xC07F);
      __builtin_amdgcn_s_barrier();  // barrier 2j+2: the ring buffer of tile j is free
      next_item(c);
      narrow();
      if (c.valid && c.first) copy_left();  // tile j+1 opens a unit: its left panel has landed
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    __builtin_amdgcn_s_barrier();  // barrier 2T+1
  }
}

// =============================================================================================
// u8-weight kernel: left operand by DMA, weights dequantised on their way into LDS
// =============================================================================================
// K % 64 == 0, block size a power of two >= 8.  The fp16 left operand goes global -> LDS by DMA
// through three stages (two slices ahead; SA = 4: four stages, three ahead).  The u8 weights of slice kt+2 are fetched into
// registers (8 weights + their scale per chunk, three chunks per lane) while slice kt runs; the
// chunks of slice kt+1 are dequantised (bit-identical to quantize.cu:53-54) and written to one
// of two fp16 LDS stages in the same swizzled layout the DMA produces, so that every weight is
// dequantised once per workgroup and the MFMA loop is the one of the fp16 kernel.
// MI16: 16x16x32 MFMAs, two k-steps per slice, all chunks dequantised in the first (the 256 x 128
// tile: 5-6 % faster; the 256 x 192 tile has no registers for the second set of fragments)
// G: groups of WM x WN wavefronts that split K between them (1: none).  A tile that has its compute
// unit to itself is bound by the chain of one slice -- barrier, fragment reads, MFMAs, the wait for
// the next slice: 0.3-0.4 us per slice of a 64 x 64 tile whatever its loads -- so with at most one
// tile per compute unit the small tiles run G such chains side by side.
template <int BM, int BN, int WM, int WN, bool MI16, int BK = 64, int G = 1, int SA = 3>
__global__ __launch_bounds__(WM* WN* G * 64, 1) void gemm_nt_u8_kernel(MatmulArgs a, TileMap map,
                                                                      int block_shift) {
  constexpr int CPR = BK / 8, MI = MI16 ? 16 : 32, KG = 64 / MI, KK = CPR / KG;
  constexpr int NW = WM * WN, NT = NW * 64;  // wavefronts and lanes of one group
  constexpr int IA = BM * CPR / NT;   // DMA instructions per lane and slice
  constexpr int LB = BN * CPR / NT;   // 8-weight chunks per lane and slice
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
  constexpr int FM = WTM / MI, FN = WTN / MI;  // MFMA blocks of the wavefront's sub-tile
  constexpr int FSTEP = MI * CPR * 16;         // bytes between the fragments of consecutive blocks
  constexpr int SLOT = 32 * (TN * 64 + 16);
  static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "slices must split evenly over lanes");
  // epilogue slots lie in the stages of the operand with the larger ones, per stage half the
  // wavefronts where they fit (the 256-row tiles), else as many as fit
  constexpr bool SLOTS_IN_B = BN > BM;
  constexpr int SLOT_STAGE = (SLOTS_IN_B ? BN : BM) * BK * 2;
  constexpr int SLOTS = (NW / 2) * SLOT <= SLOT_STAGE ? NW / 2 : SLOT_STAGE / SLOT;
  static_assert(SLOTS >= 1 && (NW + SLOTS - 1) / SLOTS <= (SLOTS_IN_B ? 2 : 3),
                "epilogue slots must fit in the stages");
  static_assert(MI16 ? LB <= 8 && FM * FN % LB == 0 : LB < KK, "no chunk is dequantised in the last k-step");
  __shared__ __attribute__((aligned(1024))) unsigned char sA0[G * BM * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sA1[G * BM * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sA2[G * BM * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sA3[SA == 4 ? G * BM * BK * 2 : 1024];
  static_assert(SA == 3 || SA == 4, "three stages of the left operand (two slices ahead) or four (three ahead)");
  __shared__ __attribute__((aligned(1024))) unsigned char sB0[G * BN * BK * 2];
  __shared__ __attribute__((aligned(1024))) unsigned char sB1[G * BN * BK * 2];

  int batch, tile_m, tile_n;
  map_tile(map, batch, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  // G groups of NW wavefronts: every group multiplies the whole tile over its own slices of K
  // (slice s of the tile's walk is the G slices s*G .. s*G+G-1 of K, one per group, in stages of
  // its own), all groups pass the same barriers, and their sums meet in LDS behind the loop
  const int lane = threadIdx.x & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = G > 1 ? wave_all / NW : 0, wave = G > 1 ? wave_all % NW : wave_all;
  const int tid = wave * 64 + lane;
  const int goA = grp * (BM * BK * 2), goB = grp * (BN * BK * 2);
  const int wm = wave / WN, wn = wave % WN;
  half_t* const out = a.output;

  const half_t* gA[IA];
#pragma unroll
  for (int i = 0; i < IA; i++) {
    int row, kc;
    lds_chunk_inv<CPR>((i * NW + wave) * 64 + lane, row, kc);
    gA[i] = a.lhs + (int64_t)min(m0 + row, a.m - 1) * a.stride_ly + kc * 8;
  }
  // weight chunk c = tid + i*NT -> (row, 8-weight group kc); rows beyond N are clamped
  const uint8_t* gQ[LB];
  const half_t* gS[LB];
  int offB[LB];
#pragma unroll
  for (int i = 0; i < LB; i++) {
    const int c = tid + i * NT, row = c / CPR, kc = c % CPR;
    const int brow = min(n0 + row, a.n - 1);
    gQ[i] = a.rhs_q + (int64_t)brow * a.k + kc * 8;
    // block of weight k0 + 8*kc: k0 is a multiple of BK and 8*kc < BK, so the two parts of the
    // index add up exactly for any power-of-two block size
    gS[i] = a.scales + (int64_t)brow * (a.k >> block_shift) + ((kc * 8) >> block_shift);
    offB[i] = lds_chunk_off<CPR>(row, kc);
  }
  const int KT = a.k / (BK * G);
  int kloadA = 0, kloadQ = 0;
  auto dmaA = [&](unsigned char* dA) {
    const int k0 = (min(kloadA, KT - 1) * G + grp) * BK;
    kloadA++;
#pragma unroll
    for (int i = 0; i < IA; i++)
      __builtin_amdgcn_global_load_lds(ADR_GLB_PTR(gA[i] + k0),
                                       ADR_LDS_PTR(dA + goA + (i * NW + wave) * 1024), 16, 0, 0);
  };
  // three register sets: the weights consumed in slice kt+1 were requested at the head of slice
  // kt-1, so the wait at the end of slice kt-1 (everything but that slice's own requests)
  // already covers them and nothing in slice kt waits for a load issued a moment ago
  u32x2_t rq[3][LB];
  half_t rs[3][LB];
  auto fetchQ = [&](int set) {
    const int ks = min(kloadQ, KT - 1) * G + grp;
    kloadQ++;
#pragma unroll
    for (int i = 0; i < LB; i++) {
      rq[set][i] = *(const u32x2_t*)(gQ[i] + ks * BK);
      rs[set][i] = gS[i][(ks * BK) >> block_shift];
    }
  };
  auto dequant_store1 = [&](int set, unsigned char* dB, int i) {
    const half2_t s2 = {rs[set][i], rs[set][i]};
    *(half8_t*)(dB + goB + offB[i]) = dequant8(rq[set][i][0], rq[set][i][1], s2);
  };
  auto dequant_store = [&](int set, unsigned char* dB) {
#pragma unroll
    for (int i = 0; i < LB; i++) dequant_store1(set, dB, i);
  };

  typedef typename std::conditional<MI16, float4_t, float16_t>::type acc_t;
  acc_t acc[FM][FN];
#pragma unroll
  for (int i = 0; i < FM; i++)
#pragma unroll
    for (int j = 0; j < FN; j++)
#pragma unroll
      for (int r = 0; r < (MI16 ? 4 : 16); r++) acc[i][j][r] = 0.0f;

  // fragment of block i: FSTEP bytes per block beyond the first one's (see gemm_nt_dma_kernel)
  const int frow = lane & (MI - 1), fkg = lane / MI;
  int offFA[KK], offFB[KK];
#pragma unroll
  for (int kk = 0; kk < KK; kk++) {
    offFA[kk] = lds_chunk_off<CPR>(wm * WTM + frow, kk * KG + fkg);
    offFB[kk] = lds_chunk_off<CPR>(wn * WTN + frow, kk * KG + fkg);
  }
  half8_t fa[2][FM], fb[2][FN];
  auto load_frags = [&](int slot, const unsigned char* cA, const unsigned char* cB, int kk) {
#pragma unroll
    for (int i = 0; i < FM; i++) fa[slot][i] = *(const half8_t*)(cA + goA + offFA[kk] + i * FSTEP);
#pragma unroll
    for (int j = 0; j < FN; j++) fb[slot][j] = *(const half8_t*)(cB + goB + offFB[kk] + j * FSTEP);
  };
  auto mfmas = [&](int slot) {
#pragma unroll
    for (int i = 0; i < FM; i++)
#pragma unroll
      for (int j = 0; j < FN; j++) {
        if constexpr (MI16)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[slot][j], fa[slot][i], acc[i][j],
                                                             0, 0, 0);
        else
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[slot][j], fa[slot][i], acc[i][j],
                                                             0, 0, 0);
      }
  };
  // Slice kt.  (cA, cB): its stages; (nA, nB): those of slice kt+1 -- nB is filled here from
  // register set `nset`; dA: the A stage refilled with slice kt+2; `fset`: the register set
  // that receives the weights of slice kt+3 (the one slice kt was dequantised from).
  auto slice = [&](const unsigned char* cA, const unsigned char* cB, const unsigned char* nA,
                   unsigned char* nB, unsigned char* dA, int fset, int nset) {
    fetchQ(fset);
    dmaA(dA);
    __builtin_amdgcn_sched_barrier(0);
    // first k-step: the fragments of the second are read and the slice's LB 8-weight chunks are
    // dequantised, their VALU work and LDS writes filling the gaps between its MFMAs
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      if (kk + 1 < KK) load_frags((kk + 1) & 1, cA, cB, kk + 1);
      // the slice's LB 8-weight chunks are dequantised one per k-step (32x32x16) or all in the
      // first (16x16x32): their VALU work and LDS writes fill the gaps between that step's MFMAs
      constexpr int PER_CHUNK = MI16 ? FM * FN / LB : FM * FN;  // MFMAs per chunk
      const bool chunks_here = MI16 ? kk == 0 : kk < LB;
      if (chunks_here) {
        if constexpr (MI16) dequant_store(nset, nB); else dequant_store1(nset, nB, kk);
      }
      mfmas(kk & 1);
      if (kk + 1 < KK) {
#pragma unroll
        for (int q = 0; q < FM * FN; q++) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          if (chunks_here) {
            __builtin_amdgcn_sched_group_barrier(0x002, 20 / PER_CHUNK + 1, 0);
            if (q % PER_CHUNK == PER_CHUNK - 1) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
          }
        }
      }
    }
    // A(kt+1) has landed: only the weight fetch and the DMA issued in this slice may still be
    // in flight; the dequantised weights of slice kt+1 are in LDS
    // (four A stages: the transfer issued in the slice before, which is younger than that slice's
    // weight requests, may stay in flight too)
    constexpr int n = 2 * LB + (SA - 2) * IA;
    __builtin_amdgcn_s_waitcnt(0x0070 | (n & 0xF) | ((n >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    load_frags(0, nA, nB, 0);
  };

  // slice kt (kt % P == p) reads A stage p % SA and B stage p % 2, dequantises register set
  // (p + 1) % 3 into the other B stage, refills the A stage read one slice earlier with slice
  // kt + SA - 1 and register set p % 3 with the weights of slice kt + 3
  auto stA = [&](int i) -> unsigned char* { return i == 0 ? sA0 : i == 1 ? sA1 : i == 2 ? sA2 : sA3; };
  auto stB = [&](int i) -> unsigned char* { return i == 0 ? sB0 : sB1; };
  constexpr int P = SA == 3 ? 6 : 12;  // the common period of the stages and the register sets
  auto slice_p = [&](int p) {
    slice(stA(p % SA), stB(p % 2), stA((p + 1) % SA), stB((p + 1) % 2), stA((p + SA - 1) % SA), p % 3,
          (p + 1) % 3);
  };
  fetchQ(0);
  fetchQ(1);
  dmaA(sA0);
  fetchQ(2);
  dmaA(sA1);
  if (SA == 4) dmaA(sA2);
  dequant_store(0, sB0);
  {
    constexpr int n = (SA - 2) * IA;
    __builtin_amdgcn_s_waitcnt(0x0070 | (n & 0xF) | ((n >> 4) << 14));
    __builtin_amdgcn_s_barrier();
  }
  load_frags(0, sA0, sB0, 0);
  int kt = 0;
  for (; kt + P <= KT; kt += P) {
#pragma unroll
    for (int p = 0; p < P; p++) slice_p(p);
  }
#pragma unroll
  for (int p = 0; p < P - 1; p++)
    if (kt < KT) { slice_p(p); kt++; }
  __builtin_amdgcn_s_waitcnt(0x0070);
  __builtin_amdgcn_s_barrier();

  if constexpr (G > 1) {
    // the groups' sums, group by group in group order, through the first A stage: a lane's
    // accumulator registers four at a time (a wavefront's four registers are 1 KiB)
    constexpr int AR = MI16 ? 4 : 16, QUADS = FM * FN * AR / 4;
    constexpr int PIECE = QUADS * NW * 1024 <= G * BM * BK * 2 ? QUADS : G * BM * BK * 2 / (NW * 1024);
    static_assert(PIECE >= 1 && QUADS % PIECE == 0, "the sums pass through the first A stage in equal pieces");
    float4_t* const red = (float4_t*)sA0 + (wave * PIECE) * 64 + lane;
    auto quad = [&](int q) -> float4_t& {  // quad q of the lane's accumulators
      constexpr int PER = AR / 4;
      return *((float4_t*)&acc[q / PER / FN][q / PER % FN] + q % PER);
    };
    for (int g = 1; g < G; g++) {
#pragma unroll
      for (int p0 = 0; p0 < QUADS; p0 += PIECE) {
        if (grp == g) {
#pragma unroll
          for (int q = 0; q < PIECE; q++) red[q * 64] = quad(p0 + q);
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_s_barrier();
        if (grp == 0) {
#pragma unroll
          for (int q = 0; q < PIECE; q++) quad(p0 + q) += red[q * 64];
        }
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_s_barrier();
      }
    }
    if (grp != 0) return;
  }
  unsigned char* slot = (SLOTS_IN_B ? (wave < SLOTS ? sB0 : sB1)
                                    : (wave < SLOTS ? sA0 : wave < 2 * SLOTS ? sA1 : sA2)) + (wave % SLOTS) * SLOT;
  wave_epilogue<TM, 2 * TN>(a, out, acc, m0 + wm * WTM, n0 + wn * WTN, slot, (half_t)a.scale, lane);
}

// =============================================================================================
// Register-staged kernel (any K % 8 == 0; Load Scale; u8 weights)
// =============================================================================================
template <int BM, int BN, int BK, int WM, int WN, int MINB, bool LOAD_SCALE, bool WQ>
__global__ __launch_bounds__(WM* WN * 64, MINB) void gemm_nt_stage_kernel(MatmulArgs a,
                                                                           TileMap map) {
  constexpr int NT = WM * WN * 64;
  constexpr int CPR = BK / 8;
  constexpr int LA = BM * CPR / NT, LB = BN * CPR / NT;  // chunks each thread stages
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32, KK = BK / 16;
  constexpr int SLOT = 32 * (TN * 64 + 16);
  static_assert(BM * CPR % NT == 0 && BN * CPR % NT == 0, "staging must divide evenly");
  static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 16 == 0, "MFMA 32x32x16 tiling");
  static_assert(WM * WN * SLOT <= 2 * (BM + BN) * BK * 2, "epilogue slots must fit in LDS");

  extern __shared__ __attribute__((aligned(1024))) unsigned char smem[];
  unsigned char* const sA = smem;                    // [2][BM][BK] halves
  unsigned char* const sB = smem + 2 * BM * BK * 2;  // [2][BN][BK] halves

  int batch, tile_m, tile_n;
  map_tile(map, batch, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  half_t* const out = a.output + (int64_t)batch * a.stride_oz;

  if (a.mask == ADR_MASK_CAUSAL && n0 > m0 + BM - 1) {
    fill_masked_tile<BM, BN, NT>(a, out, m0, n0, tid);
    return;
  }

  const half_t* const A = a.lhs + (int64_t)batch * a.stride_lz;
  const half_t* const B = a.rhs + (int64_t)batch * a.stride_rz;  // fp16 right operand (!WQ)

  // staging assignment: chunk c = tid + i*NT -> (row, kc); rows beyond the matrix are clamped
  // to the last valid row (their products are never stored)
  const half_t* gA[LA];
  const half_t* gB[LB];   // fp16 right operand
  const uint8_t* gQ[LB];  // u8 right operand: 8 weights per chunk ...
  const half_t* gS[LB];   // ... and the scale row of that weight row
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
        // beyond K get scale 0, i.e. zeros
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
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < KT) store_slice(buf ^ 1);
    __syncthreads();
  }

  wave_epilogue<TM, 2 * TN>(a, out, acc, m0 + wm * WTM, n0 + wn * WTN, smem + wave * SLOT, hscale,
                        lane);
}

// =============================================================================================
// Register-staged kernel for row-major x row-major products whose left rows have any alignment
// =============================================================================================
// P.V of the attention call sites (llama.rs:552-554, clip.rs:385-388, whisper.rs:433-436) when
// the sequence length is no multiple of 64: the probabilities [heads, S, T] are a dense tensor,
// so their rows start at any even byte address (T = 77, 257, 1500, 2001 ...) and K = T ends in the
// middle of a slice, or of a 16-byte chunk.  The left operand goes through registers: a lane
// loads the dwords around its chunk from a 4-byte aligned address and shifts them into place
// (v_alignbyte_b32), zeroes what lies beyond K, and writes the chunk to LDS in the layout of the
// other kernels.  The right operand ([K][N], N contiguous, 16-byte aligned rows: V on its head
// view) is staged as [64][BN] tiles and read with the transposing LDS reads of the DMA kernel's
// row-major form.  Two LDS stages, one barrier per slice, loads two slices ahead of the MFMAs,
// BM x BN tiles of WM x WN wavefronts (eight for the 128-row tiles; BN = 64 for heads of 64
// columns and wherever that gives a product of few tiles more workgroups).
// G > 1: G groups of WM x WN wavefronts share the tile, group g multiplying the K slices
// g, g + G, g + 2G ... in stages of its own (a slice past K is all zeros).  A compute unit does
// not fetch much more than 100 GB/s, and a tile that has one to itself is bound by the chain of
// one slice, load -> LDS -> barrier -> fragment reads -> MFMA: small tiles put a product of few
// rows on many compute units and G chains in flight shorten each G-fold (20 heads x 1..200 rows
// against 1500 frames: 24 -> 8 us).  Behind the loop the groups leave their accumulators in
// their stages and group 0 adds them in group order (the same sum every launch).
template <int BM, int BN, int WM, int WN, int G>
__global__ __launch_bounds__(WM * WN * G * 64, (G == 1 ? 2 : 1)) void gemm_nn_anyrow_kernel(MatmulArgs a, TileMap map) {
  constexpr int BK = 64, NW = WM * WN, NT = NW * 64, CPR = 8;
  constexpr int LA = (BM * CPR + NT - 1) / NT, LB = BK * (BN / 8) / NT;  // chunks each thread stages
  constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32, KK = BK / 16;
  constexpr int SLOT = 32 * (TN * 64 + 16);
  constexpr int A_STAGE = BM * BK * 2, B_STAGE = BK * BN * 2, GROUP = 2 * (A_STAGE + B_STAGE);
  static_assert(BN == 128 || BN == 64, "one or half a 256-byte line per k row");
  static_assert(TM >= 1 && TN >= 1 && BM * CPR % NT == 0 && BK * (BN / 8) % NT == 0, "tile shape");
  // chunk c of k row r of the right tile sits at position c ^ swz(r) of its row: the 16 chunks a
  // transposing read touches (4 rows x 4 chunks per 32 lanes) then fall into 16 bank groups
  auto swz = [](int krow) { return BN == 128 ? (krow & 3) << 2 : ((krow >> 1) & 1) << 2; };
  static_assert(NW * SLOT <= GROUP, "epilogue slots must fit in the stages of group 0");
  static_assert(NT * TM * TN * 64 <= GROUP, "a group's accumulators must fit in its stages");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[G][GROUP];

  int batch, tile_m, tile_n;
  map_tile(map, batch, tile_m, tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;
  const int lane = threadIdx.x & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = wave_all / NW, wave = wave_all % NW, tid = wave * 64 + lane;
  const int wm = wave / WN, wn = wave % WN;
  half_t* const out = a.output + (int64_t)batch * a.stride_oz;
  if (a.mask == ADR_MASK_CAUSAL && n0 > m0 + BM - 1) {
    fill_masked_tile<BM, BN, NT * G>(a, out, m0, n0, threadIdx.x);
    return;
  }
  const half_t* const A = a.lhs + (int64_t)batch * a.stride_lz;
  const half_t* const B = a.rhs + (int64_t)batch * a.stride_rz;
  const int K = a.k, KT = (K + BK - 1) / BK, ITERS = (KT + G - 1) / G;
  unsigned char* const mine = lds[grp];
  auto sA = [&](int buf) { return mine + buf * A_STAGE; };
  auto sB = [&](int buf) { return mine + 2 * A_STAGE + buf * B_STAGE; };

  // Left operand.  Chunk c = tid + i * NT -> (row, kc).  Rows beyond the matrix read the last
  // row again (their products are never stored).  `last` is the last dword of the left operand
  // that may be read: no load goes past the tensor, whatever comes after it in memory.
  const half_t* gA[LA];
  int offA[LA], kcA[LA];
#pragma unroll
  for (int i = 0; i < LA; i++) {
    const int c = tid + i * NT, row = c / CPR, kc = c % CPR;
    gA[i] = A + (int64_t)min(m0 + row, a.m - 1) * a.stride_ly + kc * 8;
    offA[i] = lds_chunk_off<CPR>(row, kc);
    kcA[i] = kc * 8;
  }
  const uintptr_t a_end = (uintptr_t)(a.lhs + (int64_t)(a.batches - 1) * a.stride_lz +
                                      (int64_t)(a.m - 1) * a.stride_ly + K);  // one past the last element
  const uintptr_t last = ((a_end + 3) & ~(uintptr_t)3) - 4;
  // Right operand.  Chunk c -> (k row, column chunk) of the [64][128] tile; k rows beyond K and
  // columns beyond N are zero.
  int krB[LB], ncB[LB], offB[LB];
  const half_t* gB[LB];  // the chunk in slice 0 (columns beyond N read column 0)
#pragma unroll
  for (int i = 0; i < LB; i++) {
    const int c = tid + i * NT;
    krB[i] = c / (BN / 8);
    ncB[i] = (c % (BN / 8)) * 8;
    offB[i] = krB[i] * (BN * 2) + (((ncB[i] >> 3) ^ swz(krB[i])) << 4);
    gB[i] = B + (int64_t)krB[i] * a.stride_ry + (n0 + ncB[i] < a.n ? n0 + ncB[i] : 0);
  }
  const bool cols_full = n0 + BN <= a.n;

  // What a thread holds of one slice between its loads and its LDS stores: the five dwords around
  // each chunk of the left operand (shifted into place and cut at K only when they are stored, so
  // that nothing waits for a load before the slice's MFMAs have been issued) and its chunks of the
  // right operand.
  struct Raw {
    uint32_t a[LA][5];
    u32x4_t b[LB];
  };
  // A slice that ends at least two elements before K lies inside every row with the dword that
  // follows each chunk: no address needs clamping and nothing needs cutting.  Both branches issue
  // the same loads in the same order, so the waits counted behind them hold for either.
  auto inside = [&](int k0) { return k0 + BK + 2 <= K; };
  auto issue = [&](int kt, Raw& r) {
    const int k0 = kt * BK;
    if (inside(k0)) {
#pragma unroll
      for (int i = 0; i < LA; i++) {
        const uintptr_t base = (uintptr_t)(gA[i] + k0) & ~(uintptr_t)3;
        const u32x4_t q = *(const ADR_GLOBAL_AS u32x4_dword_aligned_t*)base;
        r.a[i][0] = q[0]; r.a[i][1] = q[1]; r.a[i][2] = q[2]; r.a[i][3] = q[3];
        r.a[i][4] = *(const ADR_GLOBAL_AS uint32_t*)(base + 16);
      }
      const int64_t step = (int64_t)k0 * a.stride_ry;
#pragma unroll
      for (int i = 0; i < LB; i++) r.b[i] = *(const u32x4_t*)(gB[i] + step);
    } else {
#pragma unroll
      for (int i = 0; i < LA; i++) load5_issue(gA[i] + k0, last, r.a[i]);
#pragma unroll
      for (int i = 0; i < LB; i++) {
        const int kr = k0 + krB[i], col = n0 + ncB[i];
        r.b[i] = *(const u32x4_t*)(B + (int64_t)min(kr, K - 1) * a.stride_ry + (col < a.n ? col : 0));
      }
    }
  };
  auto finish = [&](int kt, int buf, const Raw& r) {
    const int k0 = kt * BK;
    if (inside(k0)) {
#pragma unroll
      for (int i = 0; i < LA; i++)
        *(u32x4_t*)(sA(buf) + offA[i]) = align5(r.a[i], (uint32_t)((uintptr_t)gA[i] & 2));
    } else {
#pragma unroll
      for (int i = 0; i < LA; i++) {
        u32x4_t v = load5_finish(gA[i] + k0, last, r.a[i]);
        const int valid = K - k0 - kcA[i];  // elements from `valid` on are zero
#pragma unroll
        for (int j = 0; j < 4; j++)  // elements 2j and 2j+1 of the chunk
          v[j] = 2 * j + 1 < valid ? v[j] : 2 * j < valid ? (v[j] & 0xffffu) : 0u;
        *(u32x4_t*)(sA(buf) + offA[i]) = v;
      }
    }
    if (inside(k0) && cols_full) {
#pragma unroll
      for (int i = 0; i < LB; i++) *(u32x4_t*)(sB(buf) + offB[i]) = r.b[i];
    } else {
#pragma unroll
      for (int i = 0; i < LB; i++) {
        const bool in = k0 + krB[i] < K && n0 + ncB[i] < a.n;
        *(u32x4_t*)(sB(buf) + offB[i]) = in ? r.b[i] : u32x4_t{0, 0, 0, 0};
      }
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[i][j][r] = 0.0f;

  // fragment addressing.  Left: lane -> (row lane % 32, k-group lane / 32).  Right: the
  // transposing read of the DMA kernel's row-major form (ds_read_b64_tr_b16): inside each group of
  // 16 lanes, lanes 4r..4r+3 address 16 consecutive halves of k-row r and lane i receives column
  // i of that 4 x 16 block.
  const int frow = lane & 31, fkg = lane >> 5;
  int offFB[TN][KK];
  {
    const int q = lane >> 4, r = (lane >> 2) & 3, jj = lane & 3;
#pragma unroll
    for (int kk = 0; kk < KK; kk++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int krow = kk * 16 + (q >> 1) * 8 + r;
        const int col = wn * WTN + j * 32 + 16 * (q & 1) + 4 * jj;
        offFB[j][kk] = krow * (BN * 2) + (((col >> 3) ^ swz(krow)) << 4) + (jj & 1) * 8;
      }
  }
  typedef short short4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) short4_t lds_short4_t;

  auto compute = [&](int buf) {
    const unsigned char* cA = sA(buf);
    const unsigned char* cB = sB(buf);
#pragma unroll
    for (int kk = 0; kk < KK; kk++) {
      half8_t fa[TM], fb[TN];
#pragma unroll
      for (int i = 0; i < TM; i++)
        fa[i] = *(const half8_t*)(cA + lds_chunk_off<CPR>(wm * WTM + i * 32 + frow, kk * 2 + fkg));
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4_t*)ADR_LDS_PTR(cB + offFB[j][kk]));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
            (lds_short4_t*)ADR_LDS_PTR(cB + offFB[j][kk] + 4 * (BN * 2)));  // k-rows + 4
        fb[j] = __builtin_shufflevector(__builtin_bit_cast(half4_t, lo),
                                        __builtin_bit_cast(half4_t, hi), 0, 1, 2, 3, 4, 5, 6, 7);
      }
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[j], fa[i], acc[i][j], 0, 0, 0);
    }
  };
  // The group's slice number `it` is slice it * G + grp of K.  Loads run two slices ahead of the
  // MFMAs: while slice `it` is multiplied out of one LDS stage, slice it + 1 waits in registers for
  // the other stage and slice it + 2 is on its way (loads return in order, so storing the older
  // set does not wait for the younger one).
  auto at = [&](int it) { return it * G + grp; };
  // The waits are counted statically, so inside the steady loop no branch holds a load and no exit
  // leaves from its middle: either would make the loads of the two register sets pending in an
  // order that depends on the path, and every wait would then drain them all.  Products of more
  // than four slices run the steady loop down to their last three or four slices; the rest (and
  // short products from the start) go through the tail, whose waits may be conservative.
  Raw r0, r1;
  int it = 0;
  if (ITERS > 4) {
    issue(at(0), r0);
    issue(at(1), r1);
    finish(at(0), 0, r0);
    issue(at(2), r0);
    __syncthreads();
    for (; it + 4 < ITERS; it += 2) {
      compute(0);
      __builtin_amdgcn_sched_barrier(0);
      finish(at(it + 1), 1, r1);
      issue(at(it + 3), r1);
      __syncthreads();
      compute(1);
      __builtin_amdgcn_sched_barrier(0);
      finish(at(it + 2), 0, r0);
      issue(at(it + 4), r0);
      __syncthreads();
    }
  } else {
    issue(at(0), r0);
    if (ITERS > 1) issue(at(1), r1);
    finish(at(0), 0, r0);
    if (ITERS > 2) issue(at(2), r0);
    __syncthreads();
  }
  // tail: slice `it` is in stage 0, r1 holds slice it + 1 and r0 slice it + 2 (where they exist);
  // at most four slices are left
  compute(0);
  if (it + 1 < ITERS) finish(at(it + 1), 1, r1);
  if (it + 3 < ITERS) issue(at(it + 3), r1);
  __syncthreads();
  if (it + 1 < ITERS) {
    compute(1);
    if (it + 2 < ITERS) finish(at(it + 2), 0, r0);
    __syncthreads();
  }
  if (it + 2 < ITERS) {
    compute(0);
    if (it + 3 < ITERS) finish(at(it + 3), 1, r1);
    __syncthreads();
  }
  if (it + 3 < ITERS) {
    compute(1);
    __syncthreads();
  }
  if constexpr (G > 1) {
    // [register quad][thread] float4 in the group's own stages: consecutive lanes, consecutive 16 bytes
    if (grp != 0) {
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int q = 0; q < 4; q++)
            *(float4_t*)(mine + (((i * TN + j) * 4 + q) * NT + tid) * 16) =
                float4_t{acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
    }
    __syncthreads();
    if (grp != 0) return;
#pragma unroll 1
    for (int g = 1; g < G; g++)
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const float4_t v = *(const float4_t*)(lds[g] + (((i * TN + j) * 4 + q) * NT + tid) * 16);
#pragma unroll
            for (int e = 0; e < 4; e++) acc[i][j][4 * q + e] += v[e];
          }
  }
  wave_epilogue<TM, 2 * TN>(a, out, acc, m0 + wm * WTM, n0 + wn * WTN, lds[0] + wave * SLOT,
                            (half_t)a.scale, lane);
}

// =============================================================================================
// Host side: configuration choice and launch
// =============================================================================================
TileMap make_map(const MatmulArgs& a, int bm, int bn) {
  TileMap map;
  map.tiles_m = (a.m + bm - 1) / bm;
  map.tiles_n = (a.n + bn - 1) / bn;
  map.tiles_per_batch = map.tiles_m * map.tiles_n;
  const int64_t total = (int64_t)map.tiles_per_batch * a.batches;
  map.total = total > 0x7fffffffLL ? -1 : (int)total;
  // tile rows per group: a die holds 32 tiles of 256 rows at a time (64 of the smaller ones); g
  // rows x 32/g columns of them fetch g * bm + 32/g * bn operand rows per K slice, least near
  // g = sqrt(32 bn / bm): 4 for the 256-row tiles (qkv: 21.0 instead of 23.1 MB per die and
  // round), 8 for the others
  const int g = bm >= 256 ? 4 : 8;
  map.group_m = map.tiles_m < g ? map.tiles_m : g;
  map.xcds = device_info_for_plan().xcds;
  map.splits = 1;
  return map;
}

template <int BM, int BN, int WM, int WN, int NSTAGE, int MINB, bool NN = false, int BK = 64, bool MI16 = false>
hipError_t launch_dma(hipStream_t stream, const MatmulArgs& a) {
  TileMap map = make_map(a, BM, BN);
  if (map.total < 0) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((gemm_nt_dma_kernel<BM, BN, WM, WN, NSTAGE, MINB, NN, BK, false, MI16>),
                     dim3((unsigned)map.total), dim3(WM * WN * 64), 0, stream, a, map);
  return hipGetLastError();
}

// Bytes of workspace a split product on BM x BN tiles with `splits` pieces needs.
int64_t split_workspace_bytes(const MatmulArgs& a, int bm, int bn, int splits) {
  const int64_t tiles = (int64_t)((a.m + bm - 1) / bm) * ((a.n + bn - 1) / bn) * a.batches;
  return tiles * splits * bm * bn * 4;
}

template <int BM, int BN, int WM, int WN, int NSTAGE, int MINB>
hipError_t launch_dma_split(hipStream_t stream, const MatmulArgs& a, int splits) {
  TileMap map = make_map(a, BM, BN);
  if (map.total < 0 || (int64_t)map.total * splits > 0x7fffffffLL) return hipErrorInvalidConfiguration;
  if (!a.workspace || a.workspace_bytes < split_workspace_bytes(a, BM, BN, splits)) return hipErrorInvalidValue;
  map.splits = splits;
  hipLaunchKernelGGL((gemm_nt_dma_kernel<BM, BN, WM, WN, NSTAGE, MINB, false, 64, true>),
                     dim3((unsigned)(map.total * splits)), dim3(WM * WN * 64), 0, stream, a, map);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL((splitk_reduce_kernel<BM, BN, WM, WN>), dim3((unsigned)map.total),
                     dim3(WM * WN * 64), 0, stream, a, map);
  return hipGetLastError();
}

template <int BM, int BN, int BK, int WM, int WN, int MINB>
hipError_t launch_stage(hipStream_t stream, const MatmulArgs& a) {
  TileMap map = make_map(a, BM, BN);
  if (map.total < 0) return hipErrorInvalidConfiguration;
  constexpr int LDS = 2 * (BM + BN) * BK * 2;
  static_assert(LDS <= 64 * 1024, "dynamic LDS above 64 KiB needs a per-device attribute");
  dim3 grid((unsigned)map.total), block(WM * WN * 64);
  if (a.rhs_q)
    hipLaunchKernelGGL((gemm_nt_stage_kernel<BM, BN, BK, WM, WN, MINB, false, true>), grid, block,
                       LDS, stream, a, map);
  else if (a.load == ADR_LOAD_SCALE)
    hipLaunchKernelGGL((gemm_nt_stage_kernel<BM, BN, BK, WM, WN, MINB, true, false>), grid, block,
                       LDS, stream, a, map);
  else
    hipLaunchKernelGGL((gemm_nt_stage_kernel<BM, BN, BK, WM, WN, MINB, false, false>), grid, block,
                       LDS, stream, a, map);
  return hipGetLastError();
}

template <int BM, int BN, int WM, int WN, bool MI16, int BK = 64, int G = 1, int SA = 3>
hipError_t launch_u8(hipStream_t stream, const MatmulArgs& a) {
  TileMap map = make_map(a, BM, BN);
  if (map.total < 0 || a.k % (BK * G) != 0) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((gemm_nt_u8_kernel<BM, BN, WM, WN, MI16, BK, G, SA>), dim3((unsigned)map.total),
                     dim3(WM * WN * G * 64), 0, stream, a, map, __builtin_ctz(a.block_size));
  return hipGetLastError();
}

template <int BM, int BN, int WM, int WN, int G>
hipError_t launch_nn_anyrow(hipStream_t stream, const MatmulArgs& a) {
  TileMap map = make_map(a, BM, BN);
  if (map.total < 0) return hipErrorInvalidConfiguration;
  hipLaunchKernelGGL((gemm_nn_anyrow_kernel<BM, BN, WM, WN, G>), dim3((unsigned)map.total),
                     dim3(WM * WN * G * 64), 0, stream, a, map);
  return hipGetLastError();
}

// compute units of the current device (MI355X: 256)
static int num_cu() { return device_info_for_plan().cus; }

template <int CPR>
hipError_t launch_shortk(hipStream_t stream, const MatmulArgs& a) {
  ShortKMap map;
  const int NUM_CU = num_cu();
  map.xcds = device_info_for_plan().xcds;
  map.tiles_m = (a.m + 127) / 128;
  map.tiles_n = (a.n + 127) / 128;
  const int64_t rows = (int64_t)map.tiles_m * a.batches;
  if (rows * map.tiles_n > 0x3fffffffLL) return hipErrorInvalidConfiguration;
  map.rows = (int)rows;
  // split tile rows into segments until there are at least two units per workgroup
  map.seg = map.tiles_n;
  while (rows * ((map.tiles_n + map.seg - 1) / map.seg) < 2 * NUM_CU && map.seg > 4)
    map.seg = (map.seg + 1) / 2;
  map.segs_per_row = (map.tiles_n + map.seg - 1) / map.seg;
  map.units = map.rows * map.segs_per_row;
  const unsigned grid = map.units < NUM_CU ? (unsigned)map.units : NUM_CU;
  map.prefilled = 0;
  const int64_t all_rows = (int64_t)a.m * a.batches;
  if (a.mask == ADR_MASK_CAUSAL && map.tiles_n > 1 && all_rows <= 0x7fffffffLL) {
    hipLaunchKernelGGL(fill_causal_rows_kernel, dim3((unsigned)((all_rows + 3) / 4)), dim3(256), 0,
                       stream, a);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    map.prefilled = 1;
  }
  hipLaunchKernelGGL((gemm_nt_shortk_kernel<CPR>), dim3(grid), dim3(SHORTK_THREADS), 0, stream, a, map);
  return hipGetLastError();
}

enum GemmChoice {
  GEMM_NONE = 0,
  SHORTK_64, SHORTK_128,
  U8_256x192, U8_256x128, U8_128x128, U8_128x64, U8_64x64, U8_128x64_G2, U8_64x64_G4,
  DMA_256x192, DMA_256x160, DMA_256x128, DMA_128x256, DMA_128x192, DMA_128x128, DMA_128x64, DMA_64x64, DMA_64x64_K128, DMA_128x64_K128,
  DMA_NN_256x128, DMA_NN_128x128, NN_ANYROW_128x128, NN_ANYROW_128x64,
  NN_ANYROW_64x64_G4, NN_ANYROW_32x64_G4,
  STAGE_256x128, STAGE_128x128, STAGE_64x64,
};

struct Candidate {
  GemmChoice id;
  int bm, bn;
  int slots;   // workgroups resident per CU
  float eff;   // measured relative throughput of one busy CU with this tile
};

// Estimated cost: the tiles of the busiest CU times the work of one tile over the efficiency of
// a CU running this tile shape.  (With few long tiles the transfer rate into one CU's LDS, not
// the matrix pipe, bounds a tile: spreading the same work over all CUs with smaller tiles wins.)
GemmChoice pick(const MatmulArgs& a, const Candidate* c, int n, double* cost_out = nullptr) {
  GemmChoice best = GEMM_NONE;
  double best_cost = 0;
  const int NUM_CU = num_cu();
  for (int i = 0; i < n; i++) {
    const int64_t tiles = (int64_t)((a.m + c[i].bm - 1) / c[i].bm) * ((a.n + c[i].bn - 1) / c[i].bn) *
                          a.batches;
    const int64_t per_cu = (tiles + NUM_CU - 1) / NUM_CU;
    // (between tiles that need equally many rounds, the one that pads the product less is a few
    // percent faster: M320 N11008 on 128 x 256 41.3 us, on 256 x 128 45.3)
    const double padded = (double)tiles * c[i].bm * c[i].bn / ((double)a.m * a.n * a.batches);
    const double cost = (double)per_cu * c[i].bm * c[i].bn / c[i].eff * (1.0 + 0.02 * (padded - 1.0));
    if (best == GEMM_NONE || cost < best_cost) {
      best = c[i].id;
      best_cost = cost;
    }
  }
  if (cost_out) *cost_out = best_cost;
  return best;
}

// (the two large tiles run on 16x16x32 MFMAs: 9-16 % faster than on 32x32x16 on data that is not
// constant -- qkv 170 -> 156 us, o 68 -> 58, down 162 -> 144 -- while the smaller tiles, which are
// not bound by the power limit, gain nothing from it and stay on 32x32x16)
const Candidate DMA_TILES[] = {
    {DMA_256x192, 256, 192, 1, 1.24f}, {DMA_256x128, 256, 128, 1, 1.13f},
    {DMA_128x256, 128, 256, 1, 1.13f}, {DMA_128x192, 128, 192, 1, 0.85f}, {DMA_128x128, 128, 128, 2, 0.80f}, {DMA_128x64, 128, 64, 2, 0.60f},
    {DMA_64x64, 64, 64, 4, 0.40f}, {DMA_256x160, 256, 160, 1, 1.19f}};
constexpr int N_DMA_TILES = sizeof(DMA_TILES) / sizeof(DMA_TILES[0]);

// The tiles of the u8-weight kernel.  One tile per CU, time per tile at K 11008 / K 4096 in us:
// 256x192 195 / 78, 256x128 140 / 56, 128x128 97 / 41, 128x64 68 / 30 (two K groups; one: 73 / 32),
// 64x64 47 / 22 (four K groups; one: 58 / 25).  The two smallest tiles are bound by what the L2s
// deliver to all CUs together (M256 K11008 N4096 on 64x64: 540 MB in 47 us), the larger ones by
// the path into one CU.  Over M 70..1536 x (K, N) of the LLaMA-7B and 13B layers the choice by
// these constants is the fastest forced tile or within 5 % of it, with the weights resident in
// the Infinity Cache and with weights that come from HBM (rotated through 600 MB) alike.
const Candidate U8_TILES[] = {{U8_256x192, 256, 192, 1, 1.10f}, {U8_256x128, 256, 128, 1, 1.05f},
                              {U8_128x128, 128, 128, 1, 0.72f}, {U8_128x64, 128, 64, 2, 0.52f},
                              {U8_64x64, 64, 64, 4, 0.37f}};
constexpr int N_U8_TILES = sizeof(U8_TILES) / sizeof(U8_TILES[0]);

// With at most one tile per CU the two small tiles split K over groups of wavefronts inside the
// workgroup (more slices in flight per CU; with more tiles than CUs several workgroups per CU do
// the same).
GemmChoice u8_k_groups(const MatmulArgs& a, GemmChoice c) {
  const int bm = c == U8_128x64 ? 128 : 64;
  const int64_t tiles = (int64_t)((a.m + bm - 1) / bm) * ((a.n + 63) / 64);
  if (tiles > num_cu()) return c;
  if (c == U8_128x64 && a.k % 128 == 0) return U8_128x64_G2;
  if (c == U8_64x64 && a.k % 256 == 0) return U8_64x64_G4;
  return c;
}

// The MFMA family needs 16-byte aligned, K-contiguous rows on both operands.
GemmChoice choose(const MatmulArgs& a) {
  const int NUM_CU = num_cu();
  // "NN": both the left operand (k contiguous) and the right operand (n contiguous) are row
  // major, e.g. P.V on the head views of llama.rs:552-554.  Left rows of any alignment and any K
  // (P.V of a sequence length like 77, 257, 1500 or 2001) go to the kernel that stages the left
  // operand through registers.
  const bool nn_anyrow =
      a.stride_lx == 1 && a.stride_rx == 1 && a.stride_ry != 1 && a.stride_ox == 1 && !a.rhs_q &&
      a.load == ADR_LOAD_IDENTITY && a.k >= 1 && a.n % 8 == 0 && a.n >= 8 && a.stride_ly > 0 &&
      a.stride_lz >= 0 && !((a.stride_ry % 8) | (a.stride_rz % 8)) &&
      !(a.lhs && (uintptr_t)a.rhs % 16 != 0) &&
      // (its 16-byte loads near the end of the left operand start up to 12 bytes before the last dword)
      (int64_t)(a.batches - 1) * a.stride_lz + (int64_t)(a.m - 1) * a.stride_ly + a.k >= 12;
  // Few tiles and a long K (the first steps of whisper.rs:433-436 against 1500 frames, or a few
  // query rows against a long context): a compute unit cannot fetch much more than 100 GB/s, so
  // the product goes to the smallest row tile that still gives every workgroup a compute unit of
  // its own, on 64 columns, with K split over four groups of wavefronts -- aligned or not.
  const bool nn_dma =
      a.stride_lx == 1 && a.stride_rx == 1 && a.stride_ry != 1 && a.stride_ox == 1 && !a.rhs_q &&
      a.load == ADR_LOAD_IDENTITY && a.k % 64 == 0 && a.k >= 64 && a.n % 8 == 0 && a.n >= 8 &&
      !((a.stride_ly % 8) | (a.stride_ry % 8) | (a.stride_lz % 8) | (a.stride_rz % 8)) &&
      !(a.lhs && ((uintptr_t)a.lhs % 16 != 0 || (uintptr_t)a.rhs % 16 != 0));
  // (against the direct-to-LDS kernel the small tiles win from 16 slices on: 32 heads x 256 rows
  // x K 256 take 5.4 us there and 6.1 here, one row x K 2048 16.2 and 9.1)
  if (nn_anyrow && a.k > 192 && !(nn_dma && a.k < 1024)) {
    const int64_t cols64 = (int64_t)((a.n + 63) / 64) * a.batches;
    if ((int64_t)((a.m + 31) / 32) * cols64 <= NUM_CU) return NN_ANYROW_32x64_G4;
    if ((int64_t)((a.m + 63) / 64) * cols64 <= NUM_CU) return NN_ANYROW_64x64_G4;
  }
  if (nn_dma) {
    static const Candidate nn[] = {{DMA_NN_256x128, 256, 128, 1, 1.00f},
                                   {DMA_NN_128x128, 128, 128, 2, 0.80f}};
    return pick(a, nn, 2);
  }
  if (nn_anyrow) {
    const bool narrow = a.n <= 64 || (a.n > 128 && a.n % 128 != 0 && a.n % 128 <= 64);
    // (half the compute units or fewer on 128 columns: twice the workgroups on 64)
    const int64_t tiles128 = (int64_t)((a.m + 127) / 128) * ((a.n + 127) / 128) * a.batches;
    return narrow || 2 * tiles128 <= NUM_CU ? NN_ANYROW_128x64 : NN_ANYROW_128x128;
  }
  if (a.stride_lx != 1 || a.stride_ry != 1 || a.stride_ox != 1) return GEMM_NONE;
  if (a.k % 8 != 0 || a.k < 8) return GEMM_NONE;
  if ((a.stride_ly % 8) | (a.stride_rx % 8) | (a.stride_lz % 8) | (a.stride_rz % 8)) return GEMM_NONE;
  if (a.lhs && ((uintptr_t)a.lhs % 16 != 0 || (uintptr_t)a.rhs % 16 != 0 ||
                (uintptr_t)a.rhs_q % 8 != 0)) return GEMM_NONE;
  const bool plain = !a.rhs_q && a.load == ADR_LOAD_IDENTITY;
  // One or two K slices (the attention score product): the persistent kernel, which also scales
  // its operands on the way in where the caller asks for that (whisper.rs:424-430)
  // (not for a handful of rows: its tiles are 128 rows high; M = 1, T = 2048, 32 heads takes 9.1 us
  // on it and 4.1 on 64 x 64 tiles)
  if (!a.rhs_q && (a.k == 64 || a.k == 128) && !(a.store == STORE_ACC_BETA && a.beta != 0.0f) &&
      a.m > 64 && (int64_t)((a.m + 127) / 128) * ((a.n + 127) / 128) * a.batches >= 2 * NUM_CU)
    return a.k == 64 ? SHORTK_64 : SHORTK_128;
  if (plain && a.k % 64 == 0) {
    // Few K slices and too few tiles for the persistent kernel: a tile is dominated by its load
    // latency and its epilogue; two resident workgroups per CU overlap those phases
    if (a.k <= 256) {
      static const Candidate shortk[] = {{DMA_128x128, 128, 128, 2, 1.00f},
                                         {DMA_64x64, 64, 64, 4, 0.50f}};
      return pick(a, shortk, 2);
    }
    // (tests and benchmarks can force a tile: adr_debug_knob)
    const int forced = knob(KNOB_GEMM_TILE);
    if (forced >= 1 && forced <= N_DMA_TILES) return DMA_TILES[forced - 1].id;
    GemmChoice c = pick(a, DMA_TILES, N_DMA_TILES);
    // Up to 64 rows against a matrix of a little more than one 64 x 64 tile per CU: the CUs that
    // hold two tiles finish as late as one 128 x 128 tile would, and that tile is 0-16 % ahead
    // (K6656 N17920 m=64: 72.8 -> 61.4 us, K3072 N24576: 37.9 -> 34.6, K8192 N22016: 86.2 -> 86.6);
    // with two full rounds of the small tile it is the other way round (K4096 N32000: 54.5 / 62.0)
    if (c == DMA_64x64 && a.m <= 64 && a.batches == 1 && a.k >= 3072) {
      const int tiles64 = (a.n + 63) / 64;
      if (tiles64 > NUM_CU && 2 * tiles64 <= 3 * NUM_CU) c = DMA_128x128;
    }
    // At most one 64 x 64 tile per CU (a few dozen to a few hundred rows against a weight
    // matrix): the product is bound by how DRAM serves the weight requests -- one piece of every
    // tile row per slice, a whole weight row apart -- and pieces of 256 bytes (slices of 128)
    // stream better than pieces of 128 (K11008 N4096 m <= 256: 66 -> 46-54 us; K4096 N4096:
    // 18.5 -> 14 us).  More tiles than CUs, or larger tiles, are better off with slices of 64.
    if (c == DMA_64x64 && a.k % 128 == 0 && a.k >= 1024 &&
        (int64_t)((a.m + 63) / 64) * ((a.n + 63) / 64) * a.batches <= NUM_CU)
      return DMA_64x64_K128;
    // the same for at most one 128 x 64 tile per CU (K4096 N12288 m=128: 37.4 -> 32.3 us,
    // K11008 N4096 m=512: 81 -> 71.5)
    if (c == DMA_128x64 && a.k % 128 == 0 && a.k >= 1024 &&
        (int64_t)((a.m + 127) / 128) * ((a.n + 63) / 64) * a.batches <= NUM_CU)
      return DMA_128x64_K128;
    // (One large tile on nearly every CU with a short K used to be replaced by twice as many tiles
    // of half the size, two resident per CU, whose prologues and epilogues overlap.  With the
    // 256-row tiles on 16x16x32 MFMAs that no longer pays: over K 320 .. 1280 the 256 x 128 tile is
    // 15-28 % ahead of two 128 x 128 per CU (M2048 K1024 N4096 17.9 against 21.0 us), and 128 x 64
    // instead of 128 x 128 is within +-4 % up to K 512 and 4-12 % behind above.)
    return c;
  }
  if (a.rhs_q && a.k % 64 == 0 && a.block_size >= 8 && (a.block_size & (a.block_size - 1)) == 0) {
    // (tests and benchmarks can force a tile: adr_debug_knob; 1 + N_U8_TILES: 128 x 64 with two K
    // groups, 2 + N_U8_TILES: 64 x 64 with four, 3 + N_U8_TILES: the staged kernels below)
    const int forced = knob(KNOB_U8_TILE);
    if (forced >= 1 && forced <= N_U8_TILES) return U8_TILES[forced - 1].id;
    if (forced == N_U8_TILES + 1) return a.k % 128 == 0 ? U8_128x64_G2 : U8_128x64;
    if (forced == N_U8_TILES + 2) return a.k % 256 == 0 ? U8_64x64_G4 : U8_64x64;
    if (forced != N_U8_TILES + 3) return u8_k_groups(a, pick(a, U8_TILES, N_U8_TILES));
  }
  static const Candidate stage[] = {{STAGE_256x128, 256, 128, 2, 1.00f},
                                    {STAGE_128x128, 128, 128, 2, 0.85f},
                                    {STAGE_64x64, 64, 64, 4, 0.45f}};
  return pick(a, stage, 3);
}

// Splitting K over workgroups (needs a workspace): a product with few tiles and a long K keeps
// most compute units idle while a few walk all of K.  With `splits` workgroups per tile every
// one of them walks K / splits; a second launch sums the pieces.  The estimate is pick()'s cost
// (tile area on the busiest compute unit over the tile's efficiency) times K, 2.9e6 units per
// microsecond, plus the second launch and the fp32 pieces written and read again.
struct SplitChoice {
  GemmChoice tile;
  int splits;
  int bm, bn;
};

SplitChoice choose_split(const MatmulArgs& a, int64_t avail_bytes) {
  const SplitChoice none = {GEMM_NONE, 1, 0, 0};
#ifdef ADR_PHASE_STAMPS
  return none;  // (the diagnostic build: the workspace argument receives the stamps)
#endif
  if (avail_bytes <= 0 || a.rhs_q || a.load != ADR_LOAD_IDENTITY || a.k % 64 != 0 || a.k < 1024)
    return none;
  const GemmChoice whole = choose(a);
  if (whole != DMA_128x128 && whole != DMA_128x64 && whole != DMA_64x64 && whole != DMA_64x64_K128 &&
      whole != DMA_128x64_K128 && whole != DMA_256x128)
    return none;
  const int NUM_CU = num_cu();
  double whole_cost;
  pick(a, DMA_TILES, N_DMA_TILES, &whole_cost);
  whole_cost *= a.k;
  // With about one small tile per compute unit the time is set by the latency of the K slices,
  // not by the tile's arithmetic: 0.38 us per slice of 64 (measured: K4160 N4096 m=130 25.7 us),
  // 0.25 us where the tile walks K in slices of 128.
  const double US = 2.9e6;
  auto latency_floor = [&](int k, double us_per_slice) { return ((k / 64) * us_per_slice + 2.0) * US; };
  if (whole != DMA_256x128 && whole != DMA_128x128) {
    const bool k128 = whole == DMA_64x64_K128 || whole == DMA_128x64_K128;
    const double f = latency_floor(a.k, k128 ? 0.25 : 0.38);
    if (f > whole_cost) whole_cost = f;
  }
  static const Candidate tiles[] = {{DMA_128x128, 128, 128, 2, 0.80f}, {DMA_128x64, 128, 64, 2, 0.60f},
                                    {DMA_64x64, 64, 64, 4, 0.40f}};
  SplitChoice best = none;
  double best_cost = whole_cost * 0.85;  // (a split has to win clearly)
  for (const Candidate& t : tiles) {
    const int64_t nt = (int64_t)((a.m + t.bm - 1) / t.bm) * ((a.n + t.bn - 1) / t.bn) * a.batches;
    for (int sp = 2; sp <= 16; sp++) {
      if (a.k / sp < 256) break;  // at least four slices per piece
      if (nt * sp > 4 * (int64_t)NUM_CU) break;
      const int64_t bytes = nt * sp * t.bm * t.bn * 4;
      if (bytes > avail_bytes) break;
      const int64_t per_cu = (nt * sp + NUM_CU - 1) / NUM_CU;
      double mm = (double)per_cu * t.bm * t.bn / t.eff * ((double)a.k / sp);
      const double f = latency_floor(a.k / sp, t.id == DMA_128x128 ? 0.48 : t.id == DMA_128x64 ? 0.42 : 0.38);
      if (f > mm) mm = f;
      // second launch (4 us) + pieces written and read at some 4 TB/s
      const double extra = (4.0 + 2.0 * (double)bytes / 4.0e6) * US;
      if (mm + extra < best_cost) {
        best_cost = mm + extra;
        best = {t.id, sp, t.bm, t.bn};
      }
    }
  }
  return best;
}

}  // namespace

static bool choice_name(GemmChoice c, const char** name, bool u8 = false) {
  if (u8) {
    switch (c) {
      case STAGE_256x128: *name = "gemm_nt_u8_stage_256x128x32"; return true;
      case STAGE_128x128: *name = "gemm_nt_u8_stage_128x128x32"; return true;
      case STAGE_64x64: *name = "gemm_nt_u8_stage_64x64x64"; return true;
      default: break;
    }
  }
  switch (c) {
    case SHORTK_64: *name = "gemm_nt_mfma_persistent_128x128_k64"; return true;
    case SHORTK_128: *name = "gemm_nt_mfma_persistent_128x128_k128"; return true;
    case U8_256x192: *name = "gemm_nt_u8_mfma_256x192x64"; return true;
    case U8_256x128: *name = "gemm_nt_u8_mfma_256x128x64"; return true;
    case U8_128x128: *name = "gemm_nt_u8_mfma_128x128x64"; return true;
    case U8_128x64: *name = "gemm_nt_u8_mfma_128x64x64"; return true;
    case U8_64x64: *name = "gemm_nt_u8_mfma_64x64x64"; return true;
    case U8_128x64_G2: *name = "gemm_nt_u8_mfma_128x64x64_k2"; return true;
    case U8_64x64_G4: *name = "gemm_nt_u8_mfma_64x64x64_k4"; return true;
    case DMA_256x192: *name = "gemm_nt_mfma_dma_256x192x64"; return true;
    case DMA_256x160: *name = "gemm_nt_mfma_dma_256x160x64"; return true;
    case DMA_256x128: *name = "gemm_nt_mfma_dma_256x128x64"; return true;
    case DMA_128x256: *name = "gemm_nt_mfma_dma_128x256x64"; return true;
    case DMA_128x192: *name = "gemm_nt_mfma_dma_128x192x64"; return true;
    case DMA_128x128: *name = "gemm_nt_mfma_dma_128x128x64"; return true;
    case DMA_128x64: *name = "gemm_nt_mfma_dma_128x64x64"; return true;
    case DMA_64x64: *name = "gemm_nt_mfma_dma_64x64x64"; return true;
    case DMA_64x64_K128: *name = "gemm_nt_mfma_dma_64x64x128"; return true;
    case DMA_128x64_K128: *name = "gemm_nt_mfma_dma_128x64x128"; return true;
    case DMA_NN_256x128: *name = "gemm_nn_mfma_dma_256x128x64"; return true;
    case DMA_NN_128x128: *name = "gemm_nn_mfma_dma_128x128x64"; return true;
    case NN_ANYROW_128x128: *name = "gemm_nn_mfma_anyrow_128x128x64"; return true;
    case NN_ANYROW_128x64: *name = "gemm_nn_mfma_anyrow_128x64x64"; return true;
    case NN_ANYROW_32x64_G4: *name = "gemm_nn_mfma_anyrow_32x64x64_k4"; return true;
    case NN_ANYROW_64x64_G4: *name = "gemm_nn_mfma_anyrow_64x64x64_k4"; return true;
    case STAGE_256x128: *name = "gemm_nt_mfma_stage_256x128x32"; return true;
    case STAGE_128x128: *name = "gemm_nt_mfma_stage_128x128x32"; return true;
    case STAGE_64x64: *name = "gemm_nt_mfma_stage_64x64x64"; return true;
    default: return false;
  }
}

static hipError_t launch_choice(hipStream_t stream, const MatmulArgs& a, GemmChoice c) {
  switch (c) {
    case SHORTK_64: return launch_shortk<8>(stream, a);
    case SHORTK_128: return launch_shortk<16>(stream, a);
    case U8_256x192: return launch_u8<256, 192, 4, 2, false>(stream, a);
    // (four stages of the left operand, three slices ahead, fill the 160 KB: K11008 N4096 M2048 with
    // weights from HBM 202 -> 191 us, K4096 unchanged; the smaller tiles gain nothing from a fourth stage)
    case U8_256x128: return launch_u8<256, 128, 4, 2, true, 64, 1, 4>(stream, a);
    case U8_128x128: return launch_u8<128, 128, 4, 2, true>(stream, a);
    case U8_128x64: return launch_u8<128, 64, 2, 2, true>(stream, a);
    case U8_64x64: return launch_u8<64, 64, 2, 2, true>(stream, a);
    case U8_128x64_G2: return launch_u8<128, 64, 2, 2, true, 64, 2>(stream, a);
    case U8_64x64_G4: return launch_u8<64, 64, 2, 2, true, 64, 4>(stream, a);
    case DMA_256x192: return launch_dma<256, 192, 4, 2, 6, 1, false, 64, true>(stream, a);
    case DMA_256x160: return launch_dma<256, 160, 4, 2, 6, 1, false, 64, true>(stream, a);
    case DMA_256x128: return launch_dma<256, 128, 4, 2, 7, 1, false, 64, true>(stream, a);
    case DMA_128x256: return launch_dma<128, 256, 2, 4, 3, 1, false, 64, true>(stream, a);
    case DMA_128x192: return launch_dma<128, 192, 2, 2, 3, 1>(stream, a);
    // (eight wavefronts of 32 x 64 on 16x16x32 MFMAs: two per SIMD overlap each other's slice
    // chains; 2-7 % ahead of four wavefronts of 64 x 64 on 32x32x16: M1024 K4096 N4096 37.8 -> 35.3 us.
    // Three left and four right stages with the transfers split by wavefront role: another 2-9 %,
    // M2056 K4096 N1024 29.2 -> 26.5, M768 K4096 N4096 30.4 -> 27.8; the same on the 128 x 256,
    // 128 x 192, 128 x 64 and 64 x 64 tiles changed nothing or lost.)
    case DMA_128x128: return launch_dma<128, 128, 4, 2, 7, 1, false, 64, true>(stream, a);
    case DMA_128x64: return launch_dma<128, 64, 2, 2, 3, 2>(stream, a);
    case DMA_64x64: return launch_dma<64, 64, 2, 2, 3, 3>(stream, a);
    case DMA_64x64_K128: return launch_dma<64, 64, 2, 2, 3, 1, false, 128>(stream, a);
    case DMA_128x64_K128: return launch_dma<128, 64, 2, 2, 3, 1, false, 128>(stream, a);
    case DMA_NN_256x128: return launch_dma<256, 128, 4, 2, 3, 1, true>(stream, a);
    case DMA_NN_128x128: return launch_dma<128, 128, 2, 2, 2, 2, true>(stream, a);
    case NN_ANYROW_128x128: return launch_nn_anyrow<128, 128, 4, 2, 1>(stream, a);
    case NN_ANYROW_128x64: return launch_nn_anyrow<128, 64, 4, 2, 1>(stream, a);
    case NN_ANYROW_32x64_G4: return launch_nn_anyrow<32, 64, 1, 2, 4>(stream, a);
    case NN_ANYROW_64x64_G4: return launch_nn_anyrow<64, 64, 2, 2, 4>(stream, a);
    case STAGE_256x128: return launch_stage<256, 128, 32, 2, 2, 2>(stream, a);
    case STAGE_128x128: return launch_stage<128, 128, 32, 2, 2, 2>(stream, a);
    case STAGE_64x64: return launch_stage<64, 64, 64, 2, 2, 2>(stream, a);
    default: return hipErrorInvalidValue;
  }
}

// A few rows past a multiple of the tile height (M = 2056 = 8 x 257 image tokens) would add a
// whole row of tiles that do almost no useful work and break an otherwise even split over the
// CUs (2048 x 4096 is exactly one 256 x 128 tile per CU).  Such products are issued as two
// launches: the rows up to the last multiple of 128, and the remaining rows as a small problem
// of their own.  Rows are independent in every store operator; the causal mask compares absolute
// row numbers and is therefore left alone.
static bool split_m_tail(const MatmulArgs& a, MatmulArgs& head, MatmulArgs& tail) {
  const int t = a.m % 128;
  if (a.mask != ADR_MASK_NONE || a.rhs_q || a.m < 1024 || t == 0 || t > 32) return false;
  head = a;
  head.m = a.m - t;
  tail = a;
  tail.m = t;
  // (the plan query passes no pointers)
  tail.lhs = a.lhs ? a.lhs + (int64_t)head.m * a.stride_ly : nullptr;
  tail.output = a.output ? a.output + (int64_t)head.m * a.stride_oy : nullptr;
  const GemmChoice ca = choose(a), ch = choose(head), ct = choose(tail);
  auto dma_tile = [](GemmChoice c) {
    return c == DMA_256x192 || c == DMA_256x160 || c == DMA_256x128 || c == DMA_128x256 || c == DMA_128x192 || c == DMA_128x128 ||
           c == DMA_128x64 || c == DMA_64x64;
  };
  if (!dma_tile(ca) || !dma_tile(ch) || !dma_tile(ct)) return false;
  // pick()'s cost (tile area on the busiest CU over efficiency) times K is proportional to the
  // time of a launch; one more launch is priced at 3 us (2.9e6 of those units per us, measured)
  double whole, first, rest;
  pick(a, DMA_TILES, N_DMA_TILES, &whole);
  pick(head, DMA_TILES, N_DMA_TILES, &first);
  pick(tail, DMA_TILES, N_DMA_TILES, &rest);
  return (first + rest) * a.k + 8.7e6 < whole * a.k;
}

static const char* split_name(const SplitChoice& sc) {
  // "gemm_nt_mfma_dma_128x128x64_splitk4": the tile, then the number of pieces
  static const char* const names[3][15] = {
      {"gemm_nt_mfma_dma_128x128x64_splitk2", "gemm_nt_mfma_dma_128x128x64_splitk3", "gemm_nt_mfma_dma_128x128x64_splitk4",
       "gemm_nt_mfma_dma_128x128x64_splitk5", "gemm_nt_mfma_dma_128x128x64_splitk6", "gemm_nt_mfma_dma_128x128x64_splitk7",
       "gemm_nt_mfma_dma_128x128x64_splitk8", "gemm_nt_mfma_dma_128x128x64_splitk9", "gemm_nt_mfma_dma_128x128x64_splitk10",
       "gemm_nt_mfma_dma_128x128x64_splitk11", "gemm_nt_mfma_dma_128x128x64_splitk12", "gemm_nt_mfma_dma_128x128x64_splitk13",
       "gemm_nt_mfma_dma_128x128x64_splitk14", "gemm_nt_mfma_dma_128x128x64_splitk15", "gemm_nt_mfma_dma_128x128x64_splitk16"},
      {"gemm_nt_mfma_dma_128x64x64_splitk2", "gemm_nt_mfma_dma_128x64x64_splitk3", "gemm_nt_mfma_dma_128x64x64_splitk4",
       "gemm_nt_mfma_dma_128x64x64_splitk5", "gemm_nt_mfma_dma_128x64x64_splitk6", "gemm_nt_mfma_dma_128x64x64_splitk7",
       "gemm_nt_mfma_dma_128x64x64_splitk8", "gemm_nt_mfma_dma_128x64x64_splitk9", "gemm_nt_mfma_dma_128x64x64_splitk10",
       "gemm_nt_mfma_dma_128x64x64_splitk11", "gemm_nt_mfma_dma_128x64x64_splitk12", "gemm_nt_mfma_dma_128x64x64_splitk13",
       "gemm_nt_mfma_dma_128x64x64_splitk14", "gemm_nt_mfma_dma_128x64x64_splitk15", "gemm_nt_mfma_dma_128x64x64_splitk16"},
      {"gemm_nt_mfma_dma_64x64x64_splitk2", "gemm_nt_mfma_dma_64x64x64_splitk3", "gemm_nt_mfma_dma_64x64x64_splitk4",
       "gemm_nt_mfma_dma_64x64x64_splitk5", "gemm_nt_mfma_dma_64x64x64_splitk6", "gemm_nt_mfma_dma_64x64x64_splitk7",
       "gemm_nt_mfma_dma_64x64x64_splitk8", "gemm_nt_mfma_dma_64x64x64_splitk9", "gemm_nt_mfma_dma_64x64x64_splitk10",
       "gemm_nt_mfma_dma_64x64x64_splitk11", "gemm_nt_mfma_dma_64x64x64_splitk12", "gemm_nt_mfma_dma_64x64x64_splitk13",
       "gemm_nt_mfma_dma_64x64x64_splitk14", "gemm_nt_mfma_dma_64x64x64_splitk15", "gemm_nt_mfma_dma_64x64x64_splitk16"}};
  const int t = sc.tile == DMA_128x128 ? 0 : sc.tile == DMA_128x64 ? 1 : 2;
  return names[t][sc.splits - 2];
}

int64_t mfma_gemm_workspace_bytes(const MatmulArgs& a, int64_t avail) {
  const SplitChoice sc = choose_split(a, avail);
  return sc.tile == GEMM_NONE ? 0 : split_workspace_bytes(a, sc.bm, sc.bn, sc.splits);
}

bool mfma_gemm_supported(const MatmulArgs& a, const char** name) {
  const SplitChoice sc = choose_split(a, a.workspace_bytes);
  if (sc.tile != GEMM_NONE) {
    *name = split_name(sc);
    return true;
  }
  MatmulArgs head, tail;
  if (split_m_tail(a, head, tail)) return choice_name(choose(head), name);
  return choice_name(choose(a), name);
}

hipError_t launch_mfma_gemm(hipStream_t stream, const MatmulArgs& a) {
  const SplitChoice sc = choose_split(a, a.workspace ? a.workspace_bytes : 0);
  if (sc.tile == DMA_128x128) return launch_dma_split<128, 128, 2, 2, 3, 1>(stream, a, sc.splits);
  if (sc.tile == DMA_128x64) return launch_dma_split<128, 64, 2, 2, 3, 2>(stream, a, sc.splits);
  if (sc.tile == DMA_64x64) return launch_dma_split<64, 64, 2, 2, 3, 3>(stream, a, sc.splits);
  MatmulArgs head, tail;
  if (split_m_tail(a, head, tail)) {
    const hipError_t e = launch_choice(stream, head, choose(head));
    if (e != hipSuccess) return e;
    return launch_choice(stream, tail, choose(tail));
  }
  return launch_choice(stream, a, choose(a));
}

static MatmulArgs u8_args(half_t* out, const half_t* lhs, const uint8_t* rhs, const half_t* scales,
                          int m, int p, int n, int block_size, float beta) {
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
  return a;
}

// Name of the tiled kernel the u8 product would run on (nullptr: none covers it).  The plan query
// has no pointers: a non-null marker stands for the weights, alignment is assumed.
const char* gemm_u8_mfma_plan(int m, int p, int n, int block_size) {
  const MatmulArgs a = u8_args(nullptr, nullptr, (const uint8_t*)16, nullptr, m, p, n, block_size, 0.0f);
  const char* name = nullptr;
  return choice_name(choose(a), &name, true) ? name : nullptr;
}

// Estimated time of the u8 product on the tiled u8 kernel, in us (negative: that kernel does not
// cover it): pick()'s cost of the chosen tile times K.  4 us + 4.3e-7 us per unit fits one tile per
// CU of 64 x 64 (K11008 53-59 us, K4096 23-26) and of 128 x 64 (71-85, 30-35) on weights that come
// from HBM (3.5e-7 where the Infinity Cache holds them: 47 / 21 and 68 / 30).
double gemm_u8_mfma_estimate_us(int m, int p, int n, int block_size) {
  const MatmulArgs a = u8_args(nullptr, nullptr, (const uint8_t*)16, nullptr, m, p, n, block_size, 0.0f);
  if (!(p % 64 == 0 && block_size >= 8 && (block_size & (block_size - 1)) == 0)) return -1.0;
  double cost;
  pick(a, U8_TILES, N_U8_TILES, &cost);
  return 4.0 + cost * p * 4.3e-7;
}

bool gemm_u8_mfma_supported(const half_t* lhs, const uint8_t* rhs, const half_t* scales, int m, int p,
                            int n, int block_size) {
  const MatmulArgs a = u8_args(nullptr, lhs, rhs, scales, m, p, n, block_size, 0.0f);
  return choose(a) != GEMM_NONE;
}

hipError_t launch_gemm_u8_mfma(hipStream_t stream, half_t* out, const half_t* lhs,
                               const uint8_t* rhs, const half_t* scales, int m, int p, int n,
                               int block_size, float beta) {
  return launch_mfma_gemm(stream, u8_args(out, lhs, rhs, scales, m, p, n, block_size, beta));
}

}  // namespace adr
