// RMSNorm + router GEMM + 1x128 quant in one pass over x
// (linghe/utils/norm.py:616-784, output_mode 0; kernel :616-687):
//   r = rsqrt(mean(x^2) + eps);  y = (x*r)*gamma  (fp32)
//   y_bf16 = bf16(y);  logits = y @ W^T (fp32);  q, s = 1x128 quant of y
//
// The only contraction on this path, so the only place MFMA is used.  The
// reference multiplies fp32 y by W with tl.dot; here y is split into two bf16
// terms, y = hi + lo (hi = bf16(y) is the y_bf16 output itself, lo = bf16(y - hi),
// what is left is below 2^-17 |y|), W is bf16 already, and the two products go
// through v_mfma_f32_32x32x16_bf16 with fp32 accumulation: bf16 products are
// exact in fp32, so the result carries the accuracy of an fp32 GEMM at the bf16
// MFMA rate.
//
// Two kernels share this scheme: the one below streams the rows twice (statistic,
// then the blocks) and takes any K; rmsnorm_router_quant_resident_kernel further
// down keeps the rows in registers when they fit.
//
// An fp32 router weight (what Megatron keeps) is split the same way, W = hi + lo with
// hi = bf16(W), lo = bf16(W - hi) (what is left is below 2^-17 |W|), and the two planes
// are laid side by side as "virtual" columns 2n (hi) and 2n + 1 (lo): the GEMM runs on
// 2N bf16 columns and the epilogue adds each pair, which sits in neighbouring lanes.
// More than 512 virtual columns are cut into chunks of at most 512, one launch each;
// only the first launch writes y, the codes, the scales and the statistic.
//
// One workgroup (4 or 8 waves) owns 32 rows and all N <= 512 logits of them and walks K
// in blocks of 128 (one quantisation group per row):
//   each thread normalises 2 rows x 8 columns of the block (16 lanes per row, so
//   every global access is coalesced), quantises them with the row's 1x128 scale
//   (a DPP reduction over the 16 lanes), stores y_bf16 and the codes, and writes
//   the hi/lo A operands to LDS in MFMA lane order; after one barrier each wave
//   multiplies the whole 32x128 block by its N/4 columns of W.
// Lane l of a wave holds, as MFMA wants it, row l%32 and 8 consecutive k of a
// 16-wide k step.  Which 16 of the block's 128 columns form step j is free as long
// as A and B agree: step j takes columns 8j..8j+7 (lanes 0-31) and 64+8j..64+8j+7
// (lanes 32-63), so that a lane's eight B loads of a block cover one contiguous
// 128-byte line of its W row; the 32x32 result has column l%32 and rows
// (v/4)*8 + (l/32)*4 + v%4 in register v.
#include "fq_device.hpp"
#include "fq_launch.h"
#include "fq_policy.hpp"

namespace fq {

// cache hints: fq_policy.hpp

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));

constexpr int kRouterRows = 32;

struct RouterShared {
  uint4 a[2][2][8][64];  // [buffer][hi, lo][k step][lane slot]: A operands of one 32x128 block
  float rstd[kRouterRows];
};

// 1/sqrt(mean(x^2) + eps) of four consecutive rows by one wave (their loads in
// flight together), the arithmetic of the row kernels: 8-element group sums added
// in double, so the value does not depend on the split
__device__ __forceinline__ void router_rows_rstd(const uint16_t* rows, int n, float eps, float (&out)[4]) {
  const int lane = tid_x() & 63;
  const int chunks = n >> 3;
  double ss[4] = {0.0, 0.0, 0.0, 0.0};
  for (int c0 = 0; c0 < chunks; c0 += 256) {
    uint4 v[4][4];
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * 64 + lane;
        v[k][u] = make_uint4(0, 0, 0, 0);
        if (c < chunks) v[k][u] = *(const uint4*)(rows + (int64_t)k * n + c * 8);
      }
#pragma unroll
    for (int k = 0; k < 4; ++k)
#pragma unroll
      for (int u = 0; u < 4; ++u) ss[k] += (double)sumsq8(v[k][u]);
  }
#pragma unroll
  for (int k = 0; k < 4; ++k) out[k] = 1.0f / sqrtf((float)wave_sum_d(ss[k]) / (float)n + eps);
}

// W [N, K] -> B operands in the order the main kernel reads them: one 16-byte piece
// per (k block, 32-column tile, k step, lane), so that every B load of a wave is
// 1 KB of contiguous memory.  (Read straight from the row-major matrix, each lane of
// such a load would touch a cache line of its own.)  One launch packs the `vtiles`
// 32-column tiles of one chunk, starting at virtual column vcol0; with an fp32 weight
// virtual column v is plane v & 1 (0: bf16(W), 1: bf16 of the rest) of column v >> 1.
template <bool FP32W>
__global__ __launch_bounds__(256) void pack_router_weight_kernel(const void* __restrict__ wr,
                                                                 uint4* __restrict__ packed, int K, int vcol0,
                                                                 int vtiles) {
  const int64_t idx = (int64_t)wg_x() * 256 + tid_x();  // piece number inside the chunk
  const int64_t total = (int64_t)vtiles * 32 * K / 8;
  if (idx >= total) return;
  const int lane = (int)(idx & 63);
  int64_t rest = idx >> 6;
  const int j = (int)(rest & 7);
  rest >>= 3;
  const int tile = (int)(rest % vtiles);
  const int kb = (int)(rest / vtiles);
  const int v = vcol0 + tile * 32 + (lane & 31);
  const int k = kb * kGroup + (lane >> 5) * 64 + j * 8;
  if constexpr (!FP32W) {
    packed[idx] = *(const uint4*)((const uint16_t*)wr + (int64_t)v * K + k);
  } else {
    const float4* src = (const float4*)((const float*)wr + (int64_t)(v >> 1) * K + k);
    const float4 a = src[0], b = src[1];
    float w[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    const uint4 hi = pack8_bf16(w);
    if (v & 1) {
      float back[8], lo[8];
      unpack8(hi, back);
#pragma unroll
      for (int i = 0; i < 8; ++i) lo[i] = w[i] - back[i];
      packed[idx] = pack8_bf16(lo);
    } else {
      packed[idx] = hi;
    }
  }
}

// Where a launch puts its logits.  A chunk holds `real` columns of the [M, n_logits] matrix
// starting at col0; with PAIR the accumulator columns come in (hi, lo) pairs in neighbouring
// lanes and their sum is one real column.
struct LogitsOut {
  float* logits;
  int n_logits;  // row stride
  int col0;      // first real column of this launch
};
template <bool PAIR>
__device__ __forceinline__ void store_logit(const LogitsOut& o, int64_t row, int vcol, float v) {
  if constexpr (PAIR) {
    v += dpp_mov<kDppQuadXor1>(v);  // lanes 2i, 2i+1 hold the two planes of one column
    if ((vcol & 1) == 0) o.logits[row * o.n_logits + o.col0 + (vcol >> 1)] = v;
  } else {
    o.logits[row * o.n_logits + o.col0 + vcol] = v;
  }
}

// WAVES waves per workgroup, TPW column tiles (of 32 logits) per wave: N = 32 * WAVES * TPW.
// With 8 waves a thread owns one row x 8 columns of a k block, with 4 waves two rows.
// SIDE: this launch also writes y, the codes, the scales and the statistic (the first chunk does)
template <int KIND, bool ROUND, int TPW, int WAVES, bool PAIR, bool SIDE>
__global__ __launch_bounds__(64 * WAVES) void rmsnorm_router_quant_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma, const uint4* __restrict__ wpacked,
    uint16_t* __restrict__ y, float* __restrict__ rstd_out, LogitsOut lout, uint8_t* __restrict__ q,
    float* __restrict__ s, int64_t M, int K, float eps) {
  __shared__ RouterShared sh;
  const int lane = tid_x() & 63;
  const int wave = tid_x() >> 6;
  const int64_t row0 = (int64_t)wg_x() * kRouterRows;

  constexpr int NT = TPW;
  constexpr int RPT = 8 / WAVES;  // rows per thread: 2 with 4 waves, 1 with 8
  // ---- statistic of the 32 rows, four at a time per wave
#pragma unroll 1
  for (int u = 0; u < kRouterRows / WAVES; u += 4) {
    const int r = wave * (kRouterRows / WAVES) + u;
    float rs[4];
    router_rows_rstd(x + (row0 + r) * K, K, eps, rs);
    if (lane < 4) {
      const float mine = lane == 0 ? rs[0] : lane == 1 ? rs[1] : lane == 2 ? rs[2] : rs[3];
      sh.rstd[r + lane] = mine;
      if constexpr (SIDE) rstd_out[row0 + r + lane] = mine;
    }
  }
  __syncthreads();

  // producer side: thread (rg, cg) holds rows RPT rg .. and columns 8 cg .. 8 cg + 7 of
  // the k block, so 16 lanes read, and write, 256 (128 for the codes) contiguous bytes
  const int cg = tid_x() & 15;
  const int rg = tid_x() >> 4;
  const float r0 = sh.rstd[RPT * rg], r1 = sh.rstd[RPT * rg + RPT - 1];
  const uint16_t* xrow = x + (row0 + RPT * rg) * K + cg * 8;
  uint16_t* yrow = y + (row0 + RPT * rg) * K + cg * 8;
  uint8_t* qrow = q + (row0 + RPT * rg) * K + cg * 8;
  // consumer side (MFMA lane order)
  const int arow = lane & 31;
  const int half = lane >> 5;
  floatx16_t acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

  const int kblocks = K / kGroup;
  // operands of a k block: this wave's NT column tiles of W (B operands), the
  // thread's two rows of x and its piece of gamma.  Only one workgroup of these fits
  // a CU's share of the rows, so the next block's operands are fetched while the
  // current one is worked on.
  auto fetch_w = [&](int kb, uint4 (&b)[NT][8]) {
    const uint4* wp = wpacked + ((int64_t)(kb * WAVES + wave) * NT) * 8 * 64 + lane;
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int j = 0; j < 8; ++j) b[t][j] = wp[(t * 8 + j) * 64];
  };
  auto fetch_x = [&](int kb, uint4 (&xr)[RPT], uint4& gr) {
#pragma unroll
    for (int u = 0; u < RPT; ++u) xr[u] = *(const uint4*)(xrow + (int64_t)u * K + kb * kGroup);
    gr = *(const uint4*)(gamma + kb * kGroup + cg * 8);
  };
  // column chunk cg of the block is k step (cg & 7), lanes 32*(cg >> 3).. of the A
  // operand; the row position is XORed with the k step so that the 16-byte LDS
  // writes of the eight lanes of a row group fall into different banks
  const int aj = cg & 7;
  const int ahalf = cg >> 3;

  // one k block: normalise / quantise / store the thread's piece, publish the A
  // operands, then multiply the whole block by this wave's columns of W
  auto step = [&](int kb, const uint4 (&xr)[RPT], const uint4& gr, const uint4 (&b)[NT][8]) {
    const int buf = kb & 1;
    float g[8];
    unpack8(gr, g);
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
      const float r = u ? r1 : r0;
      float a[8], yv[8];
      unpack8(xr[u], a);
      float m = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        yv[i] = (a[i] * r) * g[i];
        m = fmaxf(m, fabsf(yv[i]));
      }
      const uint4 hi = pack8_bf16(yv);
      float back[8], lo[8];
      unpack8(hi, back);
#pragma unroll
      for (int i = 0; i < 8; ++i) lo[i] = yv[i] - back[i];
      const int slot = ahalf * 32 + ((RPT * rg + u) ^ aj);
      sh.a[buf][0][aj][slot] = hi;
      sh.a[buf][1][aj][slot] = pack8_bf16(lo);
      if constexpr (SIDE) {
        m = row16_max(m);
        const float sc = make_scale<KIND, ROUND>(m);
        store16<Policy::kStoreHintRouter>(yrow + (int64_t)u * K + kb * kGroup, hi);
        const uint2 pk = quantize8<KIND, ROUND>(yv, make_quantum<ROUND>(sc));
        store8<Policy::kStoreHintRouter>(qrow + (int64_t)u * K + kb * kGroup, pk);
        if (cg == 0) s[(int64_t)kb * M + row0 + RPT * rg + u] = sc;
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int slot = half * 32 + (arow ^ j);
      const bf16x8_t ahi = __builtin_bit_cast(bf16x8_t, sh.a[buf][0][j][slot]);
      const bf16x8_t alo = __builtin_bit_cast(bf16x8_t, sh.a[buf][1][j][slot]);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const bf16x8_t bw = __builtin_bit_cast(bf16x8_t, b[t][j]);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi, bw, acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(alo, bw, acc[t], 0, 0, 0);
      }
    }
  };

  // x comes from HBM (its second read may still find it in a cache), W from L2: x is
  // fetched kAhead blocks ahead, W one block ahead.  The loop is unrolled over the
  // ring of kAhead operand sets so that a set is refilled in place right after it
  // was used: no register is copied while its load is still in flight.
  constexpr int kAhead = 4;
  uint4 b[2][NT][8], xq[kAhead][RPT], gq[kAhead];
  fetch_w(0, b[0]);
#pragma unroll
  for (int d = 0; d < kAhead; ++d)
    if (d < kblocks) fetch_x(d, xq[d], gq[d]);
#pragma unroll 1
  for (int kb0 = 0; kb0 < kblocks; kb0 += kAhead) {
#pragma unroll
    for (int d = 0; d < kAhead; ++d) {
      const int kb = kb0 + d;
      if (kb < kblocks) {
        if (kb + 1 < kblocks) fetch_w(kb + 1, b[(d + 1) & 1]);
        step(kb, xq[d], gq[d], b[d & 1]);
        if (kb + kAhead < kblocks) fetch_x(kb + kAhead, xq[d], gq[d]);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int col = (wave * NT + t) * 32 + arow;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = (v / 4) * 8 + half * 4 + (v % 4);
      store_logit<PAIR>(lout, row0 + row, col, acc[t][v]);
    }
  }
}


// The same operation for K == 128 * KB with the workgroup's rows of x held in
// registers, so that x is read from memory once and the GEMM does not wait for the
// statistic.  rstd is a per-row factor of y, hence of the logits:
//   logits[r, :] = rstd[r] * sum_k (x[r,k] * gamma[k]) * W[:, k]
// and z = x * gamma is EXACT in fp32 (two 8-bit significands), as is its split
// z = hi + lo into two bf16 values, so the contraction carries only the rounding of
// the fp32 accumulation and one final multiplication by rstd.
//   sweep 1, per k block as x arrives: z -> hi/lo A operands in LDS -> MFMA; the sum
//     of squares accumulates beside it (8-element group sums added in double, the
//     arithmetic of the row kernels); the next block's W loads are issued between
//     the MFMAs so that the memory pipeline and the matrix cores work together;
//   sweep 2, from registers: logits *= rstd; y = (x*rstd)*gamma -> bf16, codes and
//     scales, streamed out.
template <int KIND, bool ROUND, int TPW, int WAVES, int KB, int WDEPTH, bool PAIR>
__global__ __launch_bounds__(64 * WAVES) void rmsnorm_router_quant_resident_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma, const uint4* __restrict__ wpacked,
    uint16_t* __restrict__ y, float* __restrict__ rstd_out, LogitsOut lout, uint8_t* __restrict__ q,
    float* __restrict__ s, int64_t M, int K, float eps) {
  __shared__ RouterShared sh;
  __shared__ uint4 sgamma[KB * 16];  // gamma, 8 columns per piece
  const int lane = tid_x() & 63;
  const int wave = tid_x() >> 6;
  const int64_t row0 = (int64_t)wg_x() * kRouterRows;
  constexpr int NT = TPW;
  constexpr int RPT = 8 / WAVES;
  constexpr int kAhead = 6;  // k blocks of x in flight ahead of the one worked on
  constexpr int kWAhead = WDEPTH - 1;  // k blocks of W in flight ahead of the one worked on
  const int cg = tid_x() & 15;
  const int rg = tid_x() >> 4;
  const uint16_t* xrow = x + (row0 + RPT * rg) * K + cg * 8;
  const int aj = cg & 7;
  const int ahalf = cg >> 3;
  const int arow = lane & 31;
  const int half = lane >> 5;
  constexpr int kblocks = KB;  // a constant trip count lets the compiler schedule across blocks

  floatx16_t acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;

  uint4 xr[KB][RPT], b[WDEPTH][NT][8];
  double ss[RPT];
#pragma unroll
  for (int u = 0; u < RPT; ++u) ss[u] = 0.0;
  const uint4* wlane = wpacked + (int64_t)wave * NT * 8 * 64 + lane;
  auto w_piece = [&](int kb, int t, int j) { return wlane[((int64_t)kb * WAVES * NT + t) * 8 * 64 + j * 64]; };
  auto fetch_x = [&](int kb, uint4 (&xk)[RPT]) {
#pragma unroll
    for (int u = 0; u < RPT; ++u) xk[u] = load16<Policy::kLoadHintRouter>(xrow + (int64_t)u * K + kb * kGroup);
  };
#pragma unroll
  for (int d = 0; d < kWAhead; ++d)
    if (d < kblocks) {
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int j = 0; j < 8; ++j) b[d][t][j] = w_piece(d, t, j);
    }
#pragma unroll
  for (int d = 0; d < kAhead; ++d)
    if (d < kblocks) fetch_x(d, xr[d]);
  for (int p = tid_x(); p < kblocks * 16; p += 64 * WAVES) sgamma[p] = *(const uint4*)(gamma + p * 8);
  __syncthreads();

  // ---- sweep 1, software pipelined: the A operands of block kb + 1 are produced
  // while the matrix cores work on block kb (double-buffered in LDS, one barrier
  // per block)
  auto produce = [&](int kb, const uint4 (&xk)[RPT]) {
    float g[8];
    unpack8(sgamma[kb * 16 + cg], g);
#pragma unroll
    for (int u = 0; u < RPT; ++u) {
      float a[8], z[8], back[8], lo[8];
      unpack8(xk[u], a);
      ss[u] += (double)sumsq8(xk[u]);
#pragma unroll
      for (int i = 0; i < 8; ++i) z[i] = a[i] * g[i];
      const uint4 hi = pack8_bf16(z);
      unpack8(hi, back);
#pragma unroll
      for (int i = 0; i < 8; ++i) lo[i] = z[i] - back[i];
      const int slot = ahalf * 32 + ((RPT * rg + u) ^ aj);
      sh.a[kb & 1][0][aj][slot] = hi;
      sh.a[kb & 1][1][aj][slot] = pack8_bf16(lo);
    }
  };
  produce(0, xr[0]);
  if (kAhead < kblocks) fetch_x(kAhead, xr[kAhead]);
  __syncthreads();
#pragma unroll
  for (int kb = 0; kb < kblocks; ++kb) {
    const int buf = kb & 1;
    const bool more = kb + kWAhead < kblocks;
    const int kNext = (kb + kWAhead) % WDEPTH;
    if (kb + 1 < kblocks) {
      produce(kb + 1, xr[kb + 1]);
      if (kb + 1 + kAhead < kblocks) fetch_x(kb + 1 + kAhead, xr[kb + 1 + kAhead]);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if (more) {
#pragma unroll
        for (int t = 0; t < NT; ++t) b[kNext][t][j] = w_piece(kb + kWAhead, t, j);
      }
      const int slot = half * 32 + (arow ^ j);
      const bf16x8_t ahi = __builtin_bit_cast(bf16x8_t, sh.a[buf][0][j][slot]);
      const bf16x8_t alo = __builtin_bit_cast(bf16x8_t, sh.a[buf][1][j][slot]);
#pragma unroll
      for (int t = 0; t < NT; ++t) {
        const bf16x8_t bw = __builtin_bit_cast(bf16x8_t, b[kb % WDEPTH][t][j]);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ahi, bw, acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(alo, bw, acc[t], 0, 0, 0);
      }
    }
    __syncthreads();
  }

  // ---- statistic
  float rs[RPT];
#pragma unroll
  for (int u = 0; u < RPT; ++u) {
    rs[u] = 1.0f / sqrtf((float)row16_sum_d(ss[u]) / (float)K + eps);
    if (cg == 0) {
      sh.rstd[RPT * rg + u] = rs[u];
      rstd_out[row0 + RPT * rg + u] = rs[u];
    }
  }
  __syncthreads();
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int col = (wave * NT + t) * 32 + arow;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int row = (v / 4) * 8 + half * 4 + (v % 4);
      store_logit<PAIR>(lout, row0 + row, col, acc[t][v] * sh.rstd[row]);
    }
  }

  // ---- sweep 2
  uint16_t* yrow = y + (row0 + RPT * rg) * K + cg * 8;
  uint8_t* qrow = q + (row0 + RPT * rg) * K + cg * 8;
#pragma unroll
  for (int kb = 0; kb < kblocks; ++kb) {
    {
      float g[8];
      unpack8(sgamma[kb * 16 + cg], g);
#pragma unroll
      for (int u = 0; u < RPT; ++u) {
        float a[8], yv[8];
        unpack8(xr[kb][u], a);
        float m = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          yv[i] = (a[i] * rs[u]) * g[i];
          m = fmaxf(m, fabsf(yv[i]));
        }
        m = row16_max(m);
        const float sc = make_scale<KIND, ROUND>(m);
        store16<Policy::kStoreHintRouter>(yrow + (int64_t)u * K + kb * kGroup, pack8_bf16(yv));
        const uint2 pk = quantize8<KIND, ROUND>(yv, make_quantum<ROUND>(sc));
        store8<Policy::kStoreHintRouter>(qrow + (int64_t)u * K + kb * kGroup, pk);
        if (cg == 0) s[(int64_t)kb * M + row0 + RPT * rg + u] = sc;
      }
    }
  }
}

int64_t rmsnorm_router_scratch_bytes(int K, int N, int weight_fp32) {
  return (int64_t)N * K * (weight_fp32 ? 4 : 2);  // the bf16 planes of W in operand order
}

// W [N, K] (bf16 or fp32) -> the operand order of the main kernels, chunk by chunk of 512 virtual
// columns.  A router weight changes once per optimiser step, so a caller can pack it once and
// reuse the result for every forward in between.
hipError_t launch_pack_router_weight(const void* wr, int weight_fp32, void* wpacked, int K, int N,
                                     hipStream_t stream) {
  const int vcols = weight_fp32 ? 2 * N : N;  // virtual bf16 columns
  for (int v0 = 0; v0 < vcols; v0 += 512) {
    const int vtiles = (vcols - v0 < 512 ? vcols - v0 : 512) / 32;
    uint4* chunk_w = (uint4*)wpacked + (int64_t)v0 * K / 8;
    const int64_t pieces = (int64_t)vtiles * 32 * K / 8;
    const dim3 pgrid((unsigned)((pieces + 255) / 256));
    if (weight_fp32)
      hipLaunchKernelGGL(pack_router_weight_kernel<true>, pgrid, dim3(256), 0, stream, wr, chunk_w, K, v0, vtiles);
    else
      hipLaunchKernelGGL(pack_router_weight_kernel<false>, pgrid, dim3(256), 0, stream, wr, chunk_w, K, v0, vtiles);
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
  return hipSuccess;
}

// the main kernels on a weight already in operand order
hipError_t launch_rmsnorm_router_quant_packed(const void* x, const void* gamma, const void* wpacked,
                                              int weight_fp32, void* y, float* rstd, float* logits, void* q,
                                              float* s, int64_t M, int K, int N, float eps, int round_scale,
                                              int kind, hipStream_t stream) {
  if (M == 0) return hipSuccess;
  const int vcols = weight_fp32 ? 2 * N : N;  // virtual bf16 columns
  const dim3 grid((unsigned)(M / kRouterRows));
#define FQ_ROUTER_ARGS(WAVESV)                                                                                  \
  grid, dim3(64 * WAVESV), 0, stream, (const uint16_t*)x, (const uint16_t*)gamma, (const uint4*)chunk_w,        \
      (uint16_t*)y, rstd, lout, (uint8_t*)q, s, M, K, eps
#define FQ_ROUTER_STREAMED(KINDV, ROUNDV, TPWV, WAVESV)                                                         \
  if (first)                                                                                                    \
    hipLaunchKernelGGL((rmsnorm_router_quant_kernel<KINDV, ROUNDV, TPWV, WAVESV, PAIRV, true>),                 \
                       FQ_ROUTER_ARGS(WAVESV));                                                                 \
  else                                                                                                          \
    hipLaunchKernelGGL((rmsnorm_router_quant_kernel<KINDV, ROUNDV, TPWV, WAVESV, PAIRV, false>),                \
                       FQ_ROUTER_ARGS(WAVESV))
#define FQ_ROUTER_RESIDENT(KINDV, ROUNDV, TPWV, WAVESV)                                                         \
  if (single && K == 2048)                                                                                      \
    hipLaunchKernelGGL((rmsnorm_router_quant_resident_kernel<KINDV, ROUNDV, TPWV, WAVESV, 16, 2, PAIRV>),       \
                       FQ_ROUTER_ARGS(WAVESV));                                                                 \
  else if (single && K == 1024)                                                                                 \
    hipLaunchKernelGGL((rmsnorm_router_quant_resident_kernel<KINDV, ROUNDV, TPWV, WAVESV, 8, 2, PAIRV>),        \
                       FQ_ROUTER_ARGS(WAVESV));                                                                 \
  else {                                                                                                        \
    FQ_ROUTER_STREAMED(KINDV, ROUNDV, TPWV, WAVESV);                                                            \
  }
#define FQ_ROUTER_KIND(GO, TPWV, WAVESV)                                                                        \
  if (kind == kE5M2) {                                                                                          \
    if (round_scale) { GO(kE5M2, true, TPWV, WAVESV); } else { GO(kE5M2, false, TPWV, WAVESV); }                \
  } else {                                                                                                      \
    if (round_scale) { GO(kE4M3, true, TPWV, WAVESV); } else { GO(kE4M3, false, TPWV, WAVESV); }                \
  }
  // 8 waves when the column tiles split evenly over them (256, 512 virtual columns), else 4;
  // rows held in registers when there is one chunk, one column tile per wave (128 or 256
  // virtual columns) and K is one of the instantiated widths (1024, 2048); streamed twice
  // otherwise
#define FQ_ROUTER_TILES()                                                   \
  switch (vtiles) {                                                         \
    case 4: FQ_ROUTER_KIND(FQ_ROUTER_RESIDENT, 1, 4) break;                 \
    case 8: FQ_ROUTER_KIND(FQ_ROUTER_RESIDENT, 1, 8) break;                 \
    case 12: FQ_ROUTER_KIND(FQ_ROUTER_STREAMED, 3, 4) break;                \
    case 16: FQ_ROUTER_KIND(FQ_ROUTER_STREAMED, 2, 8) break;                \
    default: return hipErrorInvalidValue;                                   \
  }
  const bool single = vcols <= 512;
  for (int v0 = 0; v0 < vcols; v0 += 512) {
    const int vtiles = (vcols - v0 < 512 ? vcols - v0 : 512) / 32;
    const bool first = v0 == 0;
    const uint4* chunk_w = (const uint4*)wpacked + (int64_t)v0 * K / 8;
    const LogitsOut lout{logits, N, weight_fp32 ? v0 / 2 : v0};
    if (weight_fp32) {
      constexpr bool PAIRV = true;
      FQ_ROUTER_TILES()
    } else {
      constexpr bool PAIRV = false;
      FQ_ROUTER_TILES()
    }
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
  }
#undef FQ_ROUTER_TILES
#undef FQ_ROUTER_KIND
#undef FQ_ROUTER_RESIDENT
#undef FQ_ROUTER_STREAMED
#undef FQ_ROUTER_ARGS
  return hipSuccess;
}

hipError_t launch_rmsnorm_router_quant(const void* x, const void* gamma, const void* wr, int weight_fp32,
                                       void* wpacked, void* y, float* rstd, float* logits, void* q, float* s,
                                       int64_t M, int K, int N, float eps, int round_scale, int kind,
                                       hipStream_t stream) {
  if (M == 0) return hipSuccess;
  const hipError_t e = launch_pack_router_weight(wr, weight_fp32, wpacked, K, N, stream);
  if (e != hipSuccess) return e;
  return launch_rmsnorm_router_quant_packed(x, gamma, wpacked, weight_fp32, y, rstd, logits, q, s, M, K, N, eps,
                                            round_scale, kind, stream);
}

}  // namespace fq
