// Tile kernels: one workgroup per 128x128 output tile, a single pass over HBM.
//   blockwise_quant      plain / per-expert          (linghe/quant/block.py:65-297)
//   silu_quant_fwd       SwiGLU (+row weight) + quant (linghe/utils/silu.py:213-335, 467-950)
//   silu_quant_bwd       SwiGLU backward + quant      (linghe/utils/silu.py:338-464, 1097-1393)
//   rmsnorm_quant_tile   (x*rstd)*gamma + quant with a given rstd
//                                                    (linghe/utils/norm.py:301-340)
#include "fq_tile_geom.hpp"
#include "fq_launch.h"

// Cache policy per kernel, chosen by measurement (cold inputs, MI355X).
//   FQ_NT_<kernel>: which code stores carry the non-temporal hint (bit 0: transposed
//   codes, bit 1: row-wise codes).  With it the outputs do not displace inputs from L2
//   and the memory-side cache: gather+pad+quant 75 -> 55 us, RMSNorm+quant after the
//   statistic pass 25 -> 21 us (8192 x 2048) and 146 -> 122 us (16384 x 7168).  The
//   SwiGLU backward is 3-7 % slower when its transposed stores carry it; the plain
//   blockwise quantiser takes none (13.2 us at 8192 x 2048 against 14.2-16.1 with any), its
//   per-expert form (suffix _B) the transposed stores only (31.5 us against 39.2 without, 32.7
//   with the row-wise codes only and 36.3 with both); the RMSNorm tile kernel with the
//   statistic given (transposed output only, x read once: nothing to protect) none
//   (16384 x 7168: 66.6 -> 59.5 us).  Transposed rows that do not start
//   on 16-byte boundaries (M or a per-expert count that is not a multiple of 16) are where
//   the hint on the transposed stores costs most: the SwiGLU forward takes 100 instead of
//   70 us at 16300 x 3584 with it (and gains 3 % at 8192 x 2048), so it keeps the hint on
//   the row-wise codes only; the RMSNorm tile kernel gains 18 % from it on aligned rows
//   and loses 8 % on unaligned ones.
//   FQ_LDNT_<kernel>: the bulk loads carry it (3-5 % on the SwiGLU kernels and the
//   RMSNorm tile kernel, 12 % on the plain blockwise quantiser, 6 % on its per-expert form;
//   the gathered rows, which several experts read, are 27 % slower with it).
#ifndef FQ_NT_BLOCKWISE
#define FQ_NT_BLOCKWISE 0
#endif
#ifndef FQ_NT_BLOCKWISE_B
#define FQ_NT_BLOCKWISE_B 1
#endif
#ifndef FQ_NT_PERMUTE
#define FQ_NT_PERMUTE 3
#endif
#ifndef FQ_NT_SILU_FWD
#define FQ_NT_SILU_FWD 2
#endif
#ifndef FQ_NT_SILU_BWD
#define FQ_NT_SILU_BWD 2
#endif
#ifndef FQ_NT_SILU_FWD_M0
#define FQ_NT_SILU_FWD_M0 2
#endif
#ifndef FQ_NT_SILU_FWD_M1
#define FQ_NT_SILU_FWD_M1 1
#endif
#ifndef FQ_NT_SILU_FWD_B
#define FQ_NT_SILU_FWD_B 2
#endif
#ifndef FQ_NT_SILU_BWD_B
#define FQ_NT_SILU_BWD_B 2
#endif
#ifndef FQ_NT_RMSNORM
#define FQ_NT_RMSNORM 3
#endif
// transposed output only (the statistic is given, x is read once: nothing to protect)
#ifndef FQ_NT_RMSNORM_T
#define FQ_NT_RMSNORM_T 0
#endif
//   FQ_LEAN_BLOCKWISE: the lean form of the quantiser and of the tile loads (scalar
//   bases, paired column-maximum reduction; every other tile kernel uses it, -3 to -9 %)
//   in the PLAIN blockwise quantiser, which is 7 % slower with it (48 -> 51 us at
//   65536 x 1024); the per-expert form takes it (zipf counts: 60.6 -> 57.9 us).
#ifndef FQ_LEAN_BLOCKWISE
#define FQ_LEAN_BLOCKWISE 0
#endif
#ifndef FQ_LDNT_BLOCKWISE
#define FQ_LDNT_BLOCKWISE 1
#endif
#ifndef FQ_LDNT_BLOCKWISE_B
#define FQ_LDNT_BLOCKWISE_B 1
#endif
#ifndef FQ_LDNT_PERMUTE
#define FQ_LDNT_PERMUTE 0
#endif
#ifndef FQ_LDNT_SILU_FWD
#define FQ_LDNT_SILU_FWD 1
#endif
#ifndef FQ_LDNT_SILU_BWD
#define FQ_LDNT_SILU_BWD 1
#endif
#ifndef FQ_LDNT_SILU_FWD_B
#define FQ_LDNT_SILU_FWD_B 1
#endif
#ifndef FQ_LDNT_SILU_BWD_B
#define FQ_LDNT_SILU_BWD_B 1
#endif
#ifndef FQ_LDNT_RMSNORM
#define FQ_LDNT_RMSNORM 1
#endif
// Rows per thread (workgroup = 2048 / RPT threads).  8 rows per thread spread the
// per-thread overhead over twice the elements, 4 rows per thread put twice the waves on
// a CU.  The SwiGLU forward needs 135 registers with 8 and loses 5-9 %.  The RMSNorm tile
// kernel measured 3-4 % ahead with 8 (93 registers, five 256-thread workgroups per CU)
// when its division took three operations per element; with the current two it is level
// at 16384 x 7168 (110.5 us either way, 58.9 / 58.5 us with the statistic given) and
// 2 % behind at 8192 x 2048 (18.3 / 18.0 us), so it runs with 4.
#ifndef FQ_BWD_REMAP
#define FQ_BWD_REMAP 0
#endif
#ifndef FQ_FWD_REMAP
#define FQ_FWD_REMAP 0
#endif
#ifndef FQ_BWD_PIN
#define FQ_BWD_PIN 1
#endif
#ifndef FQ_RPT_FWD
#define FQ_RPT_FWD 4
#endif
#ifndef FQ_RPT_RMS
#define FQ_RPT_RMS 4
#endif
namespace fq {

// ---------------------------------------------------------------------------
// plain blockwise quant
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND, int MODE, bool BATCHED>
__global__ __launch_bounds__(256) void blockwise_quant_kernel(const uint16_t* __restrict__ x, OutPtrs out,
                                                              int64_t M, int N, BatchArgs batch) {
  constexpr int RPT = 8;
  __shared__ TileShared<RPT> sh;
  const TileGeom g = resolve_tile<BATCHED>(M, N / kGroup, N, batch);
  if (!g.valid) return;
  uint4 raw[RPT];
  constexpr bool LDNT = (BATCHED ? FQ_LDNT_BLOCKWISE_B : FQ_LDNT_BLOCKWISE) != 0;
  constexpr int NT = BATCHED ? FQ_NT_BLOCKWISE_B : FQ_NT_BLOCKWISE;
  constexpr bool LEAN = BATCHED || FQ_LEAN_BLOCKWISE != 0;
  const TilePart<RPT> tp = tile_part<RPT>(g);
  load_rows<RPT, LDNT, LEAN>(x + g.row0 * N + (int64_t)tp.cb * kGroup, N, tp.rows, raw, tp.sl.rgl);
  float v[RPT][8];
#pragma unroll
  for (int s = 0; s < RPT; ++s) unpack8(raw[s], v[s]);
  quantize_tile<KIND, ROUND, MODE, RPT, NT, LEAN>(v, make_out(out, g, N, g.cb), sh);
}

// ---------------------------------------------------------------------------
// gather + pad + blockwise quant (linghe/utils/gather.py:840-1113): expert e's
// region of the outputs holds count_e gathered rows, x[indices[start_e + i]],
// followed by zero rows up to the next multiple of 16; every per-expert layout
// uses the padded count as its stride.  prob_out[start_e + i] = probs[row, e].
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND>
__global__ __launch_bounds__(256) void pad_permute_quant_kernel(const uint16_t* __restrict__ x,
                                                                const int* __restrict__ indices,
                                                                const void* __restrict__ probs, int probs_bf16,
                                                                void* __restrict__ prob_out, OutPtrs out,
                                                                int64_t src_rows, int64_t M, int N,
                                                                BatchArgs batch) {
  constexpr int RPT = 8;
  __shared__ TileShared<RPT> sh;
  const TileGeom g = resolve_tile<true>(M, N / kGroup, N, batch);
  if (!g.valid) return;
  const int cg = threadIdx.x & 15;
  const TilePart<RPT> tp = tile_part<RPT>(g);
  const int rg = tp.sl.rgl;
  // the 8 source rows of this thread: two 16-byte loads (regions start at multiples of 16 rows)
  int src[RPT];
#pragma unroll
  for (int s = 0; s < RPT; ++s) src[s] = -1;
  if (g.row0 + rg * RPT < M) {  // M is a multiple of 16: the eight entries exist together
    const int4* ip = (const int4*)(indices + g.row0 + rg * RPT);
    const int4 a = ip[0], b = ip[1];
    src[0] = a.x; src[1] = a.y; src[2] = a.z; src[3] = a.w;
    src[4] = b.x; src[5] = b.y; src[6] = b.z; src[7] = b.w;
  }
  uint4 raw[RPT];
  const uint16_t* col = x + (int64_t)tp.cb * kGroup + cg * 8;
#pragma unroll
  for (int s = 0; s < RPT; ++s) {
    raw[s] = make_uint4(0, 0, 0, 0);
    // rows of the padding, and indices that do not name a source row, read as zero
    if (rg * RPT + s < tp.rows && (uint32_t)src[s] < (uint64_t)src_rows)
      raw[s] = load16<FQ_LDNT_PERMUTE != 0>(col + (int64_t)src[s] * N);
  }
  if (probs != nullptr && g.cb == 0 && threadIdx.x < kGroup) {
    const int i = threadIdx.x;
    if (i < g.rows_store) {
      const int e = g.expert;
      float pv = 0.f;
      const int r = indices[g.row0 + i];
      const bool live = i < g.rows_valid && (uint32_t)r < (uint64_t)src_rows;
      const int64_t at = (int64_t)r * batch.n_experts + e;
      if (probs_bf16) {
        uint16_t h = live ? ((const uint16_t*)probs)[at] : (uint16_t)0;
        ((uint16_t*)prob_out)[g.row0 + i] = h;
      } else {
        if (live) pv = ((const float*)probs)[at];
        ((float*)prob_out)[g.row0 + i] = pv;
      }
    }
  }
  float v[RPT][8];
#pragma unroll
  for (int s = 0; s < RPT; ++s) unpack8(raw[s], v[s]);
  quantize_tile<KIND, ROUND, 2, RPT, FQ_NT_PERMUTE>(v, make_out(out, g, N, g.cb), sh);
}

// ---------------------------------------------------------------------------
// SwiGLU forward + quant.  y = (sigmoid(x1)*x1)*x2 [*w_row]   (fp32)
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND, int MODE, bool BATCHED, bool WEIGHTED>
__global__ __launch_bounds__(2048 / FQ_RPT_FWD) void silu_quant_fwd_kernel(const uint16_t* __restrict__ x, RowWeight weight,
                                                             OutPtrs out, int64_t M, int n, BatchArgs batch) {
  constexpr int RPT = FQ_RPT_FWD;
  __shared__ TileShared<RPT> sh;
  const TileGeom g = resolve_tile<BATCHED>(M, n / kGroup, n, batch, BATCHED ? FQ_FWD_REMAP : 0);
  if (!g.valid) return;
  const int64_t ld = 2 * (int64_t)n;
  uint4 r1[RPT], r2[RPT];
  const uint16_t* p = x + g.row0 * ld + (int64_t)g.cb * kGroup;
  constexpr bool LDNT = (BATCHED ? FQ_LDNT_SILU_FWD_B : FQ_LDNT_SILU_FWD) != 0;
  constexpr int NT = MODE == 0 ? FQ_NT_SILU_FWD_M0 : MODE == 1 ? FQ_NT_SILU_FWD_M1 : BATCHED ? FQ_NT_SILU_FWD_B : FQ_NT_SILU_FWD;
  const TilePart<RPT> tp = tile_part<RPT>(g);
  load_rows<RPT, LDNT>(p + tp.sl.sub * kGroup, ld, tp.rows, r1, tp.sl.rgl);
  load_rows<RPT, LDNT>(p + n + tp.sl.sub * kGroup, ld, tp.rows, r2, tp.sl.rgl);
  const int rg = tp.sl.rgl;
  float v[RPT][8];
#pragma unroll
  for (int s = 0; s < RPT; ++s)
#pragma unroll
    for (int j = 0; j < 8; ++j) v[s][j] = 0.f;
  if (tp.sl.ws * (4 * RPT) < tp.rows) {  // waves beyond the last row of a partial tile keep zeros
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
      float a[8], b[8];
      unpack8(r1[s], a);
      unpack8(r2[s], b);
      float w = 1.0f;
      if constexpr (WEIGHTED) {
        const int i = rg * RPT + s;
        w = (i < tp.rows) ? load_weight(weight, g.row0 + i) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float y = (sigmoid_f32(a[j]) * a[j]) * b[j];
        if constexpr (WEIGHTED) y = y * w;
        v[s][j] = y;
      }
    }
  }
  quantize_tile<KIND, ROUND, MODE, RPT, NT>(v, make_out(out, g, n, g.cb), sh);
}

// ---------------------------------------------------------------------------
// SwiGLU backward + quant.  With h = g[*w]*x2 and sg = sigmoid(x1):
//   dx1 = h*sg + ((h*x1)*(1-sg))*sg        dx2 = g[*w]*(sg*x1)
//   dw_row = sum_c g*((sg*x1)*x2)          (batched form only)
// evaluated in the order fp32 autograd evaluates them.
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND, bool BATCHED>
__global__ __launch_bounds__(512, 4) void silu_quant_bwd_kernel(const uint16_t* __restrict__ gr,
                                                             const uint16_t* __restrict__ x, RowWeight weight,
                                                             OutPtrs out, float* __restrict__ dw_part, int64_t M,
                                                             int n, BatchArgs batch) {
  constexpr int RPT = 4;
  const int nb = n / kGroup;
  const int64_t N = 2 * (int64_t)n;
  const TileGeom g = resolve_tile<BATCHED>(M, nb, N, batch, BATCHED ? FQ_BWD_REMAP : 0);  // the per-expert form takes an XCD remap
  if (!g.valid) return;
  uint4 r1[RPT], r2[RPT], rgd[RPT];
  const uint16_t* p = x + g.row0 * N + (int64_t)g.cb * kGroup;
  constexpr bool LDNT = (BATCHED ? FQ_LDNT_SILU_BWD_B : FQ_LDNT_SILU_BWD) != 0;
  constexpr int NT = BATCHED ? FQ_NT_SILU_BWD_B : FQ_NT_SILU_BWD;
  const TilePart<RPT> tp = tile_part<RPT>(g);
  load_rows<RPT, LDNT>(p + tp.sl.sub * kGroup, N, tp.rows, r1, tp.sl.rgl);
  load_rows<RPT, LDNT>(p + n + tp.sl.sub * kGroup, N, tp.rows, r2, tp.sl.rgl);
  load_rows<RPT, LDNT>(gr + g.row0 * n + (int64_t)tp.cb * kGroup, n, tp.rows, rgd, tp.sl.rgl);
  const int cg = threadIdx.x & 15;
  const int rg = tp.sl.rgl;
  float d[2][RPT][8];  // dx1, dx2
  float my_dw = 0.f;
#pragma unroll
  for (int s = 0; s < RPT; ++s)
#pragma unroll
    for (int j = 0; j < 8; ++j) d[0][s][j] = d[1][s][j] = 0.f;
  if (tp.sl.ws * (4 * RPT) < tp.rows) {  // waves beyond the last row of a partial tile keep zeros
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
#if FQ_BWD_PIN
      if constexpr (BATCHED || FQ_BWD_PIN > 1) {
        // row s is widened after row s-1 is done (see fence_values): 136 -> 122 registers in the
        // per-expert form, which was capped at 128 and spilled 8 (16 KB of scratch traffic per tile,
        // a quarter of the output again in HBM writes: 97.1 -> 89.1 us at 65536 x 1024, 256 experts)
        if (s > 0) {
          fence_values(d[0][s - 1]);
          fence_values(d[1][s - 1]);
          fence_packed(r1[s]);
          fence_packed(r2[s]);
          fence_packed(rgd[s]);
        }
      }
#endif
      float a[8], b[8], go[8];
      unpack8(r1[s], a);
      unpack8(r2[s], b);
      unpack8(rgd[s], go);
      float w = 1.0f;
      const int i = rg * RPT + s;
      if constexpr (BATCHED) w = (i < tp.rows) ? load_weight(weight, g.row0 + i) : 0.f;
      float dw = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sg = sigmoid_f32(a[j]);
        const float sx = sg * a[j];
        float gw = go[j];
        if constexpr (BATCHED) {
          dw += go[j] * (sx * b[j]);
          gw = go[j] * w;
        }
        const float h = gw * b[j];
        d[1][s][j] = gw * sx;
        d[0][s][j] = h * sg + ((h * a[j]) * (1.0f - sg)) * sg;
      }
      if constexpr (BATCHED) {
        dw = row16_sum(dw);
        if (cg == s) my_dw = dw;
      }
    }
  }
  if constexpr (BATCHED) {
    if (cg < RPT) {
      const int i = rg * RPT + cg;
      if (i < tp.rows) dw_part[(g.row0 + i) * nb + tp.cb] = my_dw;
    }
  }
  if constexpr (!BATCHED) {
    // dx1 and dx2 go through the quantiser together: one set of barriers, 256 column scales
    // at once (38.5 -> 35.7 us at 8192 x 2048).  The per-expert form, which also carries the
    // tile lookup and the row weights, spills registers in that shape and is 1 % slower
    // with it, so it quantises one tile after the other.
    __shared__ TileShared<RPT, 2> sh;
    const TileOut outs[2] = {make_out(out, g, N, g.cb), make_out(out, g, N, nb + g.cb)};
    quantize_tiles<KIND, ROUND, 2, RPT, NT, true, 2>(d, outs, sh);
  } else {
    __shared__ TileShared<RPT> sh;
    const TileOut o1[1] = {make_out(out, g, N, g.cb)};
    const TileOut o2[1] = {make_out(out, g, N, nb + g.cb)};
    const float (&dx1)[1][RPT][8] = reinterpret_cast<const float (&)[1][RPT][8]>(d[0]);
    const float (&dx2)[1][RPT][8] = reinterpret_cast<const float (&)[1][RPT][8]>(d[1]);
    quantize_tiles<KIND, ROUND, 2, RPT, NT, true, 1, true>(dx1, o1, sh);
    quantize_tiles<KIND, ROUND, 2, RPT, NT, true, 1, false>(dx2, o2, sh);
  }
}

// dw[r] = sum_b part[r, b]  (fixed order), stored as fp32 or bf16
__global__ __launch_bounds__(256) void rowsum_kernel(const float* __restrict__ part, void* __restrict__ dw,
                                                     int64_t M, int nb, int out_bf16) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= M) return;
  float acc = 0.f;
  for (int b = 0; b < nb; ++b) acc += part[r * nb + b];
  if (out_bf16) ((uint16_t*)dw)[r] = (uint16_t)(pack_bf16x2(acc, 0.f) & 0xffffu);
  else ((float*)dw)[r] = acc;
}

// ---------------------------------------------------------------------------
// RMSNorm + quant on a tile with the row statistic given:
//   y = (x * rstd[row]) * gamma[col]
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND, int MODE, int NT>
__global__ __launch_bounds__(2048 / FQ_RPT_RMS) void rmsnorm_quant_tile_kernel(const uint16_t* __restrict__ x,
                                                                 const uint16_t* __restrict__ gamma,
                                                                 const float* __restrict__ rstd, OutPtrs out,
                                                                 int64_t M, int n, int remap) {
  constexpr int RPT = FQ_RPT_RMS;
  __shared__ TileShared<RPT> sh;
  BatchArgs none{nullptr, 0, 0};
  const TileGeom g = resolve_tile<false>(M, n / kGroup, n, none, remap);
  if (!g.valid) return;
  uint4 raw[RPT];
  load_rows<RPT, FQ_LDNT_RMSNORM != 0>(x + g.row0 * n + (int64_t)g.cb * kGroup, n, g.rows_valid, raw);
  const int cg = threadIdx.x & 15;
  const int rg = threadIdx.x >> 4;
  float gm[8];
  unpack8(*(const uint4*)(gamma + (int64_t)g.cb * kGroup + cg * 8), gm);
  float v[RPT][8];
#pragma unroll
  for (int s = 0; s < RPT; ++s) {
    const int i = rg * RPT + s;
    const float r = (i < g.rows_valid) ? rstd[g.row0 + i] : 0.f;
    float a[8];
    unpack8(raw[s], a);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[s][j] = (a[j] * r) * gm[j];
  }
  quantize_tile<KIND, ROUND, MODE, RPT, NT>(v, make_out(out, g, n, g.cb), sh);
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
hipError_t launch_blockwise_quant(const void* x, void* q, float* s, void* qt, float* st, int64_t M, int N,
                                  int round_scale, int mode, int kind, const void* counts, int counts_i64,
                                  int n_experts, int64_t row_blocks, hipStream_t stream) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  BatchArgs b{counts, counts_i64, n_experts};
  const int64_t tiles = row_blocks * (N / kGroup);
  if (tiles == 0) return hipSuccess;
  const dim3 grid((unsigned)tiles), block(256);
  const bool batched = counts != nullptr;
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      FQ_DISPATCH_MODE(mode, MD,
        FQ_DISPATCH_BOOL(batched, B,
          hipLaunchKernelGGL((blockwise_quant_kernel<K, R, MD, B>), grid, block, 0, stream,
                             (const uint16_t*)x, out, M, N, b);))))
  return hipGetLastError();
}

hipError_t launch_pad_permute_quant(const void* x, const void* indices, const void* probs, int probs_bf16,
                                    void* prob_out, void* q, float* s, void* qt, float* st, int64_t src_rows,
                                    int64_t M, int N, int round_scale, int kind, const void* counts, int counts_i64,
                                    int n_experts, int64_t row_blocks, hipStream_t stream) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  BatchArgs b{counts, counts_i64, n_experts, 16};
  const int64_t tiles = row_blocks * (N / kGroup);
  if (tiles == 0) return hipSuccess;
  const dim3 grid((unsigned)tiles), block(256);
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      hipLaunchKernelGGL((pad_permute_quant_kernel<K, R>), grid, block, 0, stream, (const uint16_t*)x,
                         (const int*)indices, probs, probs_bf16, prob_out, out, src_rows, M, N, b);))
  return hipGetLastError();
}

hipError_t launch_silu_quant_fwd(const void* x, const void* weight, int weight_bf16, void* q, float* s, void* qt,
                                 float* st, int64_t M, int n, int round_scale, int mode, int kind,
                                 const void* counts, int counts_i64, int n_experts, int64_t row_blocks,
                                 hipStream_t stream) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  BatchArgs b{counts, counts_i64, n_experts};
  RowWeight w{weight, weight_bf16};
  const int64_t tiles = row_blocks * (n / kGroup);
  if (tiles == 0) return hipSuccess;
  const dim3 grid((unsigned)tiles), block(2048 / FQ_RPT_FWD);
  const bool batched = counts != nullptr;
  const bool weighted = weight != nullptr;
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      FQ_DISPATCH_MODE(mode, MD,
        FQ_DISPATCH_BOOL(batched, B,
          FQ_DISPATCH_BOOL(weighted, W,
            hipLaunchKernelGGL((silu_quant_fwd_kernel<K, R, MD, B, W>), grid, block, 0, stream,
                               (const uint16_t*)x, w, out, M, n, b);)))))
  return hipGetLastError();
}

hipError_t launch_silu_quant_bwd(const void* g, const void* x, const void* weight, int weight_bf16, void* q,
                                 float* s, void* qt, float* st, float* dw_part, void* dw, int64_t M, int n,
                                 int round_scale, int kind, const void* counts, int counts_i64, int n_experts,
                                 int64_t row_blocks, hipStream_t stream) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  BatchArgs b{counts, counts_i64, n_experts};
  RowWeight w{weight, weight_bf16};
  const int nb = n / kGroup;
  const int64_t tiles = row_blocks * nb;
  if (tiles == 0) return hipSuccess;
  const dim3 grid((unsigned)tiles), block(512);
  const bool batched = counts != nullptr;
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      FQ_DISPATCH_BOOL(batched, B,
        hipLaunchKernelGGL((silu_quant_bwd_kernel<K, R, B>), grid, block, 0, stream, (const uint16_t*)g,
                           (const uint16_t*)x, w, out, dw_part, M, n, b);)))
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  if (batched && M > 0) {
    hipLaunchKernelGGL(rowsum_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, stream, dw_part, dw, M, nb,
                       weight_bf16);
    err = hipGetLastError();
  }
  return err;
}

hipError_t launch_rmsnorm_quant_tile(const void* x, const void* gamma, const float* rstd, void* q, float* s,
                                     void* qt, float* st, int64_t M, int n, int round_scale, int mode, int kind,
                                     hipStream_t stream) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  const int64_t tiles = ((M + kGroup - 1) / kGroup) * (n / kGroup);
  if (tiles == 0) return hipSuccess;
  const dim3 grid((unsigned)tiles), block(2048 / FQ_RPT_RMS);
  // transposed rows start every M bytes: off 16-byte boundaries their stores go out plain
  const bool aligned_rows = M % 16 == 0;
  // XCD remap (see resolve_tile): wide rows and several waves of workgroups
  const int remap = aligned_rows && n >= 4096 && tiles >= 3072;
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      FQ_DISPATCH_MODE(mode, MD,
        FQ_DISPATCH_BOOL(aligned_rows, A,
          hipLaunchKernelGGL((rmsnorm_quant_tile_kernel<K, R, MD, MD == 1 ? FQ_NT_RMSNORM_T : A ? FQ_NT_RMSNORM : (FQ_NT_RMSNORM & 2)>), grid,
                             block, 0, stream, (const uint16_t*)x, (const uint16_t*)gamma, rstd, out, M, n,
                             remap);))))
  return hipGetLastError();
}

}  // namespace fq
