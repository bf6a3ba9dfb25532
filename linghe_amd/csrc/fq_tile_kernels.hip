// Tile kernels: one workgroup per 128x128 output tile, a single pass over HBM.
//   blockwise_quant      plain / per-expert          (linghe/quant/block.py:65-297)
//   silu_quant_fwd       SwiGLU (+row weight) + quant (linghe/utils/silu.py:213-335, 467-950)
//   silu_quant_bwd       SwiGLU backward + quant      (linghe/utils/silu.py:338-464, 1097-1393)
//   rmsnorm_quant_tile   (x*rstd)*gamma + quant with a given rstd
//                                                    (linghe/utils/norm.py:301-340)
#include "fq_tile_geom.hpp"
#include "fq_launch.h"

#include "fq_policy.hpp"

namespace fq {

// ---------------------------------------------------------------------------
// plain blockwise quant
// ---------------------------------------------------------------------------
// PLANNED: the per-expert form with its tiles read from a plan (same code; another cache policy,
// because its tile numbering lets an XCD's L2 merge the partial lines of the transposed codes)
template <int KIND, bool ROUND, int MODE, bool BATCHED, bool PLANNED = false>
__global__ __launch_bounds__(2048 / (BATCHED ? Policy::kRowsPerThreadBlockwiseBatched : Policy::kRowsPerThreadBlockwise))
void blockwise_quant_kernel(const uint16_t* __restrict__ x, OutPtrs out, int64_t M, int N, BatchArgs batch) {
  constexpr int RPT = BATCHED ? Policy::kRowsPerThreadBlockwiseBatched : Policy::kRowsPerThreadBlockwise;
  __shared__ TileShared<RPT> sh;
  const TileGeom g = resolve_tile<BATCHED>(M, N / kGroup, N, batch);
  if (!g.valid) return;
  uint4 raw[RPT];
  constexpr bool LDNT = BATCHED ? Policy::kLoadHintBlockwiseBatched : Policy::kLoadHintBlockwise;
  constexpr int NT = PLANNED ? Policy::kStoreHintBlockwisePlanned
                     : BATCHED ? Policy::kStoreHintBlockwiseBatched : Policy::kStoreHintBlockwise;
  constexpr bool LEAN = BATCHED || Policy::kLeanBlockwise;
  const TilePart<RPT> tp = tile_part<RPT>(g);
  load_rows<RPT, LDNT, LEAN>(x + g.row0 * N + (int64_t)(g.cb + tp.asub) * kGroup, N, tp.rows, raw, tp.sl.rgl);
  mask_rows<RPT>(tp.rows, raw, tp.sl.rgl);
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
  const int cg = tile_tid() & 15;
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
  // Rows of the padding, and indices that do not name a source row, read as zero.  The eight loads
  // carry no condition (such a row fetches source row 0, which exists, and is zeroed afterwards):
  // behind a per-row branch the compiler waited for each gathered row before it asked for the
  // next one, eight memory round trips in a row at the start of every tile.
  bool live[RPT];
#pragma unroll
  for (int s = 0; s < RPT; ++s) {
    live[s] = rg * RPT + s < tp.rows && (uint32_t)src[s] < (uint64_t)src_rows;
    raw[s] = load16<Policy::kLoadHintPermute>(col + (int64_t)(live[s] ? src[s] : 0) * N);
  }
#pragma unroll
  for (int s = 0; s < RPT; ++s)
    if (!live[s]) raw[s] = make_uint4(0, 0, 0, 0);
  if (probs != nullptr && g.cb == 0 && tile_tid() < kGroup) {
    const int i = tile_tid();
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
  quantize_tile<KIND, ROUND, 2, RPT, Policy::kStoreHintPermute>(v, make_out(out, g, N, g.cb), sh);
}

// ---------------------------------------------------------------------------
// SwiGLU forward + quant.  y = (sigmoid(x1)*x1)*x2 [*w_row]   (fp32)
// ---------------------------------------------------------------------------
// ALL_FULL: single matrix with M a multiple of 128 (see quantize_tiles)
template <int KIND, bool ROUND, int MODE, bool BATCHED, bool WEIGHTED, bool ALL_FULL>
__global__ __launch_bounds__(2048 / Policy::kRowsPerThreadSiluFwd) void silu_quant_fwd_kernel(const uint16_t* __restrict__ x, RowWeight weight,
                                                             OutPtrs out, int64_t M, int n, BatchArgs batch) {
  constexpr int RPT = Policy::kRowsPerThreadSiluFwd;
  __shared__ TileShared<RPT> sh;
  const TileGeom g = resolve_tile<BATCHED>(M, n / kGroup, n, batch);
  if (!g.valid) return;
  const int64_t ld = 2 * (int64_t)n;
  uint4 r1[RPT], r2[RPT];
  const uint16_t* p = x + g.row0 * ld + (int64_t)g.cb * kGroup;
  constexpr bool LDNT = BATCHED ? Policy::kLoadHintSiluFwdBatched : Policy::kLoadHintSiluFwd;
  constexpr int NT = MODE == 0 ? Policy::kStoreHintSiluFwdRows : MODE == 1 ? Policy::kStoreHintSiluFwdCols : BATCHED ? Policy::kStoreHintSiluFwdBatched : Policy::kStoreHintSiluFwd;
  TilePart<RPT> tp = tile_part<RPT>(g);
  if constexpr (ALL_FULL) tp.rows = kGroup;  // a constant: the masked loads and the zero fill fold away
  const int rg = tp.sl.rgl;
  // The row weights are fetched first, ahead of the tile: loads return in the order they were issued,
  // and a weight fetched where it is used (inside a row's arithmetic) is a memory round trip in the
  // middle of the tile's critical path (four of them in the backward kernel, whose rows are fenced
  // apart: 85.2 -> 77.5 us without the weights at 65536 x 1024, 256 experts).
  uint32_t wbits[RPT];
  if constexpr (WEIGHTED) {
    // no per-row condition on the loads: a row beyond the end of the tile fetches the tile's first
    // row's weight (a valid address) and counts as zero where it is used
    int64_t wr[RPT];
#pragma unroll
    for (int s = 0; s < RPT; ++s) wr[s] = g.row0 + (rg * RPT + s < tp.rows ? rg * RPT + s : 0);
    load_weight_bits<RPT>(weight, wr, wbits);
  }
  load_rows<RPT, LDNT>(p + tp.asub * kGroup, ld, tp.rows, r1, tp.sl.rgl);
  load_rows<RPT, LDNT>(p + n + tp.asub * kGroup, ld, tp.rows, r2, tp.sl.rgl);
  if constexpr (!ALL_FULL) {
    mask_rows<RPT>(tp.rows, r1, tp.sl.rgl);
    mask_rows<RPT>(tp.rows, r2, tp.sl.rgl);
  }
  // Every wave does the arithmetic, also one whose rows all lie beyond the last row of a partial tile
  // (its inputs read as zeros and give zeros): a branch around the arithmetic keeps the zero-filled results
  // and the packed inputs alive side by side and costs 13-20 registers (73 -> 60 in the per-expert form:
  // three -> four workgroups per CU), while skipping the arithmetic gained nothing measurable.
  float v[RPT][8];
  {
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
      float a[8], b[8];
      unpack8(r1[s], a);
      unpack8(r2[s], b);
      const float w = !WEIGHTED ? 1.0f : rg * RPT + s < tp.rows ? weight_from_bits(weight, wbits[s]) : 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float y = (sigmoid_f32(a[j]) * a[j]) * b[j];
        if constexpr (WEIGHTED) y = y * w;
        v[s][j] = y;
      }
    }
  }
  quantize_tile<KIND, ROUND, MODE, RPT, NT, true, ALL_FULL>(v, make_out(out, g, n, g.cb), sh);
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
  const TileGeom g = resolve_tile<BATCHED>(M, nb, N, batch);
  if (!g.valid) return;
  uint4 r1[RPT], r2[RPT], rgd[RPT];
  const uint16_t* p = x + g.row0 * N + (int64_t)g.cb * kGroup;
  constexpr bool LDNT = BATCHED ? Policy::kLoadHintSiluBwdBatched : Policy::kLoadHintSiluBwd;
  constexpr int NT = BATCHED ? Policy::kStoreHintSiluBwdBatched : Policy::kStoreHintSiluBwd;
  TilePart<RPT> tp = tile_part<RPT>(g);
  if constexpr (!BATCHED) tp.rows = kGroup;  // single matrix: M % 128 == 0
  // row weights first (see the forward kernel)
  uint32_t wbits[RPT];
  if constexpr (BATCHED) {
    int64_t wr[RPT];
#pragma unroll
    for (int s = 0; s < RPT; ++s) wr[s] = g.row0 + (tp.sl.rgl * RPT + s < tp.rows ? tp.sl.rgl * RPT + s : 0);
    load_weight_bits<RPT>(weight, wr, wbits);
  }
  load_rows<RPT, LDNT>(p + tp.asub * kGroup, N, tp.rows, r1, tp.sl.rgl);
  load_rows<RPT, LDNT>(p + n + tp.asub * kGroup, N, tp.rows, r2, tp.sl.rgl);
  load_rows<RPT, LDNT>(gr + g.row0 * n + (int64_t)(g.cb + tp.asub) * kGroup, n, tp.rows, rgd, tp.sl.rgl);
  if constexpr (BATCHED) {
    mask_rows<RPT>(tp.rows, r1, tp.sl.rgl);
    mask_rows<RPT>(tp.rows, r2, tp.sl.rgl);
    mask_rows<RPT>(tp.rows, rgd, tp.sl.rgl);
  }
  const int cg = tile_tid() & 15;
  const int rg = tp.sl.rgl;
  float d[2][RPT][8];  // dx1, dx2
  float my_dw = 0.f;
  {  // every wave does the arithmetic (see the forward kernel): zero inputs give zero results
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
      if constexpr (BATCHED ? Policy::kPinBwdRowsBatched : Policy::kPinBwdRows) {
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
      float a[8], b[8], go[8];
      unpack8(r1[s], a);
      unpack8(r2[s], b);
      unpack8(rgd[s], go);
      const float w = !BATCHED ? 1.0f : rg * RPT + s < tp.rows ? weight_from_bits(weight, wbits[s]) : 0.f;
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
      if (i < tp.rows) dw_part[(int64_t)tp.cb * M + (g.row0 + i)] = my_dw;  // [nb, M]: a wave writes consecutive floats
    }
  }
  if constexpr (!BATCHED) {
    // dx1 and dx2 go through the quantiser together: one set of barriers, 256 column scales
    // at once (38.5 -> 35.7 us at 8192 x 2048).  The per-expert form, which also carries the
    // tile lookup and the row weights, spills registers in that shape and is 1 % slower
    // with it, so it quantises one tile after the other.
    __shared__ TileShared<RPT, 2> sh;
    const TileOut outs[2] = {make_out(out, g, N, g.cb), make_out(out, g, N, nb + g.cb)};
    // the single-matrix form takes M % 128 == 0 only (as the reference): no partial tile
    quantize_tiles<KIND, ROUND, 2, RPT, NT, true, 2, false, true>(d, outs, sh);
  } else {
    // a full tile (most of them) goes the same way; a partial one, which may be packed, one tile after the other
    __shared__ union { TileShared<RPT, 2> both; TileShared<RPT> one; } sh;
    if (g.rows_store == kGroup) {
      const TileOut outs[2] = {make_out(out, g, N, g.cb), make_out(out, g, N, nb + g.cb)};
      quantize_tiles<KIND, ROUND, 2, RPT, NT, true, 2, false, true>(d, outs, sh.both);
    } else {
      const TileOut o1[1] = {make_out(out, g, N, g.cb)};
      const TileOut o2[1] = {make_out(out, g, N, nb + g.cb)};
      const float (&dx1)[1][RPT][8] = reinterpret_cast<const float (&)[1][RPT][8]>(d[0]);
      const float (&dx2)[1][RPT][8] = reinterpret_cast<const float (&)[1][RPT][8]>(d[1]);
      quantize_tiles_impl<KIND, ROUND, 2, RPT, false, NT, true, 1, true>(dx1, o1, sh.one);
      quantize_tiles_impl<KIND, ROUND, 2, RPT, false, NT, true, 1, false>(dx2, o2, sh.one);
    }
  }
}

// dw[r] = sum_b part[b, r]  (fixed order), stored as fp32 or bf16
__global__ __launch_bounds__(256) void rowsum_kernel(const float* __restrict__ part, void* __restrict__ dw,
                                                     int64_t M, int nb, int out_bf16) {
  const int64_t r = (int64_t)wg_x() * 256 + tile_tid();
  if (r >= M) return;
  float acc = 0.f;
  for (int b = 0; b < nb; ++b) acc += part[(int64_t)b * M + r];
  if (out_bf16) ((uint16_t*)dw)[r] = (uint16_t)(pack_bf16x2(acc, 0.f) & 0xffffu);
  else ((float*)dw)[r] = acc;
}

// ---------------------------------------------------------------------------
// RMSNorm + quant on a tile with the row statistic given:
//   y = (x * rstd[row]) * gamma[col]
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND, int MODE, int NT>
__global__ __launch_bounds__(2048 / Policy::kRowsPerThreadRmsnorm) void rmsnorm_quant_tile_kernel(const uint16_t* __restrict__ x,
                                                                 const uint16_t* __restrict__ gamma,
                                                                 const float* __restrict__ rstd, OutPtrs out,
                                                                 int64_t M, int n, int remap, int first) {
  constexpr int RPT = Policy::kRowsPerThreadRmsnorm;
  // A launch that the chip holds all at once (every workgroup starts together and there is no second
  // generation): waves run at raised priority until their loads are out, so that every wave of a CU has
  // asked for its rows before the first of them goes on to anything else (17.7 against 18.3 us for
  // RMSNorm + quant at 8192 x 2048).  With workgroups arriving one after the other the same priority
  // lets the newcomers push aside the stores of the ones at work: 4 % slower at 16384 x 7168.
  if (first) __builtin_amdgcn_s_setprio(3);
  __shared__ TileShared<RPT> sh;
  BatchArgs none{nullptr, 0, 0, 0, nullptr, 0, 0, 0, 0, 0};
  const TileGeom g = resolve_tile<false>(M, n / kGroup, n, none, remap);
  if (!g.valid) return;
  uint4 raw[RPT];
  load_rows<RPT, Policy::kLoadHintRmsnorm>(x + g.row0 * n + (int64_t)g.cb * kGroup, n, g.rows_valid, raw);
  const int cg = tile_tid() & 15;
  const int rg = tile_tid() >> 4;
  // every load of the tile is issued before the first of them is waited for: the statistic of a
  // row beyond the end is fetched from the tile's first row (a valid address) and not used
  const uint4 gmraw = *(const uint4*)(gamma + (int64_t)g.cb * kGroup + cg * 8);
  float rs[RPT];
#pragma unroll
  for (int s = 0; s < RPT; ++s) rs[s] = rstd[g.row0 + (rg * RPT + s < g.rows_valid ? rg * RPT + s : 0)];
  if (first) __builtin_amdgcn_s_setprio(0);
  mask_rows<RPT>(g.rows_valid, raw, rg);
  float gm[8];
  unpack8(gmraw, gm);
  float v[RPT][8];
#pragma unroll
  for (int s = 0; s < RPT; ++s) {
    const int i = rg * RPT + s;
    const float r = (i < g.rows_valid) ? rs[s] : 0.f;
    float a[8];
    unpack8(raw[s], a);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[s][j] = (a[j] * r) * gm[j];
  }
  quantize_tile<KIND, ROUND, MODE, RPT, NT>(v, make_out(out, g, n, g.cb), sh);
}

// ---------------------------------------------------------------------------
// The per-row-block table of a set of counts (PlanEntry): one workgroup of 1024 threads, one
// expert per thread and pass.  Every pass scans its experts' row blocks, rows and the members of
// the table's three sections over the workgroup, leaves the exclusive sums in shared memory and
// writes the pass's records, one per thread and step, each finding its expert by bisection over
// the exclusive block sums.  The sizes of the sections are the host's; where the device-side
// counts give a section fewer members the rest of it is marked empty, where they give it more the
// surplus is dropped (the launches then leave those row blocks out: the counts disagree).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(1024) void expert_plan_kernel(const void* __restrict__ counts, int counts_i64,
                                                           int n_experts, int pad, int b0, int b1, int b2,
                                                           PlanEntry* __restrict__ plan) {
  int* __restrict__ expert_of = (int*)(plan + ((int64_t)b0 + b1 + b2));
  constexpr int T = 1024, W = T / 64;
  __shared__ int eb[T + 1];  // exclusive sums of the pass: row blocks,
  __shared__ int ez[T];      // unpacked row blocks,
  __shared__ int ep[T];      // packed last blocks (two-fold in the low half, four-fold in the high half),
  __shared__ int64_t er[T];  // rows
  __shared__ int ec[T];      // the counts themselves
  __shared__ int wb[W], wz[W], wp[W];
  __shared__ int64_t wr[W];
  __shared__ int pass_z, pass_p;
  const int t = (int)tid_x(), lane = t & 63, wave = t >> 6;
  int64_t run_rows = 0;
  int run_blocks = 0, run_z = 0, run_p1 = 0, run_p2 = 0;
  for (int base = 0; base < n_experts; base += T) {
    const int e = base + t;
    const int cr = e < n_experts ? load_count(counts, counts_i64, e) : 0;
    const int c = cr > 0 ? cr : 0;
    const int pc = (c + pad - 1) & -pad;  // rows of the expert's region in the outputs (pad: 1 or 16)
    const int nb = (c + kGroup - 1) / kGroup;
    const int sh = nb > 0 ? pack_shift(pc - (nb - 1) * kGroup) : 0;
    const int p = (sh == 1) + ((sh == 2) << 16);
    const int z = nb - (sh > 0);
    const int ib = wave_inclusive_scan(nb);
    const int iz = wave_inclusive_scan(z);
    const int ip = wave_inclusive_scan(p);
    // the rows of 64 experts fit 32 bits for every matrix the entry points accept; the sums over
    // waves and passes are 64-bit
    const int ir = wave_inclusive_scan(pc);
    if (lane == 63) { wb[wave] = ib; wz[wave] = iz; wp[wave] = ip; wr[wave] = ir; }
    __syncthreads();
    int ob = 0, oz = 0, op = 0;
    int64_t orow = 0;
    for (int w = 0; w < wave; ++w) { ob += wb[w]; oz += wz[w]; op += wp[w]; orow += wr[w]; }
    eb[t] = ob + ib - nb;
    ez[t] = oz + iz - z;
    ep[t] = op + ip - p;
    er[t] = orow + ir - pc;
    ec[t] = c;
    if (t == T - 1) {
      eb[T] = ob + ib;
      pass_z = oz + iz;
      pass_p = op + ip;
    }
    __syncthreads();
    const int pass_blocks = eb[T];
    for (int j = t; j < pass_blocks; j += T) {
      int lo = 0, hi = T - 1;  // the last expert of the pass whose exclusive sum is <= j
      while (lo < hi) {
        const int mid = (lo + hi + 1) >> 1;
        if (eb[mid] <= j) lo = mid; else hi = mid - 1;
      }
      const int cl = ec[lo], rb = j - eb[lo];
      const int nbl = (cl + kGroup - 1) / kGroup;
      const int shift = rb == nbl - 1 ? pack_shift(((cl + pad - 1) & -pad) - rb * kGroup) : 0;
      // place inside the record's section, the section's start and size
      const int64_t in = shift == 0 ? (int64_t)run_z + ez[lo] + rb
                         : shift == 1 ? (int64_t)run_p1 + (ep[lo] & 0xffff) : (int64_t)run_p2 + (ep[lo] >> 16);
      const int64_t first = shift == 0 ? 0 : shift == 1 ? (int64_t)b0 : (int64_t)b0 + b1;
      const int size = shift == 0 ? b0 : shift == 1 ? b1 : b2;
      if (in < size) {
        PlanEntry pe;
        pe.row0 = (uint32_t)(run_rows + er[lo] + (int64_t)rb * kGroup);
        pe.rb = rb;
        pe.count = cl;
        pe.where = (shift == 0 ? kPlanUnpacked : shift == 1 ? kPlanPacked2 : kPlanPacked4) << 30 |
                   (uint32_t)(run_blocks + j);
        plan[first + in] = pe;
        expert_of[first + in] = base + lo;
      }
    }
    run_blocks += pass_blocks;
    run_rows += er[T - 1] + ((ec[T - 1] + pad - 1) & -pad);
    run_z += pass_z;
    run_p1 += pass_p & 0xffff;
    run_p2 += pass_p >> 16;
    __syncthreads();
  }
  PlanEntry none;
  none.row0 = 0;
  none.rb = 0;
  none.count = 0;
  none.where = kPlanEmpty << 30;
  for (int64_t at = (int64_t)run_z + t; at < b0; at += T) { plan[at] = none; expert_of[at] = -1; }
  for (int64_t at = (int64_t)b0 + run_p1 + t; at < (int64_t)b0 + b1; at += T) { plan[at] = none; expert_of[at] = -1; }
  for (int64_t at = (int64_t)b0 + b1 + run_p2 + t; at < (int64_t)b0 + b1 + b2; at += T) { plan[at] = none; expert_of[at] = -1; }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
static BatchArgs batch_args(const void* counts, int counts_i64, int n_experts, const void* plan,
                            const PlanShape* ps, bool packed_first, int xcd_rows_scan,
                            int xcd_rows_planned = Policy::kXcdRowsPlanned) {
  if (plan != nullptr)
    return BatchArgs{nullptr, 0, n_experts, ps->pad > 1 ? ps->pad : 0, plan, (int)ps->unpacked, (int)ps->packed2,
                     (int)ps->packed4, xcd_rows_planned, packed_first};
  return BatchArgs{counts, counts_i64, n_experts, 0, nullptr, 0, 0, 0, xcd_rows_scan, 0};
}

int64_t expert_plan_bytes(const PlanShape& ps) { return ps.blocks() * (int64_t)(sizeof(PlanEntry) + sizeof(int)); }

PlanShape expert_plan_shape(const int64_t* host_counts, int n_experts, int pad) {
  PlanShape ps{0, 0, 0, pad};
  for (int e = 0; e < n_experts; ++e) {
    const int64_t c = host_counts[e] > 0 ? host_counts[e] : 0;
    const int64_t nb = (c + kGroup - 1) / kGroup;
    if (nb == 0) continue;
    const int last = (int)(((c + pad - 1) & -(int64_t)pad) - (nb - 1) * kGroup);
    const int shift = last <= 32 ? 2 : last <= 64 ? 1 : 0;  // pack_shift, on the host
    ps.unpacked += nb - (shift > 0);
    ps.packed2 += shift == 1;
    ps.packed4 += shift == 2;
  }
  return ps;
}

hipError_t launch_expert_plan(const void* counts, int counts_i64, int n_experts, const PlanShape& ps, void* plan,
                              hipStream_t stream) {
  if (ps.blocks() == 0) return hipSuccess;
  hipLaunchKernelGGL(expert_plan_kernel, dim3(1), dim3(1024), 0, stream, counts, counts_i64, n_experts, ps.pad,
                     (int)ps.unpacked, (int)ps.packed2, (int)ps.packed4, (PlanEntry*)plan);
  return hipGetLastError();
}

hipError_t launch_blockwise_quant(const void* x, void* q, float* s, void* qt, float* st, int64_t M, int N,
                                  int round_scale, int mode, int kind, const void* counts, int counts_i64,
                                  int n_experts, int64_t row_blocks, hipStream_t stream, const void* plan,
                                  const PlanShape* ps) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  const BatchArgs b = batch_args(counts, counts_i64, n_experts, plan, ps, Policy::kPlanPackedFirstBlockwise, 0);
  const int64_t tiles = plan ? plan_workgroups(ps->unpacked, ps->packed2, ps->packed4, N / kGroup)
                             : row_blocks * (N / kGroup);
  if (tiles == 0) return hipSuccess;
  const bool batched = counts != nullptr || plan != nullptr;
  const dim3 grid((unsigned)tiles),
      block(2048 / (batched ? Policy::kRowsPerThreadBlockwiseBatched : Policy::kRowsPerThreadBlockwise));
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      FQ_DISPATCH_MODE(mode, MD,
        FQ_DISPATCH_BOOL(batched, B,
          FQ_DISPATCH_BOOL(plan != nullptr, P,
            hipLaunchKernelGGL((blockwise_quant_kernel<K, R, MD, B || P, P>), grid, block, 0, stream,
                               (const uint16_t*)x, out, M, N, b);)))))
  return hipGetLastError();
}

hipError_t launch_pad_permute_quant(const void* x, const void* indices, const void* probs, int probs_bf16,
                                    void* prob_out, void* q, float* s, void* qt, float* st, int64_t src_rows,
                                    int64_t M, int N, int round_scale, int kind, const void* counts, int counts_i64,
                                    int n_experts, int64_t row_blocks, hipStream_t stream, const void* plan,
                                    const PlanShape* ps) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  BatchArgs b{counts, counts_i64, n_experts, 16, nullptr, 0, 0, 0, 0, 0};
  if (plan != nullptr)
    b = batch_args(nullptr, 0, n_experts, plan, ps, Policy::kPlanPackedFirstPermute, 0, Policy::kXcdRowsPermutePlanned);
  const int64_t tiles = plan ? plan_workgroups(ps->unpacked, ps->packed2, ps->packed4, N / kGroup)
                             : row_blocks * (N / kGroup);
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
                                 hipStream_t stream, const void* plan, const PlanShape* ps) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  const BatchArgs b = batch_args(counts, counts_i64, n_experts, plan, ps, Policy::kPlanPackedFirstSiluFwd, 0);
  RowWeight w{weight, weight_bf16};
  const int64_t tiles = plan ? plan_workgroups(ps->unpacked, ps->packed2, ps->packed4, n / kGroup)
                             : row_blocks * (n / kGroup);
  if (tiles == 0) return hipSuccess;
  const dim3 grid((unsigned)tiles), block(2048 / Policy::kRowsPerThreadSiluFwd);
  const bool batched = counts != nullptr || plan != nullptr;
  const bool weighted = weight != nullptr;
  const bool all_full = !batched && M % kGroup == 0;
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      FQ_DISPATCH_MODE(mode, MD,
        FQ_DISPATCH_BOOL(batched, B,
          FQ_DISPATCH_BOOL(weighted, W,
            FQ_DISPATCH_BOOL(all_full, AF,
              hipLaunchKernelGGL((silu_quant_fwd_kernel<K, R, MD, B, W, AF && !B>), grid, block, 0, stream,
                                 (const uint16_t*)x, w, out, M, n, b);))))))
  return hipGetLastError();
}

hipError_t launch_silu_quant_bwd(const void* g, const void* x, const void* weight, int weight_bf16, void* q,
                                 float* s, void* qt, float* st, float* dw_part, void* dw, int64_t M, int n,
                                 int round_scale, int kind, const void* counts, int counts_i64, int n_experts,
                                 int64_t row_blocks, hipStream_t stream, const void* plan, const PlanShape* ps) {
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  const BatchArgs b = batch_args(counts, counts_i64, n_experts, plan, ps, Policy::kPlanPackedFirstSiluBwd,
                                   Policy::kXcdRowsSiluBwdCounts);
  RowWeight w{weight, weight_bf16};
  const int nb = n / kGroup;
  const int64_t tiles = plan ? plan_workgroups(ps->unpacked, ps->packed2, ps->packed4, nb) : row_blocks * nb;
  if (tiles == 0) return hipSuccess;
  const dim3 grid((unsigned)tiles), block(512);
  const bool batched = counts != nullptr || plan != nullptr;
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
  const dim3 grid((unsigned)tiles), block(2048 / Policy::kRowsPerThreadRmsnorm);
  // transposed rows start every M bytes: off 16-byte boundaries their stores go out plain
  const bool aligned_rows = M % 16 == 0;
  // XCD remap (see resolve_tile): wide rows and several waves of workgroups
  // ... and, behind the statistic pass, wherever that pass handed out the rows by XCD
  const int remap = (aligned_rows && n >= 4096 && tiles >= 3072) || (mode == 2 && rmsnorm_passes_by_xcd(M, n));
  // raised priority until the loads are out: only when the whole launch is resident at once (four
  // workgroups per CU of a 256-CU device; more tiles than that arrive in generations)
  const int first = Policy::kStartPriorityRmsnorm && tiles <= 1024;
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      FQ_DISPATCH_MODE(mode, MD,
        FQ_DISPATCH_BOOL(aligned_rows, A,
          hipLaunchKernelGGL((rmsnorm_quant_tile_kernel<K, R, MD, MD == 1 ? Policy::kStoreHintRmsnormCols : A ? Policy::kStoreHintRmsnorm : (Policy::kStoreHintRmsnorm & 2)>), grid,
                             block, 0, stream, (const uint16_t*)x, (const uint16_t*)gamma, rstd, out, M, n,
                             remap, first);))))
  return hipGetLastError();
}

}  // namespace fq
