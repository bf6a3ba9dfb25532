// RMSNorm + 1x128 / 128x1 quant in ONE pass over x (linghe/utils/norm.py:343-502,
// output_mode 2; the reference uses two kernels and reads x twice).
//
// The column quantisation needs 128 rows, the row statistic needs a whole row.
// A 128-row slab of x is therefore shared by P = n/128 workgroups, one per
// 128x128 tile, each keeping its tile in registers while the slab's statistic is
// assembled through a small scratch buffer:
//   1. workgroup (slab, cb) writes the 128 per-row partial sums of squares of its
//      tile into slots  part[slab][row][cb];
//   2. it owns the rows r = cb, cb+P, cb+2P, ... of the slab: for each of them one
//      wave reads the P slots of the row, adds them in tile order 0..P-1
//      (compensated), and writes rstd into slot  stat[slab][r]  and into the rms
//      output;
//   3. every workgroup reads the 128 slots stat[slab][*], then normalises and
//      quantises its tile from registers.
// A slot is 8 bytes {value, tag}, written and read with ONE 64-bit access, so a
// reader either sees the tag of this launch together with its value or an older
// tag (the tag is a launch counter kept by the host library: nothing is ever
// reset, and slots left over from earlier launches are simply "not ready").
//
// Latency: the P workgroups of a slab are given workgroup ids that are equal
// modulo 8.  The hardware deals workgroups to the 8 XCDs round-robin by id, so
// they normally share one L2, which makes the exchange a little faster; nothing
// depends on it for correctness (all slot accesses are agent scope).
//
// Forward progress / safety: ids are slab-major per XCD and workgroups start in id
// order, so the peers a workgroup waits for are resident or start before
// anything that could block them.  Every wait is nevertheless bounded
// (wait_limit polls).  A workgroup that gives up computes
// the statistic of its 128 rows itself from global memory with exactly the same
// arithmetic and carries on, so every wave reaches the end of the kernel and the
// results do not depend on which path was taken.
#include "fq_tile_geom.cuh"
#include "fq_launch.h"

namespace fq {

constexpr int kXcds = 8;

typedef unsigned long long slot_t;  // low 32 bits: fp32 value, high 32 bits: tag

__device__ __forceinline__ slot_t make_slot(float v, uint32_t tag) {
  return (slot_t)as_u32(v) | ((slot_t)tag << 32);
}
// One 64-bit access each, at agent scope (sc1): the store writes through to the
// level every XCD sees and the load bypasses what is not coherent at that level.
// Measured on an idle MI355X, one store->load hop takes ~330 ns between
// workgroups of one XCD and ~430 ns across XCDs; plain stores are only seen by
// sc1 loads of the SAME XCD, and sc0 loads keep hitting the per-CU cache, so
// agent scope on both sides is the one combination that is correct wherever the
// workgroups run.
__device__ __forceinline__ void slot_store(slot_t* p, slot_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ slot_t slot_load(const slot_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// poll until the slot carries this launch's tag; false after `limit` polls
__device__ __forceinline__ bool slot_wait(const slot_t* p, uint32_t tag, int limit, float& value) {
  for (int it = 0; it < limit; ++it) {
    const slot_t s = slot_load(p);
    if ((uint32_t)(s >> 32) == tag) {
      value = as_f32((uint32_t)s);
      return true;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  value = 0.f;
  return false;
}

// running sum with the rounding error of every addition carried along (TwoSum):
// the total of the P partials is as good as a single rounding, whatever P
struct CompSum {
  float hi = 0.f, lo = 0.f;
  __device__ __forceinline__ void add(float x) {
    const float t = hi + x;
    const float bp = t - hi;
    lo += (hi - (t - bp)) + (x - bp);
    hi = t;
  }
  __device__ __forceinline__ float value() const { return hi + lo; }
};

__device__ __forceinline__ float rstd_of(float sumsq, int n, float eps) {
  return 1.0f / sqrtf(sumsq / (float)n + eps);
}

// per-row partial sum of squares of the thread's RPT x 8 block: lane cg == s of
// each 16-lane row returns the sum of row rg*RPT+s over the tile's 128 columns
template <int RPT>
__device__ __forceinline__ float tile_row_sumsq(const uint4 (&raw)[RPT]) {
  const int cg = threadIdx.x & 15;
  float mine = 0.f;
#pragma unroll
  for (int s = 0; s < RPT; ++s) {
    const float ss = row16_sum(sumsq8(raw[s]));
    if (cg == s) mine = ss;
  }
  return mine;
}

struct FusedShared {
  float rstd[kGroup];
  int gave_up;
};

template <int KIND, bool ROUND, int MODE>
__global__ __launch_bounds__(256, 4) void rmsnorm_quant_fused_kernel(const uint16_t* __restrict__ x,
                                                                     const uint16_t* __restrict__ gamma,
                                                                     OutPtrs out, float* __restrict__ rstd_out,
                                                                     slot_t* part_slots, slot_t* stat_slots,
                                                                     uint32_t tag, int64_t M, int n, float eps,
                                                                     int wait_limit) {
  constexpr int RPT = 8;
  __shared__ TileShared<RPT> sh;
  __shared__ FusedShared fs;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int cg = tid & 15;
  const int rg = tid >> 4;
  const int P = n / kGroup;
  // workgroup id -> (slab, tile): the tiles of a slab get ids that are equal mod 8
  const int xcd = blockIdx.x % kXcds;
  const int j = blockIdx.x / kXcds;
  const int slab = (j / P) * kXcds + xcd;
  const int cb = j - (j / P) * P;
  const int64_t row0 = (int64_t)slab * kGroup;
  if (row0 >= M) return;

  TileGeom g;
  g.cb = cb;
  g.row0 = row0;
  const int64_t left = M - row0;
  g.rows_valid = left < kGroup ? (int)left : kGroup;
  g.rows_store = g.rows_valid;
  g.s_base = row0;
  g.s_stride = M;
  g.t_base = row0;
  g.t_stride = M;
  g.st_row = slab;
  g.expert = 0;

  if (tid == 0) fs.gave_up = 0;
  uint4 raw[RPT];
  const uint16_t* slab_x = x + row0 * n;
  load_rows<RPT>(slab_x + (int64_t)cb * kGroup, n, g.rows_valid, raw);
  float gm[8];
  unpack8(*(const uint4*)(gamma + (int64_t)cb * kGroup + cg * 8), gm);

  // ---- 1. publish the partial sums of this tile
  slot_t* slab_part = part_slots + (int64_t)slab * kGroup * P;  // [row][tile]
  slot_t* slab_stat = stat_slots + (int64_t)slab * kGroup;      // [row]
  {
    const float mine = tile_row_sumsq<RPT>(raw);
    if (cg < RPT) slot_store(slab_part + (rg * RPT + cg) * P + cb, make_slot(mine, tag));
  }
  __syncthreads();  // fs.gave_up initialised

  // ---- 2. finish the statistic of the rows this workgroup owns
  for (int r = cb + wave * P; r < kGroup; r += 4 * P) {
    float pv = 0.f;
    bool ok = true;
    if (lane < P) ok = slot_wait(slab_part + r * P + lane, tag, wait_limit, pv);
    if (__builtin_amdgcn_ballot_w64(!ok) != 0) {  // wave-uniform
      if (lane == 0) fs.gave_up = 1;
      break;
    }
    CompSum tot;
    for (int p = 0; p < P; ++p) tot.add(as_f32(__builtin_amdgcn_readlane(as_u32(pv), p)));
    const float rs = rstd_of(tot.value(), n, eps);
    if (lane == 0) {
      slot_store(slab_stat + r, make_slot(rs, tag));
      if (r < g.rows_valid) rstd_out[row0 + r] = rs;
    }
  }

  // ---- 3. collect the statistic of all 128 rows
  if (tid < kGroup) {
    float rs;
    const bool ok = slot_wait(slab_stat + tid, tag, wait_limit, rs);
    fs.rstd[tid] = rs;
    if (!ok) fs.gave_up = 1;
  }
  __syncthreads();
  if (fs.gave_up) {
    // gave up waiting: recompute the statistic of the slab's 128 rows from global
    // memory, tile by tile, with exactly the arithmetic of steps 1 and 2
    CompSum tot;
    for (int p = 0; p < P; ++p) {
      uint4 tmp[RPT];
      load_rows<RPT>(slab_x + (int64_t)p * kGroup, n, g.rows_valid, tmp);
      tot.add(tile_row_sumsq<RPT>(tmp));
    }
    if (cg < RPT) {
      const int r = rg * RPT + cg;
      const float rs = rstd_of(tot.value(), n, eps);
      fs.rstd[r] = rs;
      // keep the contract of step 2 for the rows this workgroup owns
      if (r % P == cb) {
        slot_store(slab_stat + r, make_slot(rs, tag));
        if (r < g.rows_valid) rstd_out[row0 + r] = rs;
      }
    }
    __syncthreads();
  }

  // ---- normalise and quantise from registers
  float v[RPT][8];
#pragma unroll
  for (int s = 0; s < RPT; ++s) {
    const float r = fs.rstd[rg * RPT + s];
    float a[8];
    unpack8(raw[s], a);
#pragma unroll
    for (int jj = 0; jj < 8; ++jj) v[s][jj] = (a[jj] * r) * gm[jj];
  }
  quantize_tile<KIND, ROUND, MODE, RPT>(v, make_out(out, g, n, cb), sh);
}

int64_t rmsnorm_fused_scratch_bytes(int64_t M, int n) {
  const int64_t slabs = (M + kGroup - 1) / kGroup;
  const int P = n / kGroup;
  return slabs * kGroup * (int64_t)(P + 1) * (int64_t)sizeof(slot_t);
}

hipError_t launch_rmsnorm_quant_fused(const void* x, const void* gamma, void* q, float* s, float* rstd, void* qt,
                                      float* st, void* scratch_ws, uint32_t tag, int64_t M, int n, float eps,
                                      int round_scale, int mode, int kind, int wait_limit, hipStream_t stream) {
  const int64_t slabs = (M + kGroup - 1) / kGroup;
  if (slabs == 0) return hipSuccess;
  const int P = n / kGroup;
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  slot_t* part_slots = (slot_t*)scratch_ws;
  slot_t* stat_slots = part_slots + slabs * kGroup * P;
  const int64_t groups = (slabs + kXcds - 1) / kXcds;
  const dim3 grid((unsigned)(groups * P * kXcds)), block(256);
  if (wait_limit <= 0) wait_limit = 4096;
#define FQ_FUSED(MD)                                                                                          \
  FQ_DISPATCH_KIND(kind, K,                                                                                   \
    FQ_DISPATCH_BOOL(round_scale, R,                                                                          \
      hipLaunchKernelGGL((rmsnorm_quant_fused_kernel<K, R, MD>), grid, block, 0, stream, (const uint16_t*)x,  \
                         (const uint16_t*)gamma, out, rstd, part_slots, stat_slots, tag, M, n, eps,           \
                         wait_limit);))
  if (mode == 0) { FQ_FUSED(0) } else { FQ_FUSED(2) }
#undef FQ_FUSED
  return hipGetLastError();
}

}  // namespace fq
