// RMSNorm + 1x128 / 128x1 quant in ONE pass over x (linghe/utils/norm.py:343-502,
// output_mode 2; the reference uses two kernels and reads x twice).
//
// The column quantisation needs 128 rows, the row statistic needs a whole row.
// A 128-row slab of x is therefore shared by P = n/128 tiles of 128x128, worked on
// by P different workgroups at the same time, each keeping its tile in registers
// while the slab's statistic is assembled through a small scratch buffer:
//   1. the workgroup of tile (slab, cb) writes the 128 per-row partial sums of
//      squares of its tile into slots  part[slab][row][cb];
//   2. it owns the rows r = cb, cb+P, cb+2P, ... of the slab: for each of them one
//      wave reads the P slots of the row, adds them and writes rstd into slot
//      stat[slab][r]  and into the rms output;
//   3. every workgroup reads the 128 slots stat[slab][*], then normalises and
//      quantises its tile from registers.
// One such exchange hop takes 0.3-0.4 us on an idle device and several us behind the
// bulk loads and stores of a busy one, so a workgroup does not wait for it: it walks
// a sequence of tiles (tile  step*G + workgroup id,  G workgroups in the grid) as a
// pipeline of three stages that belong to three different tiles,
//      tile i+1: loads arrive, partial sums published          (stage A)
//      tile i  : owned rows finished, rstd published           (stage B)
//      tile i-1: rstd collected, tile quantised and stored     (stage C)
//      tile i+2: loads issued                                  (stage D)
// and every hop has a whole pipeline step to complete.  G is a multiple of P, so
// the P tiles of a slab are always at the same step of P neighbouring workgroups.
//
// A partial sum is the double-precision sum of the tile row's sixteen 8-element
// group sums (the arithmetic of every other kernel that computes the statistic),
// which is exact, so the total does not depend on the order of addition.  It
// travels as two 8-byte slots {low word, tag}, {high word, tag}; a slot is
// written and read with ONE 64-bit access, so a reader sees either this launch's
// tag together with its value or an older tag (the tag is a launch counter kept by
// the host library: nothing is ever reset, and slots left over from earlier
// launches are simply "not ready").
//
// Forward progress / safety: at every step the workgroups publish before they wait,
// and whatever they wait for is published by workgroups at the same or an earlier
// step, which are resident or were.  Every wait is nevertheless bounded
// (wait_limit polls).  A workgroup that gives up computes the statistic of its 128
// rows itself from global memory with exactly the same arithmetic and carries on,
// so every wave reaches the end of the kernel and the results do not depend on
// which path was taken.
#include "fq_tile_geom.cuh"
#include "fq_launch.h"

namespace fq {

// cache policy of the tile loads and of the code stores (see load16/store16)
#ifndef FQ_NT_STREAM
#define FQ_NT_STREAM 2
#endif
#ifndef FQ_LDNT_STREAM
#define FQ_LDNT_STREAM 1
#endif

typedef unsigned long long slot_t;  // low 32 bits: payload, high 32 bits: tag

__device__ __forceinline__ slot_t make_slot(uint32_t v, uint32_t tag) { return (slot_t)v | ((slot_t)tag << 32); }
// One 64-bit access each, at agent scope (sc1): the store writes through to the
// level every XCD sees and the load bypasses what is not coherent at that level
// (plain stores are only seen by sc1 loads of the SAME XCD, and sc0 loads keep
// hitting the per-CU cache, so agent scope on both sides is the one combination
// that is correct wherever the workgroups run).
__device__ __forceinline__ void slot_store(slot_t* p, slot_t v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ slot_t slot_load(const slot_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool slot_ready(slot_t s, uint32_t tag) { return (uint32_t)(s >> 32) == tag; }

__device__ __forceinline__ float rstd_of(double sumsq, int n, float eps) {
  return 1.0f / sqrtf((float)sumsq / (float)n + eps);
}

constexpr int kStreamThreads = 512;
constexpr int kStreamRpt = 4;

struct StreamShared {
  float rstd[kGroup];
  int gave_up;
};

// the tile a workgroup works on at a step of its sequence
struct StreamTile {
  bool exists;
  int slab, cb;
  int64_t row0;
  int rows_valid;
};

template <int KIND, bool ROUND>
__global__ __launch_bounds__(kStreamThreads) void rmsnorm_quant_stream_kernel(
    const uint16_t* __restrict__ x, const uint16_t* __restrict__ gamma, OutPtrs out, float* __restrict__ rstd_out,
    slot_t* part_slots, slot_t* stat_slots, uint32_t tag, int64_t M, int n, float eps, int wait_limit, int tiles,
    int steps) {
  constexpr int RPT = kStreamRpt;
  __shared__ TileShared<RPT> sh;
  __shared__ StreamShared fs;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int cg = tid & 15;
  const int rg = tid >> 4;
  const int P = n / kGroup;
  const int G = (int)gridDim.x;

  auto tile_at = [&](int step) {
    StreamTile t;
    const int id = step * G + (int)blockIdx.x;
    t.exists = step >= 0 && step < steps && id < tiles;
    t.slab = id / P;
    t.cb = id - t.slab * P;
    t.row0 = (int64_t)t.slab * kGroup;
    const int64_t left = M - t.row0;
    t.rows_valid = left < kGroup ? (int)left : kGroup;
    return t;
  };
  auto issue_loads = [&](const StreamTile& t, uint4 (&raw)[RPT]) {
    load_rows<RPT, FQ_LDNT_STREAM != 0>(x + t.row0 * n + (int64_t)t.cb * kGroup, n, t.rows_valid, raw);
  };
  // stage A: partial sums of the tile's rows -> part[slab][row][cb]
  auto publish_partials = [&](const StreamTile& t, const uint4 (&raw)[RPT]) {
    double mine = 0.0;
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
      const double ss = row16_sum_d((double)sumsq8(raw[s]));
      if (cg == s) mine = ss;
    }
    if (cg < RPT) {
      const uint64_t bits = __builtin_bit_cast(uint64_t, mine);
      slot_t* p = part_slots + (((int64_t)t.slab * kGroup + rg * RPT + cg) * P + t.cb) * 2;
      slot_store(p, make_slot((uint32_t)bits, tag));
      slot_store(p + 1, make_slot((uint32_t)(bits >> 32), tag));
    }
  };
  // stage B: finish the rows this tile's workgroup owns (wave w: row cb + w*P).  The
  // first look at the slots is a pair of loads issued at the top of the pipeline step
  // (poll_owned), so that their latency passes while stage A works.
  auto poll_owned = [&](const StreamTile& t, slot_t& lo, slot_t& hi) {
    lo = make_slot(0, tag);
    hi = make_slot(0, tag);
    const int r = t.cb + wave * P;
    if (r < kGroup && lane < P) {
      const slot_t* p = part_slots + (((int64_t)t.slab * kGroup + r) * P + lane) * 2;
      lo = slot_load(p);
      hi = slot_load(p + 1);
    }
  };
  auto finish_owned_rows = [&](const StreamTile& t, slot_t lo, slot_t hi) {
    bool first = true;
    for (int r = t.cb + wave * P; r < kGroup; r += (kStreamThreads / 64) * P) {
      const slot_t* p = part_slots + (((int64_t)t.slab * kGroup + r) * P + lane) * 2;
      double d = 0.0;
      bool ok = false;
      for (int it = 0; it < wait_limit; ++it) {
        if (!first) {
          lo = make_slot(0, tag);
          hi = make_slot(0, tag);
          if (lane < P) {
            lo = slot_load(p);
            hi = slot_load(p + 1);
          }
        }
        first = false;
        const bool ready = slot_ready(lo, tag) && slot_ready(hi, tag);
        if (__builtin_amdgcn_ballot_w64(!ready) == 0) {
          d = __builtin_bit_cast(double, (uint64_t)(uint32_t)lo | ((uint64_t)(uint32_t)hi << 32));
          ok = true;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      if (!ok) return;  // the collecting stage of this tile will not find the row and recomputes
      const float rs = rstd_of(wave_sum_d(d), n, eps);
      if (lane == 0) {
        slot_store(stat_slots + (int64_t)t.slab * kGroup + r, make_slot(as_u32(rs), tag));
        if (r < t.rows_valid) rstd_out[t.row0 + r] = rs;
      }
    }
  };
  // stage C: collect rstd of the slab (first look issued early by poll_stat), normalise
  // and quantise the tile from registers
  auto poll_stat = [&](const StreamTile& t, slot_t& v) {
    v = 0;
    if (tid < kGroup) v = slot_load(stat_slots + (int64_t)t.slab * kGroup + tid);
  };
  auto finish_tile = [&](const StreamTile& t, const uint4 (&raw)[RPT], slot_t seen) {
    if (tid == 0) fs.gave_up = 0;
    __syncthreads();
    if (tid < kGroup) {
      const slot_t* p = stat_slots + (int64_t)t.slab * kGroup + tid;
      bool ok = false;
      for (int it = 0; it < wait_limit; ++it) {
        if (it) seen = slot_load(p);
        if (slot_ready(seen, tag)) {
          fs.rstd[tid] = as_f32((uint32_t)seen);
          ok = true;
          break;
        }
        __builtin_amdgcn_s_sleep(2);
      }
      if (!ok) fs.gave_up = 1;
    }
    __syncthreads();
    if (fs.gave_up) {
      // gave up waiting: the statistic of the slab's 128 rows from global memory, tile
      // by tile, with the arithmetic of stages A and B
      double tot = 0.0;
      for (int p = 0; p < P; ++p) {
        uint4 tmp[RPT];
        load_rows<RPT>(x + t.row0 * n + (int64_t)p * kGroup, n, t.rows_valid, tmp);
#pragma unroll
        for (int s = 0; s < RPT; ++s) {
          const double ss = row16_sum_d((double)sumsq8(tmp[s]));
          if (cg == s) tot += ss;
        }
      }
      if (cg < RPT) {
        const int r = rg * RPT + cg;
        const float rs = rstd_of(tot, n, eps);
        fs.rstd[r] = rs;
        if (r % P == t.cb) {  // keep the owner's contract for the others
          slot_store(stat_slots + (int64_t)t.slab * kGroup + r, make_slot(as_u32(rs), tag));
          if (r < t.rows_valid) rstd_out[t.row0 + r] = rs;
        }
      }
      __syncthreads();
    }
    float gm[8];
    unpack8(*(const uint4*)(gamma + (int64_t)t.cb * kGroup + cg * 8), gm);
    float v[RPT][8];
#pragma unroll
    for (int s = 0; s < RPT; ++s) {
      const float r = fs.rstd[rg * RPT + s];
      float a[8];
      unpack8(raw[s], a);
#pragma unroll
      for (int j = 0; j < 8; ++j) v[s][j] = (a[j] * r) * gm[j];
    }
    TileGeom g;
    g.cb = t.cb;
    g.row0 = t.row0;
    g.rows_valid = t.rows_valid;
    g.rows_store = t.rows_valid;
    g.s_base = t.row0;
    g.s_stride = M;
    g.t_base = t.row0;
    g.t_stride = M;
    g.st_row = t.slab;
    g.expert = 0;
    g.valid = true;
    quantize_tile<KIND, ROUND, 2, RPT, FQ_NT_STREAM>(v, make_out(out, g, n, t.cb), sh);
  };

  // three tiles in registers with fixed roles: ra = tile i+1 (arriving), rw = tile i
  // (its statistic is travelling), rc = tile i-1 (being finished).  After stage C the
  // roles move up by register copies of two loaded tiles (32 moves per step), then
  // the next tile's loads go into ra.
  uint4 ra[RPT], rw[RPT], rc[RPT];
  {
    const StreamTile t0 = tile_at(0), t1 = tile_at(1);
    if (t0.exists) issue_loads(t0, rw);
    if (t1.exists) issue_loads(t1, ra);
    if (t0.exists) publish_partials(t0, rw);
  }
  // iteration i: A(i+1), B(i), C(i-1), D(i+2)
#pragma unroll 1
  for (int i = 0; i <= steps; ++i) {
    const StreamTile ta = tile_at(i + 1), tb = tile_at(i), tc = tile_at(i - 1), td = tile_at(i + 2);
    slot_t olo = 0, ohi = 0, sv = 0;
    if (tb.exists) poll_owned(tb, olo, ohi);
    if (tc.exists) poll_stat(tc, sv);
    if (ta.exists) publish_partials(ta, ra);
    if (tb.exists) finish_owned_rows(tb, olo, ohi);
    if (tc.exists) finish_tile(tc, rc, sv);
#pragma unroll
    for (int k = 0; k < RPT; ++k) {
      rc[k] = rw[k];
      rw[k] = ra[k];
    }
    if (td.exists) issue_loads(td, ra);
  }
}

int64_t rmsnorm_fused_scratch_bytes(int64_t M, int n) {
  const int64_t slabs = (M + kGroup - 1) / kGroup;
  const int P = n / kGroup;
  return slabs * kGroup * (int64_t)(2 * P + 1) * (int64_t)sizeof(slot_t);
}

hipError_t launch_rmsnorm_quant_fused(const void* x, const void* gamma, void* q, float* s, float* rstd, void* qt,
                                      float* st, void* scratch_ws, uint32_t tag, int64_t M, int n, float eps,
                                      int round_scale, int mode, int kind, int wait_limit, hipStream_t stream) {
  const int64_t slabs = (M + kGroup - 1) / kGroup;
  if (slabs == 0) return hipSuccess;
  (void)mode;
  const int P = n / kGroup;
  const int64_t tiles = slabs * P;
  OutPtrs out{(uint8_t*)q, s, (uint8_t*)qt, st};
  slot_t* part_slots = (slot_t*)scratch_ws;
  slot_t* stat_slots = part_slots + slabs * kGroup * P * 2;
  // The workgroups of a step wait for each other, so the whole grid must be resident:
  // G = P * (slabs per step) <= what the device holds of this kernel.
  int dev = 0, cus = 0, per_cu = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return e;
  const void* fn = nullptr;
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R, fn = (const void*)rmsnorm_quant_stream_kernel<K, R>;))
  e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, fn, kStreamThreads, 0);
  if (e != hipSuccess) return e;
  if (per_cu < 1 || cus < 1) return hipErrorInvalidValue;
  int64_t per_step = ((int64_t)per_cu * cus) / P;
  if (per_step < 1) return hipErrorInvalidValue;  // not even one slab fits: the caller takes two passes
  if (per_step > slabs) per_step = slabs;
  const int64_t G = per_step * P;
  const int steps = (int)((tiles + G - 1) / G);
  if (wait_limit <= 0) wait_limit = 4096;
  const dim3 grid((unsigned)G), block(kStreamThreads);
  FQ_DISPATCH_KIND(kind, K,
    FQ_DISPATCH_BOOL(round_scale, R,
      hipLaunchKernelGGL((rmsnorm_quant_stream_kernel<K, R>), grid, block, 0, stream, (const uint16_t*)x,
                         (const uint16_t*)gamma, out, rstd, part_slots, stat_slots, tag, M, n, eps, wait_limit,
                         (int)tiles, steps);))
  return hipGetLastError();
}

}  // namespace fq
