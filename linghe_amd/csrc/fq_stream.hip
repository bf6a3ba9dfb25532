// A kernel that does no work: it reads `read_bytes` and writes `write_bytes` with the
// same 16-byte global accesses the product kernels use.  Timed on a configuration's
// own byte counts it gives the time the memory system alone needs for that
// configuration (the measured ceiling the kernels are compared with, beside the
// 8 TB/s of the data sheet); on a known size it calibrates the profiler's
// FETCH_SIZE / WRITE_SIZE counters.
//
// The ceiling is only as good as the best way of moving the bytes, so the kernel comes
// in variants: 16-byte chunks in flight per lane (4 / 8 / 16), number of workgroups
// (a multiple of the CU count, or one step per workgroup), the order in which the
// workgroups of an XCD walk the buffers, and the non-temporal hint on loads and on
// stores separately.  The benchmark takes the fastest of a short list per byte count.
#include "fq_device.hpp"
#include "fq_launch.h"

namespace fq {

// UNROLL chunks per lane and step, loads first: UNROLL*16 bytes in flight per lane
template <int UNROLL, bool NT_LOAD, bool NT_STORE>
__global__ __launch_bounds__(256) void stream_rw_kernel(const uint4* __restrict__ src, int64_t read_chunks,
                                                        uint4* __restrict__ dst, int64_t write_chunks,
                                                        uint4* __restrict__ sink, int order) {
  const int64_t most = read_chunks > write_chunks ? read_chunks : write_chunks;
  constexpr int kStep = 256 * UNROLL;  // chunks per workgroup and step
  const int64_t steps = (most + kStep - 1) / kStep;
  const int G = (int)n_wg_x();
  int wg = (int)wg_x();
  if (order == 2) {
    // workgroup i runs on XCD i % 8: give every XCD one contiguous eighth of the steps
    const int per = (G + 7) >> 3;
    const int xcd = wg & 7, slot = wg >> 3;
    const int full = (G & 7) ? (G & 7) : 8;
    wg = xcd < full ? xcd * per + slot : full * per + (xcd - full) * (per - 1) + slot;
  }
  uint4 acc = make_uint4(0, 0, 0, 0);
  // order 0: workgroup wg takes the steps wg, wg + G, wg + 2G, ... (at any time the grid works on one
  // contiguous window of the buffers); order 1 / 2: a contiguous run of per_wg steps per workgroup
  const int64_t per_wg = (steps + G - 1) / G;
  const bool strided = order == 0 || order == 3;
  int64_t s0 = strided ? wg : (int64_t)wg * per_wg;
  int64_t s1 = strided ? steps : s0 + per_wg;
  if (s1 > steps) s1 = steps;
  const int64_t ds = strided ? G : 1;
  // order 3: a step is a TILE of 16 * UNROLL rows x 256 bytes of a matrix with 4096-byte rows (the access
  // pattern of the 128 x 128 tile kernels: 16 lanes per 256-byte row segment), steps interleaved over the
  // workgroups as in order 0; the tail that does not fill a block of rows is walked linearly
  constexpr int kRowChunks = 256;                        // 16-byte chunks per matrix row
  constexpr int64_t kBlockChunks = (int64_t)16 * UNROLL * kRowChunks;  // chunks per block of rows = 16 steps
  for (int64_t s = s0; s < s1; s += ds) {
    const int64_t base = s * kStep + tid_x();
    int64_t idx[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) idx[u] = base + u * 256;
    if (order == 3) {
      const int64_t rb = s >> 4;
      if ((rb + 1) * kBlockChunks <= most) {
        const int cb = (int)(s & 15), row = ((int)tid_x() >> 4) * UNROLL, cgp = (int)tid_x() & 15;
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) idx[u] = rb * kBlockChunks + (int64_t)(row + u) * kRowChunks + cb * 16 + cgp;
      }
    }
    uint4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      v[u] = make_uint4((uint32_t)idx[u], 0, 0, 0);
      if (idx[u] < read_chunks) v[u] = load16<NT_LOAD>(src + idx[u]);
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w;
      if (idx[u] < write_chunks) store16<NT_STORE>(dst + idx[u], v[u]);
    }
  }
  // keeps the loads alive when nothing is written; never true for the all-zero or small-integer data of the bench
  if ((acc.x & acc.y & acc.z & acc.w) == 0xffffffffu) *sink = acc;
}

// chunks_per_lane: 4, 8 or 16.  workgroups: how many to launch; 0 = one step per workgroup.
// order: 0 interleaved steps, 1 a contiguous run per workgroup, 2 the same with one contiguous eighth per XCD,
// 3 interleaved steps that are tiles of 16 * chunks_per_lane rows x 256 bytes of a matrix with 4096-byte rows.
hipError_t launch_stream_rw(const void* src, int64_t read_bytes, void* dst, int64_t write_bytes, void* sink,
                            int chunks_per_lane, int64_t workgroups, int order, int nt_loads,
                            int nt_stores, hipStream_t stream) {
  const int64_t rc = read_bytes / 16, wc = write_bytes / 16;
  const int64_t most = rc > wc ? rc : wc;
  if (most == 0) return hipSuccess;
  if (chunks_per_lane != 4 && chunks_per_lane != 8 && chunks_per_lane != 16) return hipErrorInvalidValue;
  if (order < 0 || order > 3) return hipErrorInvalidValue;
  const int64_t steps = (most + 256 * chunks_per_lane - 1) / (256 * chunks_per_lane);
  int64_t wgs = workgroups <= 0 || workgroups > steps ? steps : workgroups;
  if (wgs > (1 << 30)) return hipErrorInvalidValue;
  const dim3 grid((unsigned)wgs), block(256);
#define FQ_STREAM(U, L, S)                                                                              \
  hipLaunchKernelGGL((stream_rw_kernel<U, L, S>), grid, block, 0, stream, (const uint4*)src, rc, (uint4*)dst, wc, \
                     (uint4*)sink, order)
#define FQ_STREAM_HINTS(U)                                       \
  if (nt_loads) { if (nt_stores) FQ_STREAM(U, true, true); else FQ_STREAM(U, true, false); } \
  else { if (nt_stores) FQ_STREAM(U, false, true); else FQ_STREAM(U, false, false); }
  if (chunks_per_lane == 4) { FQ_STREAM_HINTS(4) }
  else if (chunks_per_lane == 8) { FQ_STREAM_HINTS(8) }
  else { FQ_STREAM_HINTS(16) }
#undef FQ_STREAM_HINTS
#undef FQ_STREAM
  return hipGetLastError();
}

}  // namespace fq
