// A kernel that does no work: it reads `read_bytes` and writes `write_bytes` with the
// same 16-byte global accesses the product kernels use.  Timed on a configuration's
// own byte counts it gives the time the memory system alone needs for that
// configuration (the measured ceiling the kernels are compared with, beside the
// 8 TB/s of the data sheet); on a known size it calibrates the profiler's
// FETCH_SIZE / WRITE_SIZE counters.
#include "fq_device.hpp"
#include "fq_launch.h"

namespace fq {

template <bool STREAM>
__global__ __launch_bounds__(256) void stream_rw_kernel(const uint4* __restrict__ src, int64_t read_chunks,
                                                        uint4* __restrict__ dst, int64_t write_chunks,
                                                        uint4* __restrict__ sink) {
  const int64_t stride = (int64_t)gridDim.x * 256 * 4;
  const int64_t most = read_chunks > write_chunks ? read_chunks : write_chunks;
  uint4 acc = make_uint4(0, 0, 0, 0);
  // four chunks per thread and step, loads first: 64 bytes in flight per lane, as in the tile kernels
  for (int64_t base = (int64_t)blockIdx.x * 1024 + threadIdx.x; base < most; base += stride) {
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = base + u * 256;
      v[u] = make_uint4((uint32_t)i, 0, 0, 0);
      if (i < read_chunks) v[u] = load16<STREAM>(src + i);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t i = base + u * 256;
      acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w;
      if (i < write_chunks) store16<STREAM>(dst + i, v[u]);
    }
  }
  // keeps the loads alive when nothing is written; never true for the all-zero or small-integer data of the bench
  if ((acc.x & acc.y & acc.z & acc.w) == 0xffffffffu) *sink = acc;
}

hipError_t launch_stream_rw(const void* src, int64_t read_bytes, void* dst, int64_t write_bytes, void* sink,
                            int nontemporal, hipStream_t stream) {
  const int64_t rc = read_bytes / 16, wc = write_bytes / 16;
  const int64_t most = rc > wc ? rc : wc;
  if (most == 0) return hipSuccess;
  int64_t wgs = (most + 1023) / 1024;
  if (wgs > 256 * 64) wgs = 256 * 64;
  if (nontemporal)
    hipLaunchKernelGGL(stream_rw_kernel<true>, dim3((unsigned)wgs), dim3(256), 0, stream, (const uint4*)src, rc,
                       (uint4*)dst, wc, (uint4*)sink);
  else
    hipLaunchKernelGGL(stream_rw_kernel<false>, dim3((unsigned)wgs), dim3(256), 0, stream, (const uint4*)src, rc,
                       (uint4*)dst, wc, (uint4*)sink);
  return hipGetLastError();
}

}  // namespace fq
