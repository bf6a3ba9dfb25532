// Row kernels: a workgroup owns whole rows (the RMSNorm statistic needs the full
// row) and keeps the row in registers between the reduction and the outputs, so
// every element is read from HBM once.
//   rmsnorm_fwd          bf16 RMSNorm                       (linghe/utils/norm.py:13-93)
//   rmsnorm_quant_row    RMSNorm + row-wise 1x128 quant      (linghe/utils/norm.py:252-297)
//   rmsnorm_bwd          dx (bf16) + dgamma partial sums      (linghe/utils/norm.py:96-179)
//   colsum               dgamma = sum of the partials
//   group_quant          row-wise 1x128 quant, scale [M, N/128] (linghe/quant/group.py:11-63)
//
// Thread t of a T-thread workgroup owns the 8-column chunks t, t+T, t+2T, ...
// (one 128-bit load each); 16 consecutive lanes therefore share a 128-column
// quantisation group.  The next row is prefetched while the current one is
// processed.
#include <mutex>

#include "fq_device.hpp"
#include "fq_launch.h"
#include "fq_policy.hpp"

namespace fq {

// cache hints of the row kernels: fq_policy.hpp
__device__ __forceinline__ void st16(void* p, const uint4& v) { store16<Policy::kStoreHintRows>(p, v); }
__device__ __forceinline__ void st8(void* p, const uint2& v) { store8<Policy::kStoreHintRows>(p, v); }
__device__ __forceinline__ uint4 ld16(const void* p) { return load16<Policy::kLoadHintRows>(p); }


template <int T>
struct RowShared {
  float red[2][2][T / 64];  // [parity][value][wave]
  double redd[2][T / 64];   // [parity][wave]
};

// sum of (a, b) over the workgroup, fixed order; one barrier per call
template <int T>
__device__ __forceinline__ void block_sum2(float& a, float& b, RowShared<T>& sh, int parity) {
  a = wave_sum(a);
  b = wave_sum(b);
  if constexpr (T > 64) {
    const int wave = tid_x() >> 6;
    if ((tid_x() & 63) == 0) {
      sh.red[parity][0][wave] = a;
      sh.red[parity][1][wave] = b;
    }
    __syncthreads();
    a = sh.red[parity][0][0];
    b = sh.red[parity][1][0];
#pragma unroll
    for (int w = 1; w < T / 64; ++w) {
      a += sh.red[parity][0][w];
      b += sh.red[parity][1][w];
    }
  }
}

// the same with the first value a double
template <int T>
__device__ __forceinline__ void block_sum2(double& a, float& b, RowShared<T>& sh, int parity) {
  a = wave_sum_d(a);
  b = wave_sum(b);
  if constexpr (T > 64) {
    const int wave = tid_x() >> 6;
    if ((tid_x() & 63) == 0) {
      sh.redd[parity][wave] = a;
      sh.red[parity][1][wave] = b;
    }
    __syncthreads();
    a = sh.redd[parity][0];
    b = sh.red[parity][1][0];
#pragma unroll
    for (int w = 1; w < T / 64; ++w) {
      a += sh.redd[parity][w];
      b += sh.red[parity][1][w];
    }
  }
}

template <int T, int NCHUNK, bool STREAM = false>
__device__ __forceinline__ void load_row(const uint16_t* row, int n, uint4 (&raw)[NCHUNK]) {
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) {
    const int c = tid_x() + k * T;
    raw[k] = make_uint4(0, 0, 0, 0);
    if (c * 8 < n) raw[k] = load16<STREAM>(row + c * 8);
  }
}

// The same without a branch: a chunk beyond the end of the row reads the row's last
// chunk again (a valid address).  Loads that sit behind a per-lane condition are issued
// one by one, each behind its own exec-mask branch; these go out back to back.  What is
// computed from such a chunk must not be stored, and must be left out of row sums
// (sumsq_live).
template <int T, int NCHUNK, bool STREAM = false>
__device__ __forceinline__ void load_row_clamped(const uint16_t* row, int n, uint4 (&raw)[NCHUNK]) {
  const int last = (n >> 3) - 1;
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) {
    const int c = tid_x() + k * T;
    raw[k] = load16<STREAM>(row + (c < last ? c : last) * 8);
  }
}

// make the compiler forget what it knows about a packed row, so that the fp32
// copies made before a reduction are not kept alive across it (they are cheap to
// remake and cost four times the registers)
template <int NCHUNK>
__device__ __forceinline__ void forget(uint4 (&raw)[NCHUNK]) {
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k)
    asm volatile("" : "+v"(raw[k].x), "+v"(raw[k].y), "+v"(raw[k].z), "+v"(raw[k].w));
}

__device__ __forceinline__ float rstd_from_sumsq(float ss, int n, float eps) {
  // rsqrt(sum/n + eps) as the fp32 CPU oracle evaluates it: true division,
  // correctly rounded sqrt, true reciprocal
  return 1.0f / sqrtf(ss / (float)n + eps);
}

// the thread's share of a row's sum of squares: every aligned group of 8 elements
// is summed in fp32 in a fixed order (exact products), the groups are added in
// double.  The row total then does not depend on how the groups are split over
// lanes and waves, so every kernel that computes the statistic (forward,
// backward, any row shape) gets the same fp32 value: the exact sum of the group
// sums, rounded once
template <int NCHUNK>
__device__ __forceinline__ double sumsq(const uint4 (&raw)[NCHUNK]) {
  double ss = 0.0;
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) ss += (double)sumsq8(raw[k]);
  return ss;
}
// the same for a row fetched by load_row_clamped: chunks beyond the end of the row count as zero
template <int T, int NCHUNK>
__device__ __forceinline__ double sumsq_live(const uint4 (&raw)[NCHUNK], int n) {
  double ss = 0.0;
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) {
    const float part = sumsq8(raw[k]);
    ss += (double)((((int)tid_x() & (T - 1)) + k * T) * 8 < n ? part : 0.f);  // T a power of two; a wave-per-row kernel passes T = 64
  }
  return ss;
}

// ---------------------------------------------------------------------------
// forward: OUT = 0 -> bf16 y ; 1 -> fp8 codes + [nb, M] scales
// ---------------------------------------------------------------------------
template <int T, int NCHUNK, bool REUSE, int OUT, int KIND, bool ROUND>
__global__ __launch_bounds__(T) void rmsnorm_fwd_kernel(const uint16_t* __restrict__ x,
                                                        const uint16_t* __restrict__ gamma, void* __restrict__ out,
                                                        float* __restrict__ scale, float* __restrict__ rstd,
                                                        int64_t M, int n, float eps, int rows_per_wg) {
  __shared__ RowShared<T> sh;
  const int tid = tid_x();
  uint4 gm[NCHUNK];
  load_row<T, NCHUNK>(gamma, n, gm);
  const int64_t G = n_wg_x();  // rows b, b + G, b + 2G, ... with b the workgroup's logical index:
  // workgroup i runs on XCD i % 8, and every XCD takes one contiguous eighth of the
  // indices in the quantising form (3-7 % faster; the bf16 form is 8-20 % slower with it)
  int64_t r0 = wg_x();
  if constexpr (OUT == 1 && Policy::kXcdContiguousRowQuant) {
    const int Gi = (int)n_wg_x();
    const int per = (Gi + 7) >> 3;
    const int xcd = (int)wg_x() & 7, slot = (int)wg_x() >> 3;
    const int full = (Gi & 7) ? (Gi & 7) : 8;
    r0 = xcd < full ? xcd * per + slot : full * per + (xcd - full) * (per - 1) + slot;
  }
  const int64_t r1 = M;
  (void)rows_per_wg;
  if (r0 >= r1) return;

  auto process = [&](const uint4 (&raw)[NCHUNK], int64_t row, int parity) {
    float r;
    if constexpr (REUSE) {
      r = rstd[row];
    } else {
      double ss = sumsq_live<T, NCHUNK>(raw, n);
      float dummy = 0.f;
      block_sum2<T>(ss, dummy, sh, parity);
      r = rstd_from_sumsq((float)ss, n, eps);
      if (tid == 0) rstd[row] = r;
    }
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      const int c = tid + k * T;
      float a[8], w[8], y[8];
      unpack8(raw[k], a);
      unpack8(gm[k], w);
#pragma unroll
      for (int j = 0; j < 8; ++j) y[j] = (a[j] * r) * w[j];
      if constexpr (OUT == 0) {
        if (c * 8 < n) st16((uint16_t*)out + row * n + c * 8, pack8_bf16(y));
      } else {
        float m = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(y[j]));
        m = row16_max(m);
        const float sc = make_scale<KIND, ROUND>(m);
        const uint2 pk = quantize8<KIND, ROUND>(y, make_quantum<ROUND>(sc));
        if (c * 8 < n) {
          // codes of wide rows (the four-waves-per-row form) go out with ordinary stores: 71 -> 67.6 us at
          // 16384 x 7168; narrow rows keep the hint (12.5 against 13.0 us at 8192 x 2048)
          store8<Policy::kStoreHintRows && T == 64>((uint8_t*)out + row * n + c * 8, pk);
          if ((c & 15) == 0) scale[(int64_t)(c >> 4) * M + row] = sc;
        }
      }
    }
  };

  if constexpr (OUT == 1 && !(T == 256 && Policy::kPrefetchRowQuantWide)) {
    // the quantising form has enough arithmetic per row to want several waves per SIMD:
    // one row in registers, the other waves cover its loads
    uint4 buf[NCHUNK];
    int parity = 0;
    // the first row's loads leave before gamma is waited for (see the fences below)
    load_row_clamped<T, NCHUNK, Policy::kLoadHintRows>(x + r0 * n, n, buf);
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) fence_packed(gm[k]);
    for (int64_t row = r0;;) {
      process(buf, row, parity);
      parity ^= 1;
      row += G;
      if (row >= r1) break;
      load_row_clamped<T, NCHUNK, Policy::kLoadHintRows>(x + row * n, n, buf);
    }
    return;
  }
  uint4 bufA[NCHUNK], bufB[NCHUNK];
  load_row_clamped<T, NCHUNK, Policy::kLoadHintRows>(x + r0 * n, n, bufA);
  // gamma is widened to fp32 once, before the loop; fenced here so that this happens (and gamma is
  // waited for) after the first row's loads have left, not before (a wave has only M / 8192 rows)
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) fence_packed(gm[k]);
  for (int64_t row = r0; row < r1; row += 2 * G) {
    if (row + G < r1) load_row_clamped<T, NCHUNK, Policy::kLoadHintRows>(x + (row + G) * n, n, bufB);
    process(bufA, row, 0);
    if (row + G < r1) {
      if (row + 2 * G < r1) load_row_clamped<T, NCHUNK, Policy::kLoadHintRows>(x + (row + 2 * G) * n, n, bufA);
      process(bufB, row + G, 1);
    }
  }
}

// ---------------------------------------------------------------------------
// statistic only (the first pass of RMSNorm + quant, output_mode 2): one wave per
// row, eight 16-byte loads per lane in flight, nothing kept.  Few registers, so a
// CU holds its 32 waves and a 16384-row input is two rows per wave with no tail.
// Same arithmetic as everywhere else: 8-element group sums added in double.
// ---------------------------------------------------------------------------
// U: 16-byte loads per lane and step (a step covers U * 512 columns); 4 for rows of at most 2048
// columns, 8 beyond.  The loads carry no per-lane condition: a chunk beyond the end of the row
// reads the row's last chunk again and counts as zero.
template <int U>
__global__ __launch_bounds__(64 * Policy::kRowstatWaves) void rowstat_kernel(const uint16_t* __restrict__ x, float* __restrict__ rstd,
                                                     int64_t M, int n, float eps, int by_xcd) {
  constexpr int kW = Policy::kRowstatWaves;  // waves (rows) per workgroup
  const int lane = tid_x() & 63;
  const int chunks = n >> 3;
  // Rows are taken from the END of the matrix backwards.  The tile kernel that follows
  // walks the matrix forwards, so it starts with the rows this kernel read last, which
  // are the ones still in the last-level cache: for an input about the size of that
  // cache roughly half of the second read never reaches HBM.
  // by_xcd: workgroup w runs on XCD w % 8, and XCD X takes the X-th eighth of the rows, again from its
  // end backwards: the tile kernel hands the same eighth to the same XCD (rmsnorm_passes_by_xcd)
  const int64_t span = by_xcd ? M >> 3 : M;
  const int64_t first = by_xcd ? (int64_t)(wg_x() & 7) * span : 0;
  const int64_t k0 = by_xcd ? (int64_t)(wg_x() >> 3) * kW + (tid_x() >> 6) : (int64_t)wg_x() * kW + (tid_x() >> 6);
  const int64_t step = by_xcd ? (int64_t)(n_wg_x() >> 3) * kW : (int64_t)n_wg_x() * kW;
  for (int64_t k = k0; k < span; k += step) {
    const int64_t row = first + span - 1 - k;
    const uint4* p = (const uint4*)(x + row * n);
    double ss = 0.0;
    for (int c0 = 0; c0 < chunks; c0 += U * 64) {
      uint4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = c0 + u * 64 + lane;
        v[u] = p[c < chunks ? c : chunks - 1];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float part = sumsq8(v[u]);
        ss += (double)(c0 + u * 64 + lane < chunks ? part : 0.f);
      }
    }
    ss = wave_sum_d(ss);
    if (lane == 0) rstd[row] = rstd_from_sumsq((float)ss, n, eps);
  }
}

// ---------------------------------------------------------------------------
// backward: dx = r*g*w - r^3 * x * sum(x*g*w)/n ; dgamma partial += x*g*r
// ---------------------------------------------------------------------------
template <int T, int NCHUNK, bool REUSE>
__global__ __launch_bounds__(T, 4) void rmsnorm_bwd_kernel(const uint16_t* __restrict__ dy,
                                                        const uint16_t* __restrict__ x,
                                                        const uint16_t* __restrict__ gamma,
                                                        const float* __restrict__ rstd_in,
                                                        uint16_t* __restrict__ dx, float* __restrict__ dg_part,
                                                        int64_t M, int n, float eps, int rows_per_wg) {
  __shared__ RowShared<T> sh;
  const int tid = tid_x();
  const int chunks = n >> 3;
  // A thread's chunk k is column chunk tid + k*T.  Beyond the end of the row it reads the
  // row's last chunk again (a valid address, no branch) and takes part with gamma = 0:
  // its share of the row sums is zero and none of its results is stored.
  int cidx[NCHUNK];
  bool live[NCHUNK];
  float w[NCHUNK][8];  // gamma, unpacked once
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) {
    const int c = tid + k * T;
    live[k] = c < chunks;
    cidx[k] = live[k] ? c : chunks - 1;
    unpack8(*(const uint4*)(gamma + cidx[k] * 8), w[k]);
    if (!live[k]) {
#pragma unroll
      for (int j = 0; j < 8; ++j) w[k][j] = 0.f;
    }
  }
  float acc[NCHUNK][8];
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[k][j] = 0.f;

  // rows wg_x(), wg_x() + G, wg_x() + 2G, ...: at any moment the
  // workgroups of the grid work on neighbouring rows (one moving front in memory)
  const int64_t G = n_wg_x();
  (void)rows_per_wg;

  // One row in registers at a time (about 100 of them with two chunks per thread), so
  // that two 512-thread workgroups fit a CU and cover each other's waits.  Prefetching
  // the next row's packed data into a second register set spills (142 -> 198 us at
  // 16384 x 7168 with 512 threads, 155 -> 179 us with 256 threads and four chunks).
  auto fetch = [&](int64_t row, uint4 (&rx)[NCHUNK], uint4 (&rg)[NCHUNK]) {
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      rx[k] = load16<Policy::kLoadHintRows>(x + row * n + cidx[k] * 8);
      rg[k] = load16<Policy::kLoadHintRows>(dy + row * n + cidx[k] * 8);
    }
  };
  auto process = [&](int64_t row, uint4 (&rx)[NCHUNK], uint4 (&rg)[NCHUNK], int parity) {
    double ss = 0.0;
    float dot = 0.f;
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      float a[8], g[8];
      unpack8(rx[k], a);
      unpack8(rg[k], g);
      if constexpr (!REUSE) {
        const float part = sumsq8(rx[k]);
        ss += (double)(live[k] ? part : 0.f);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) dot = __builtin_fmaf(a[j] * g[j], w[k][j], dot);
    }
    if constexpr (REUSE) {
      float unused = 0.f;
      block_sum2<T>(unused, dot, sh, parity);
    } else {
      block_sum2<T>(ss, dot, sh, parity);
    }
    forget<NCHUNK>(rx);
    forget<NCHUNK>(rg);
    float r;
    if constexpr (REUSE) r = rstd_in[row];
    else r = rstd_from_sumsq((float)ss, n, eps);
    const float coef = ((r * r) * r) * dot / (float)n;
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      float a[8], g[8], o[8];
      unpack8(rx[k], a);
      unpack8(rg[k], g);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        o[j] = (r * g[j]) * w[k][j] - coef * a[j];
        acc[k][j] = __builtin_fmaf(a[j] * g[j], r, acc[k][j]);  // dgamma: one rounding fewer per term
      }
      if (live[k]) st16(dx + row * n + cidx[k] * 8, pack8_bf16(o));
    }
  };
  if constexpr (Policy::kPrefetchRowBwdWide && NCHUNK == 1) {
    uint4 xa[NCHUNK], ga[NCHUNK], xb[NCHUNK], gb[NCHUNK];
    const int64_t r0 = wg_x();
    if (r0 < M) fetch(r0, xa, ga);
    for (int64_t row = r0; row < M; row += 2 * G) {
      if (row + G < M) fetch(row + G, xb, gb);
      process(row, xa, ga, 0);
      if (row + G < M) {
        if (row + 2 * G < M) fetch(row + 2 * G, xa, ga);
        process(row + G, xb, gb, 1);
      }
    }
  } else {
    int parity = 0;
    for (int64_t row = wg_x(); row < M; row += G) {
      uint4 rx[NCHUNK], rg[NCHUNK];
      fetch(row, rx, rg);
      process(row, rx, rg, parity);
      parity ^= 1;
    }
  }
  // every workgroup writes its (possibly zero) partial: the reduction reads all of them
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) {
    const int c = tid + k * T;
    if (c * 8 < n) {
      float4* dst = (float4*)(dg_part + (int64_t)wg_x() * n + c * 8);
      dst[0] = make_float4(acc[k][0], acc[k][1], acc[k][2], acc[k][3]);
      dst[1] = make_float4(acc[k][4], acc[k][5], acc[k][6], acc[k][7]);
    }
  }
}

// Backward for narrow rows (n <= 2048): one wave per row, so the two row sums are
// wave reductions and no barrier or LDS traffic sits between a row's loads and its
// stores.  The four waves of a workgroup walk their own rows and keep their own
// dgamma accumulators, added in wave order at the end: one partial row per workgroup
// as in the kernel above.  Lane l holds the 16-byte chunks l, l+64, ...
template <int NCHUNK, bool REUSE>
__global__ __launch_bounds__(256) void rmsnorm_bwd_wave_kernel(const uint16_t* __restrict__ dy,
                                                               const uint16_t* __restrict__ x,
                                                               const uint16_t* __restrict__ gamma,
                                                               const float* __restrict__ rstd_in,
                                                               uint16_t* __restrict__ dx,
                                                               float* __restrict__ dg_part, int64_t M, int n,
                                                               float eps) {
  __shared__ float4 combine[3][NCHUNK * 2][64];  // waves 1..3: [chunk half][lane]
  const int lane = tid_x() & 63;
  const int wave = tid_x() >> 6;
  const int chunks = n >> 3;
  float w[NCHUNK][8];  // gamma, unpacked once; zero beyond the end of the row
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k) {
    const int c = lane + k * 64;
    uint4 gm = make_uint4(0, 0, 0, 0);
    if (c < chunks) gm = *(const uint4*)(gamma + c * 8);
    unpack8(gm, w[k]);
  }
  float acc[NCHUNK][8];
#pragma unroll
  for (int k = 0; k < NCHUNK; ++k)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[k][j] = 0.f;

  const int64_t stride = (int64_t)n_wg_x() * 4;
  for (int64_t row = (int64_t)wg_x() * 4 + wave; row < M; row += stride) {
    uint4 rx[NCHUNK], rg[NCHUNK];
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      // no per-lane condition on the loads: a chunk beyond the end of the row reads the last
      // chunk again; its gamma is zero, so it adds nothing to the row sums, and it is not stored
      const int c = lane + k * 64;
      const int cc = c < chunks ? c : chunks - 1;
      rx[k] = ld16(x + row * n + cc * 8);
      rg[k] = ld16(dy + row * n + cc * 8);
    }
    float dot = 0.f;
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      float a[8], g[8];
      unpack8(rx[k], a);
      unpack8(rg[k], g);
#pragma unroll
      for (int j = 0; j < 8; ++j) dot = __builtin_fmaf(a[j] * g[j], w[k][j], dot);
    }
    dot = wave_sum(dot);
    float r;
    if constexpr (REUSE) {
      r = rstd_in[row];
    } else {
      r = rstd_from_sumsq((float)wave_sum_d(sumsq_live<64, NCHUNK>(rx, n)), n, eps);
    }
    const float coef = ((r * r) * r) * dot / (float)n;
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      const int c = lane + k * 64;
      float a[8], g[8], o[8];
      unpack8(rx[k], a);
      unpack8(rg[k], g);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        o[j] = (r * g[j]) * w[k][j] - coef * a[j];
        acc[k][j] = __builtin_fmaf(a[j] * g[j], r, acc[k][j]);
      }
      if (c < chunks) st16(dx + row * n + c * 8, pack8_bf16(o));
    }
  }
  // waves 1..3 hand their accumulators to wave 0, which adds them in wave order
  if (wave > 0) {
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
      combine[wave - 1][2 * k][lane] = make_float4(acc[k][0], acc[k][1], acc[k][2], acc[k][3]);
      combine[wave - 1][2 * k + 1][lane] = make_float4(acc[k][4], acc[k][5], acc[k][6], acc[k][7]);
    }
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int k = 0; k < NCHUNK; ++k) {
#pragma unroll
      for (int w = 0; w < 3; ++w) {
        const float4 lo = combine[w][2 * k][lane], hi = combine[w][2 * k + 1][lane];
        acc[k][0] += lo.x; acc[k][1] += lo.y; acc[k][2] += lo.z; acc[k][3] += lo.w;
        acc[k][4] += hi.x; acc[k][5] += hi.y; acc[k][6] += hi.z; acc[k][7] += hi.w;
      }
      const int c = lane + k * 64;
      if (c < chunks) {
        float4* dst = (float4*)(dg_part + (int64_t)wg_x() * n + c * 8);
        dst[0] = make_float4(acc[k][0], acc[k][1], acc[k][2], acc[k][3]);
        dst[1] = make_float4(acc[k][4], acc[k][5], acc[k][6], acc[k][7]);
      }
    }
  }
}

// dgamma[c] = sum_p part[p, c] in a fixed order: 16 strided slices of p, each
// summed sequentially (loads issued eight ahead), then combined 0..15.
// 64 columns per workgroup of 1024 threads.
constexpr int kColsumSlices = 16;
__global__ __launch_bounds__(1024) void colsum_kernel(const float* __restrict__ part, float* __restrict__ out,
                                                      int P, int n) {
  __shared__ float red[kColsumSlices][64];
  const int lane = tid_x() & 63;
  const int col = wg_x() * 64 + lane;
  const int slice = tid_x() >> 6;
  float acc = 0.f;
  if (col < n) {
    const float* src = part + col;
    int p = slice;
    for (; p + 7 * kColsumSlices < P; p += 8 * kColsumSlices) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = src[(int64_t)(p + u * kColsumSlices) * n];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc += v[u];
    }
    for (; p < P; p += kColsumSlices) acc += src[(int64_t)p * n];
  }
  red[slice][lane] = acc;
  __syncthreads();
  if (slice == 0 && col < n) {
    float tot = red[0][lane];
#pragma unroll
    for (int k = 1; k < kColsumSlices; ++k) tot += red[k][lane];
    out[col] = tot;
  }
}

// ---------------------------------------------------------------------------
// row-wise 1x128 group quant of a flat run of groups (scale index == group index)
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND>
__global__ __launch_bounds__(256) void group_quant_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ q,
                                                          float* __restrict__ s, int64_t n_groups) {
  const int64_t g0 = ((int64_t)wg_x() * 256 + tid_x()) >> 4;
  const int64_t stride = ((int64_t)n_wg_x() * 256) >> 4;
  const int sub = tid_x() & 15;
  // kU groups per thread and step, their loads in flight together.  No condition on loads or stores: a
  // group beyond the end repeats the last group (same result stored to the same place again).
  constexpr int kU = Policy::kGroupQuantUnroll;
  for (int64_t g = g0; g < n_groups; g += kU * stride) {
    uint4 raw[kU];
    int64_t gi[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      gi[u] = g + u * stride < n_groups ? g + u * stride : n_groups - 1;
      raw[u] = ld16(x + gi[u] * kGroup + sub * 8);
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      float a[8];
      unpack8(raw[u], a);
      float m = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(a[j]));
      m = row16_max(m);
      const float sc = make_scale<KIND, ROUND>(m);
      const uint2 pk = quantize8<KIND, ROUND>(a, make_quantum<ROUND>(sc));
      st8(q + gi[u] * kGroup + sub * 8, pk);
      if (sub == 0) s[gi[u]] = sc;
    }
  }
}

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------
// Forward kernels: one wave per row (64-thread workgroups, no barrier), every load
// of a row in flight at once and the next row prefetched.
// Backward kernels: one wave per row up to n = 2048, 512 threads per row beyond (they
// also carry the dgamma accumulators).
static void pick_row_shape(int n, int T, int& nchunk) {
  const int chunks = (n + 7) / 8;
  nchunk = (chunks + T - 1) / T;
}

#define FQ_ROW_CASE(TT, NC, ...) \
  if (nchunk == NC) { constexpr int kT = TT; constexpr int kNC = NC; __VA_ARGS__ } else
#define FQ_FWD_SHAPES(...)                                                                         \
  FQ_ROW_CASE(64, 1, __VA_ARGS__) FQ_ROW_CASE(64, 2, __VA_ARGS__) FQ_ROW_CASE(64, 3, __VA_ARGS__)  \
  FQ_ROW_CASE(64, 4, __VA_ARGS__) FQ_ROW_CASE(64, 5, __VA_ARGS__) FQ_ROW_CASE(64, 6, __VA_ARGS__)  \
  FQ_ROW_CASE(64, 7, __VA_ARGS__) FQ_ROW_CASE(64, 8, __VA_ARGS__) FQ_ROW_CASE(64, 9, __VA_ARGS__)  \
  FQ_ROW_CASE(64, 10, __VA_ARGS__) FQ_ROW_CASE(64, 11, __VA_ARGS__) FQ_ROW_CASE(64, 12, __VA_ARGS__) \
  FQ_ROW_CASE(64, 13, __VA_ARGS__) FQ_ROW_CASE(64, 14, __VA_ARGS__) FQ_ROW_CASE(64, 15, __VA_ARGS__) \
  FQ_ROW_CASE(64, 16, __VA_ARGS__) { return hipErrorInvalidValue; }

hipError_t launch_rmsnorm_fwd(const void* x, const void* gamma, void* out, float* scale, float* rstd, int64_t M,
                              int n, float eps, int reuse_rstd, int quant, int round_scale, int kind,
                              hipStream_t stream) {
  if (M == 0) return hipSuccess;
  int nchunk;
  pick_row_shape(n, 64, nchunk);
  const int rows_per_wg = 1;
  // one wave per workgroup; at most 32 of them per CU, rows beyond that by striding
  int64_t wgs = M;
  if (wgs > 256 * 32) wgs = 256 * 32;
  const dim3 grid((unsigned)wgs);
#define FQ_LAUNCH_FWD(REUSE, QUANT, KINDV, ROUNDV)                                                          \
  FQ_FWD_SHAPES(hipLaunchKernelGGL((rmsnorm_fwd_kernel<kT, kNC, REUSE, QUANT, KINDV, ROUNDV>), grid,       \
                                   dim3(kT), 0, stream, (const uint16_t*)x, (const uint16_t*)gamma, out,   \
                                   scale, rstd, M, n, eps, rows_per_wg);)
  // quant: 0 = bf16 output, 1 = fp8 codes + scales, 2 = statistic only (its own kernel)
  if (quant == 2) {
    const dim3 sgrid((unsigned)((wgs + Policy::kRowstatWaves - 1) / Policy::kRowstatWaves)), sblock(64 * Policy::kRowstatWaves);
    const int by_xcd = rmsnorm_passes_by_xcd(M, n) && sgrid.x % 8 == 0;
    if (n <= 2048) hipLaunchKernelGGL(rowstat_kernel<4>, sgrid, sblock, 0, stream, (const uint16_t*)x, rstd, M, n, eps, by_xcd);
    else hipLaunchKernelGGL(rowstat_kernel<8>, sgrid, sblock, 0, stream, (const uint16_t*)x, rstd, M, n, eps, by_xcd);
  } else if (!quant) {
    if (reuse_rstd) { FQ_LAUNCH_FWD(true, 0, kE4M3, false) } else { FQ_LAUNCH_FWD(false, 0, kE4M3, false) }
  } else if (n > 2048) {
    // wide rows, quantising form: four waves per row (a wave per row needs up to ~230 registers)
    int64_t wg4 = M;
    if (wg4 > 256 * Policy::kRowQuantWideWgsPerCu) wg4 = 256 * Policy::kRowQuantWideWgsPerCu;
    const dim3 grid4((unsigned)wg4);
    const int nc4 = (n / 8 + 255) / 256;
#define FQ_LAUNCH_FWD4(NC, KINDV, ROUNDV)                                                                      \
  hipLaunchKernelGGL((rmsnorm_fwd_kernel<256, NC, false, 1, KINDV, ROUNDV>), grid4, dim3(256), 0, stream,       \
                     (const uint16_t*)x, (const uint16_t*)gamma, out, scale, rstd, M, n, eps, rows_per_wg)
#define FQ_LAUNCH_FWD4_NC(KINDV, ROUNDV) \
  if (nc4 == 2) { FQ_LAUNCH_FWD4(2, KINDV, ROUNDV); } else if (nc4 == 3) { FQ_LAUNCH_FWD4(3, KINDV, ROUNDV); } \
  else { FQ_LAUNCH_FWD4(4, KINDV, ROUNDV); }
    if (kind == kE5M2) {
      if (round_scale) { FQ_LAUNCH_FWD4_NC(kE5M2, true) } else { FQ_LAUNCH_FWD4_NC(kE5M2, false) }
    } else {
      if (round_scale) { FQ_LAUNCH_FWD4_NC(kE4M3, true) } else { FQ_LAUNCH_FWD4_NC(kE4M3, false) }
    }
#undef FQ_LAUNCH_FWD4_NC
#undef FQ_LAUNCH_FWD4
  } else if (kind == kE5M2) {
    if (round_scale) { FQ_LAUNCH_FWD(false, 1, kE5M2, true) } else { FQ_LAUNCH_FWD(false, 1, kE5M2, false) }
  } else {
    if (round_scale) { FQ_LAUNCH_FWD(false, 1, kE4M3, true) } else { FQ_LAUNCH_FWD(false, 1, kE4M3, false) }
  }
#undef FQ_LAUNCH_FWD
  return hipGetLastError();
}

bool rmsnorm_passes_by_xcd(int64_t M, int n) {
  return M % 1024 == 0 && M * n * 2 <= (int64_t)Policy::kRmsnormByXcdMaxBytes;
}

int64_t rmsnorm_bwd_partials(int64_t M) {
  // one partial row of dgamma per workgroup; 512 workgroups (two per CU) at most
  const int64_t min_rows = 8;
  int64_t p = (M + min_rows - 1) / min_rows;
  if (p > 512) p = 512;
  if (p < 1) p = 1;
  return p;
}

hipError_t launch_rmsnorm_bwd(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx,
                              float* dgamma, float* dg_part, int64_t n_partials, int64_t M, int n, float eps,
                              hipStream_t stream) {
  if (M == 0) {  // no rows: dgamma = 0, and no kernel touches dy, x, gamma or dx
    hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)((n + 63) / 64)), dim3(1024), 0, stream, dg_part, dgamma, 0, n);
    return hipGetLastError();
  }
  const int64_t P = n_partials;
  const int rows_per_wg = (int)((M + P - 1) / P);
  const dim3 grid((unsigned)P);
#define FQ_LAUNCH_BWD_BLOCK(NC, REUSE)                                                                      \
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<512, NC, REUSE>), grid, dim3(512), 0, stream, (const uint16_t*)dy, \
                     (const uint16_t*)x, (const uint16_t*)gamma, rstd, (uint16_t*)dx, dg_part, M, n, eps,   \
                     rows_per_wg)
#define FQ_LAUNCH_BWD_WAVE(NC, REUSE)                                                                       \
  hipLaunchKernelGGL((rmsnorm_bwd_wave_kernel<NC, REUSE>), grid, dim3(256), 0, stream, (const uint16_t*)dy, \
                     (const uint16_t*)x, (const uint16_t*)gamma, rstd, (uint16_t*)dx, dg_part, M, n, eps)
#define FQ_BWD_REUSE(LAUNCH, NC) \
  if (rstd) { LAUNCH(NC, true); } else { LAUNCH(NC, false); }
  if (n <= 2048) {  // one wave per row, n/512 chunks per lane
    const int wc = (n / 8 + 63) / 64;
    if (wc == 1) { FQ_BWD_REUSE(FQ_LAUNCH_BWD_WAVE, 1) }
    else if (wc == 2) { FQ_BWD_REUSE(FQ_LAUNCH_BWD_WAVE, 2) }
    else if (wc == 3) { FQ_BWD_REUSE(FQ_LAUNCH_BWD_WAVE, 3) }
    else { FQ_BWD_REUSE(FQ_LAUNCH_BWD_WAVE, 4) }
  } else if (n <= 4096) {  // 512 threads per row, one chunk each
    FQ_BWD_REUSE(FQ_LAUNCH_BWD_BLOCK, 1)
  } else {  // two chunks each
    FQ_BWD_REUSE(FQ_LAUNCH_BWD_BLOCK, 2)
  }
#undef FQ_BWD_REUSE
#undef FQ_LAUNCH_BWD_WAVE
#undef FQ_LAUNCH_BWD_BLOCK
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) return err;
  hipLaunchKernelGGL(colsum_kernel, dim3((unsigned)((n + 63) / 64)), dim3(1024), 0, stream, dg_part, dgamma, (int)P,
                     n);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// RMSNorm backward for callers that cannot allocate: the dgamma partial rows live
// in a fixed array in device memory instead of a caller-provided buffer.
// Every GPU the library runs on holds its own copy of the array (16 MiB) at its
// own address until the process ends; the address is looked up once per device,
// with that device current, and kernels only ever see the looked-up pointer.
// The kernels write every partial row they later read, so nothing is cleared
// between calls; two calls that overlap in time on one GPU share the array and race.
// ---------------------------------------------------------------------------
constexpr int64_t kStaticPartialRows = 512;    // the most rmsnorm_bwd_partials() returns
constexpr int64_t kStaticPartialWidth = 8192;  // the widest row the RMSNorm kernels accept
static __device__ __align__(256) float scratch[kStaticPartialRows * kStaticPartialWidth];

int64_t rmsnorm_bwd_static_scratch_bytes() { return (int64_t)sizeof(float) * kStaticPartialRows * kStaticPartialWidth; }

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_lock;
float* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the device that owns `device_ptr` (one of the call's tensors).
// That device has to be the current one: kernels are launched on the current device, and the
// symbol lookup answers for it.  A caller whose current device differs gets an error instead of
// another GPU's array address.
hipError_t static_scratch_ptr(const void* device_ptr, float** out) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess) return err;
  if (dev < 0 || dev >= kMaxDevices) return hipErrorInvalidDevice;
  if (device_ptr != nullptr) {
    hipPointerAttribute_t attr;
    err = hipPointerGetAttributes(&attr, device_ptr);
    if (err != hipSuccess) return err;
    if (attr.device != dev) return hipErrorInvalidDevice;
  }
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    err = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (err != hipSuccess) return err;
    if (p == nullptr) return hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = (float*)p;
  }
  *out = g_scratch_ptr[dev];
  return hipSuccess;
}
}  // namespace

hipError_t launch_rmsnorm_bwd_static(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx,
                                     float* dgamma, int64_t M, int n, float eps, hipStream_t stream) {
  const int64_t P = rmsnorm_bwd_partials(M);
  if (P > kStaticPartialRows || n > kStaticPartialWidth) return hipErrorInvalidValue;
  float* part = nullptr;
  const hipError_t err = static_scratch_ptr(dgamma, &part);
  if (err != hipSuccess) return err;
  return launch_rmsnorm_bwd(dy, x, gamma, rstd, dx, dgamma, part, P, M, n, eps, stream);
}

hipError_t launch_group_quant(const void* x, void* q, float* s, int64_t n_groups, int round_scale, int kind,
                              hipStream_t stream) {
  if (n_groups == 0) return hipSuccess;
  int64_t wgs = (n_groups + 15) / 16;  // 16 groups per workgroup pass
  if (wgs > 256 * 16) wgs = 256 * 16;
  const dim3 grid((unsigned)wgs), block(256);
#define FQ_GQ(KINDV, ROUNDV) \
  hipLaunchKernelGGL((group_quant_kernel<KINDV, ROUNDV>), grid, block, 0, stream, (const uint16_t*)x, (uint8_t*)q, s, n_groups)
  if (kind == kE5M2) { if (round_scale) FQ_GQ(kE5M2, true); else FQ_GQ(kE5M2, false); }
  else if (kind == kE5M2Max448) { if (round_scale) FQ_GQ(kE5M2Max448, true); else FQ_GQ(kE5M2Max448, false); }
  else { if (round_scale) FQ_GQ(kE4M3, true); else FQ_GQ(kE4M3, false); }
#undef FQ_GQ
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// bf16 SwiGLU without quantisation (linghe/utils/silu.py:98-210): one wave per
// row, lanes stride over the row in 16-byte chunks, four chunks in flight.
//   forward:  out = ((sigmoid(x1)*x1)*x2)[*w_row]                    -> bf16 [M, n]
//   backward: dx1 = h*sg + ((h*x1)*(1-sg))*sg, dx2 = g[*w]*(sg*x1)   -> bf16 [M, 2n]
//             dw_row = sum_c g*((sg*x1)*x2)   (weighted form only)
// in the order fp32 autograd evaluates them (the SwiGLU + quant kernels use the
// same expressions).
// ---------------------------------------------------------------------------
template <bool WEIGHTED>
__global__ __launch_bounds__(64) void swiglu_fwd_rows_kernel(const uint16_t* __restrict__ x, RowWeight weight,
                                                             uint16_t* __restrict__ out, int64_t M, int n) {
  const int lane = tid_x();
  const int chunks = n >> 3;
  for (int64_t row = wg_x(); row < M; row += n_wg_x()) {
    const uint16_t* p = x + row * 2 * (int64_t)n;
    float w = 1.0f;
    if constexpr (WEIGHTED) w = load_weight_uniform(weight, row);
    for (int c0 = 0; c0 < chunks; c0 += 256) {
      uint4 r1[4], r2[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        // No condition on loads or stores: beyond the end of the row a lane reads the row's last chunk
        // again and stores the same result to the same place again.  (With the stores behind per-chunk
        // branches the compiler waited for a step's stores before it issued the next step's loads.)
        const int c = c0 + u * 64 + lane;
        const int cc = c < chunks ? c : chunks - 1;
        r1[u] = ld16(p + cc * 8);
        r2[u] = ld16(p + n + cc * 8);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int c = c0 + u * 64 + lane;
        const int cc = c < chunks ? c : chunks - 1;
        float a[8], b[8], y[8];
        unpack8(r1[u], a);
        unpack8(r2[u], b);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          y[j] = (sigmoid_f32(a[j]) * a[j]) * b[j];
          if constexpr (WEIGHTED) y[j] = y[j] * w;
        }
        st16(out + row * n + cc * 8, pack8_bf16(y));
      }
    }
  }
}

template <bool WEIGHTED>
__global__ __launch_bounds__(64) void swiglu_bwd_rows_kernel(const uint16_t* __restrict__ gr,
                                                             const uint16_t* __restrict__ x, RowWeight weight,
                                                             uint16_t* __restrict__ dx, void* __restrict__ dw,
                                                             int64_t M, int n) {
  const int lane = tid_x();
  const int chunks = n >> 3;
  for (int64_t row = wg_x(); row < M; row += n_wg_x()) {
    const uint16_t* p = x + row * 2 * (int64_t)n;
    const uint16_t* gp = gr + row * (int64_t)n;
    uint16_t* o = dx + row * 2 * (int64_t)n;
    float w = 1.0f;
    if constexpr (WEIGHTED) w = load_weight_uniform(weight, row);
    float dws = 0.f;
    constexpr int kU = Policy::kSwigluBwdRowsUnroll;  // 16-byte chunks per lane, matrix and step
    for (int c0 = 0; c0 < chunks; c0 += 64 * kU) {
      uint4 r1[kU], r2[kU], rg[kU];
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        // no condition on loads or stores (see the forward kernel); a repeated chunk adds nothing to dw
        const int c = c0 + u * 64 + lane;
        const int cc = c < chunks ? c : chunks - 1;
        r1[u] = ld16(p + cc * 8);
        r2[u] = ld16(p + n + cc * 8);
        rg[u] = ld16(gp + cc * 8);
      }
#pragma unroll
      for (int u = 0; u < kU; ++u) {
        const int c = c0 + u * 64 + lane;
        const int cc = c < chunks ? c : chunks - 1;
        float a[8], b[8], go[8], d1[8], d2[8];
        unpack8(r1[u], a);
        unpack8(r2[u], b);
        unpack8(rg[u], go);
        float part = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float sg = sigmoid_f32(a[j]);
          const float sx = sg * a[j];
          float gw = go[j];
          if constexpr (WEIGHTED) {
            part += go[j] * (sx * b[j]);
            gw = go[j] * w;
          }
          const float h = gw * b[j];
          d2[j] = gw * sx;
          d1[j] = h * sg + ((h * a[j]) * (1.0f - sg)) * sg;
        }
        if constexpr (WEIGHTED) dws += c < chunks ? part : 0.f;
        st16(o + cc * 8, pack8_bf16(d1));
        st16(o + n + cc * 8, pack8_bf16(d2));
      }
    }
    if constexpr (WEIGHTED) {
      dws = wave_sum(dws);
      if (lane == 0) {
        if (weight.is_bf16) ((uint16_t*)dw)[row] = (uint16_t)(pack_bf16x2(dws, 0.f) & 0xffffu);
        else ((float*)dw)[row] = dws;
      }
    }
  }
}

hipError_t launch_swiglu_rows_fwd(const void* x, const void* weight, int weight_bf16, void* out, int64_t M, int n,
                                  hipStream_t stream) {
  if (M == 0) return hipSuccess;
  int64_t wgs = M < 256 * 32 ? M : 256 * 32;
  RowWeight w{weight, weight_bf16};
  if (weight) hipLaunchKernelGGL(swiglu_fwd_rows_kernel<true>, dim3((unsigned)wgs), dim3(64), 0, stream,
                                 (const uint16_t*)x, w, (uint16_t*)out, M, n);
  else hipLaunchKernelGGL(swiglu_fwd_rows_kernel<false>, dim3((unsigned)wgs), dim3(64), 0, stream,
                          (const uint16_t*)x, w, (uint16_t*)out, M, n);
  return hipGetLastError();
}

hipError_t launch_swiglu_rows_bwd(const void* g, const void* x, const void* weight, int weight_bf16, void* dx,
                                  void* dw, int64_t M, int n, hipStream_t stream) {
  if (M == 0) return hipSuccess;
  int64_t wgs = M < 256 * 32 ? M : 256 * 32;
  RowWeight w{weight, weight_bf16};
  if (weight) hipLaunchKernelGGL(swiglu_bwd_rows_kernel<true>, dim3((unsigned)wgs), dim3(64), 0, stream,
                                 (const uint16_t*)g, (const uint16_t*)x, w, (uint16_t*)dx, dw, M, n);
  else hipLaunchKernelGGL(swiglu_bwd_rows_kernel<false>, dim3((unsigned)wgs), dim3(64), 0, stream,
                          (const uint16_t*)g, (const uint16_t*)x, w, (uint16_t*)dx, dw, M, n);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// 128x128 block quant of a weight (linghe/quant/block.py:11-62): one scale per
// block, s[rb * (N/128) + cb]; one workgroup per block, 8 rows x 8 columns per
// thread as in the tile kernels, no transposed copy.
// ---------------------------------------------------------------------------
template <int KIND, bool ROUND>
__global__ __launch_bounds__(256) void block_quant_kernel(const uint16_t* __restrict__ x, uint8_t* __restrict__ q,
                                                          float* __restrict__ s, int N) {
  __shared__ float wmax[4];
  const int ncb = N / kGroup;
  const int rb = wg_x() / ncb, cb = wg_x() - rb * ncb;
  const int cg = tid_x() & 15, rg = tid_x() >> 4;
  const uint8_t* src = (const uint8_t*)(x + ((int64_t)rb * kGroup) * N + (int64_t)cb * kGroup);
  uint8_t* dst = q + ((int64_t)rb * kGroup) * N + (int64_t)cb * kGroup;
  const uint32_t off = (uint32_t)(rg * 8) * (uint32_t)N + (uint32_t)cg * 8u;  // in elements
  uint4 raw[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) raw[k] = ld16(src + 2u * (off + (uint32_t)k * (uint32_t)N));
  float m = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float a[8];
    unpack8(raw[k], a);
#pragma unroll
    for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(a[j]));
  }
  m = wave_max(m);
  if ((tid_x() & 63) == 0) wmax[tid_x() >> 6] = m;
  __syncthreads();
  m = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
  const float sc = make_scale<KIND, ROUND>(m);
  const Quantum<ROUND> d = make_quantum<ROUND>(sc);
  if (tid_x() == 0) s[(int64_t)rb * ncb + cb] = sc;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float a[8];
    unpack8(raw[k], a);
    const uint2 pk = quantize8<KIND, ROUND>(a, d);
    st8(dst + (off + (uint32_t)k * (uint32_t)N), pk);
  }
}

hipError_t launch_block_quant(const void* x, void* q, float* s, int64_t M, int N, int round_scale, int kind,
                              hipStream_t stream) {
  const int64_t blocks = (M / kGroup) * (N / kGroup);
  if (blocks == 0) return hipSuccess;
  const dim3 grid((unsigned)blocks), block(256);
#define FQ_BQ(KINDV, ROUNDV) \
  hipLaunchKernelGGL((block_quant_kernel<KINDV, ROUNDV>), grid, block, 0, stream, (const uint16_t*)x, (uint8_t*)q, s, N)
  if (kind == kE5M2) { if (round_scale) FQ_BQ(kE5M2, true); else FQ_BQ(kE5M2, false); }
  else { if (round_scale) FQ_BQ(kE4M3, true); else FQ_BQ(kE4M3, false); }
#undef FQ_BQ
  return hipGetLastError();
}

}  // namespace fq
