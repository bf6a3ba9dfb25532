// 128x128 tile quantiser shared by every "tile" kernel of the path:
// a workgroup owns one 128-row x 128-column tile of the (already computed, fp32)
// matrix to be quantised and emits, in one pass,
//   * row-wise 1x128 codes + one fp32 scale per row          (MODE 0 or 2)
//   * column-wise 128x1 codes, transposed through LDS, + one
//     fp32 scale per column                                   (MODE 1 or 2)
//
// Thread mapping (RPT = rows per thread, 8 -> 256 threads, 4 -> 512 threads):
//   cg = tid & 15   column group: columns cg*8 .. cg*8+7 (one 128-bit bf16 load)
//   rg = tid >> 4   row group:    rows    rg*RPT .. rg*RPT+RPT-1
// so the 16 lanes of one DPP row share a matrix row (row amax = DPP reduction),
// and a thread owns RPT consecutive rows of 8 columns (the transposed codes of
// one column are RPT consecutive bytes -> one LDS store).
#pragma once
#include "fq_device.hpp"

namespace fq {

template <int RPT>
struct TileShape {
  static_assert(RPT == 8 || RPT == 4, "rows per thread");
  static constexpr int kRowGroups = kGroup / RPT;
  static constexpr int kThreads = 16 * kRowGroups;
  static constexpr int kWaves = kThreads / 64;
  // LDS tile of transposed codes: one row of kPitch bytes per column, its 128 code bytes as eight
  // 16-byte chunks of which chunk k sits at position k ^ swizzle(column group).  With 4 rows per
  // thread the 4-byte column writes of a wave pair up column groups cg and cg + 8 on one bank; a
  // pitch of 144 bytes with the swizzle on cg >> 1, which spreads a wave's 64 writes over 64
  // distinct banks, was measured and is not used: more LDS instructions (the compiler no longer
  // pairs the writes), 10 % MORE conflict cycles in total (688128 against 622592 per dispatch at
  // 8192 x 2048) and the same kernel times within 1 % - most of the counted cycles are the
  // natural extra cycles of the 16-byte-per-lane reads, not the writes.
  static constexpr int kPitch = kGroup;
  __device__ static __forceinline__ int swizzle(int cg) { return cg & 7; }
};

// where the four outputs of one tile go (element offsets; see the layout
// formulas in linghe/utils/silu.py:248-276 and :507-554)
struct TileOut {
  uint8_t* q;       // row-wise codes:       q[q_off + i*q_ld + c]
  int64_t q_off;
  int64_t q_ld;
  float* s;         // row scales:           s[s_off + i]
  int64_t s_off;
  uint8_t* qt;      // transposed codes:     qt[t_off + c*t_ld + i]
  int64_t t_off;
  int64_t t_ld;
  float* st;        // column scales:        st[st_off + c]
  int64_t st_off;
  int rows_valid;   // rows i < rows_valid exist (1..128)
  // A PACKED partial tile: the workgroup covers 2^kc_shift neighbouring column blocks of a row
  // block with at most 128 >> kc_shift rows (see SubTile); the offsets above are those of the
  // first column block, the next ones lie s_cb / t_cb elements further (q and st: 128).
  int kc_shift;     // 0 (one column block, up to 128 rows), 1 or 2
  int n_sub;        // column blocks that exist (1 .. 1 << kc_shift)
  int64_t s_cb;     // distance between the row scales of neighbouring column blocks
  int64_t t_cb;     // distance between their transposed codes (128 * t_ld)
};

// Which part of a (possibly packed) tile a thread works on.  With kc_shift = k the row groups of
// the workgroup are split into 2^k sub-tiles of 128 >> k rows, one per column block; a sub-tile is
// a whole number of waves, so `sub` is the same in every lane of a wave.
template <int RPT>
struct SubTile {
  int sub;   // column block inside the workgroup's run (wave-uniform)
  int rgl;   // row group inside the sub-tile: rows rgl*RPT .. rgl*RPT+RPT-1
  int ws;    // wave inside the sub-tile
};
template <int RPT>
__device__ __forceinline__ SubTile<RPT> sub_tile(int kc_shift) {
  const int rg = tile_tid() >> 4;
  const int rgs = (kGroup / RPT) >> kc_shift;  // row groups per sub-tile
  SubTile<RPT> t;
  t.sub = __builtin_amdgcn_readfirstlane(rg / rgs);
  t.rgl = rg & (rgs - 1);
  t.ws = __builtin_amdgcn_readfirstlane((int)(tile_tid() >> 6) & ((rgs >> 2) - 1));
  return t;
}

// NV: value tiles quantised together by one workgroup (2 in the SwiGLU backward: dx1, dx2)
template <int RPT, int NV = 1>
struct alignas(16) TileShared {
  uint8_t t[NV][kGroup * TileShape<RPT>::kPitch];         // transposed codes, 16-byte chunks XOR-swizzled
  float colmax[NV][TileShape<RPT>::kWaves][kGroup];       // per-wave column amax
  float2 cdiv[NV][NV == 1 ? 4 : 1][kGroup];               // per column (and sub-tile of a packed tile) what the quantiser keeps per scale (Quantum)
  float2 rdiv[NV][kGroup];                                // per row    the same
};

// Column maxima of a wave.  Lane (r, cg) = (lane >> 4, lane & 15) holds cm[j], the
// maximum of column cg*8+j over its own rows; the four row groups r of the wave are
// combined with the gfx950 permlane swaps, two columns per swap:
//   permlane32_swap(a, b) -> {[a.lo, b.lo], [a.hi, b.hi]}: their maximum holds column a
//     reduced over lanes l, l^32 in the lower half and column b in the upper half;
//   permlane16_swap does the same with the odd/even 16-lane rows.
// 8 values -> 4 -> 2 registers with 6 swaps and 6 maxima.  On return lane (r, cg) holds
// the wave's maximum of column cg*8 + kColOfRow[r] in lo and of column
// cg*8 + 4 + kColOfRow[r] in hi, kColOfRow = {0, 2, 1, 3}.
__device__ __forceinline__ float swap32_max(float a, float b) {
  auto t = __builtin_amdgcn_permlane32_swap(as_u32(a), as_u32(b), false, false);
  return fmaxf(as_f32(t[0]), as_f32(t[1]));
}
__device__ __forceinline__ float swap16_max(float a, float b) {
  auto t = __builtin_amdgcn_permlane16_swap(as_u32(a), as_u32(b), false, false);
  return fmaxf(as_f32(t[0]), as_f32(t[1]));
}
// every lane ends with the maximum over the four lanes l, l^16, l^32, l^48
__device__ __forceinline__ float max_across_rows(float v) {
  const float t = swap32_max(v, v);
  return swap16_max(t, t);
}
__device__ __forceinline__ void wave_column_max(const float (&cm)[8], float& lo, float& hi) {
  const float r0 = swap32_max(cm[0], cm[1]), r1 = swap32_max(cm[2], cm[3]);
  const float r2 = swap32_max(cm[4], cm[5]), r3 = swap32_max(cm[6], cm[7]);
  lo = swap16_max(r0, r1);
  hi = swap16_max(r2, r3);
}

// 16 / 8 / 4 / 2 bytes stored at ANY byte address: gfx950 runs with unaligned
// vector memory access enabled, so one store instruction serves whatever the
// alignment (per-expert transposed rows are packed back to back with a stride of
// count_e bytes and start anywhere)
typedef uint32_t u32x2_any __attribute__((ext_vector_type(2), aligned(1)));
typedef uint32_t u32_any __attribute__((aligned(1)));
typedef uint16_t u16_any __attribute__((aligned(1)));
// STREAM: with the non-temporal hint (fq_device.hpp)
typedef uint32_t u32x4_any __attribute__((ext_vector_type(4), aligned(1)));
template <bool STREAM>
__device__ __forceinline__ void store16_any(uint8_t* dst, const uint4& v) {
  FQ_GLOBAL u32x4_any* g = (FQ_GLOBAL u32x4_any*)dst;
  const u32x4_any t = {v.x, v.y, v.z, v.w};
  if constexpr (STREAM) __builtin_nontemporal_store(t, g);
  else *g = t;
}

// dword k (k = 0..3, lane-variable) of a 16-byte chunk held in four registers
// (by value: an aggregate whose address is taken here ends up in memory)
__device__ __forceinline__ uint32_t pick_dword(uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, int k) {
  const uint32_t lo = (k & 1) ? d1 : d0;
  const uint32_t hi = (k & 1) ? d3 : d2;
  return (k & 2) ? hi : lo;
}

// Write the first `len` bytes of one transposed row from LDS (`lds_row`: 128 bytes
// as eight 16-byte chunks, chunk k stored at position k ^ swz) to `dst_row`.
// Called by the 8 threads ch = 0..7 that share the row: thread ch owns source
// bytes [16 ch, 16 ch + 16); a chunk cut by the end of the row leaves as at most
// one 8-, 4-, 2- and 1-byte store.
// In a packed tile the 128 bytes of an LDS row hold the rows of several sub-tiles one after
// the other: the thread reads chunk `ch` of the LDS row and writes it as chunk `chd` of its
// sub-tile's transposed row (ch == chd in an unpacked tile).
template <bool STREAM>
__device__ __forceinline__ void store_t_row(const uint8_t* lds_row, int swz, uint8_t* dst_row, int len, int ch,
                                            int chd) {
  const int rem = len - 16 * chd;
  if (rem <= 0) return;
  const uint4 v = *(const uint4*)(lds_row + ((ch ^ swz) * 16));
  uint8_t* dst = dst_row + 16 * chd;
  if (rem >= 16) {
    store16_any<STREAM>(dst, v);
    return;
  }
  const uint32_t d0 = v.x, d1 = v.y, d2 = v.z, d3 = v.w;
  int p = 0;
  if (rem & 8) { *(FQ_GLOBAL u32x2_any*)dst = u32x2_any{d0, d1}; p = 8; }
  if (rem & 4) { *(FQ_GLOBAL u32_any*)(dst + p) = pick_dword(d0, d1, d2, d3, p >> 2); p += 4; }
  if (rem & 2) { *(FQ_GLOBAL u16_any*)(dst + p) = (uint16_t)(pick_dword(d0, d1, d2, d3, p >> 2) >> (8 * (p & 3))); p += 2; }
  if (rem & 1) *(FQ_GLOBAL uint8_t*)(dst + p) = (uint8_t)(pick_dword(d0, d1, d2, d3, p >> 2) >> (8 * (p & 3)));
}

// Quantise NV tiles held in registers (v[t][s][j] = element (rg*RPT+s, cg*8+j) of tile t;
// rows >= rows_valid must hold 0; the tiles share rows_valid).  All threads of the
// workgroup must call it.  The tiles go through the column stage together: one set
// of barriers for all of them, and the NV*128 column scales are computed by as many
// threads at once.
// FULL: the tiles have all 128 rows, so no load or store needs a mask.
// TAIL_SYNC: end with a barrier (needed only when the shared memory is used again).
template <int KIND, bool ROUND, int MODE, int RPT, bool FULL, int NT, bool LEAN, int NV, bool TAIL_SYNC>
__device__ __forceinline__ void quantize_tiles_impl(const float (&v)[NV][RPT][8], const TileOut (&o)[NV],
                                                    TileShared<RPT, NV>& sh) {
  using Shape = TileShape<RPT>;
  static_assert(NV * kGroup <= Shape::kThreads, "one thread per column scale");
  const int tid = tile_tid();
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int cg = tid & 15;
  const int rg = tid >> 4;
  const int rows_valid = o[0].rows_valid;
  // packed partial tiles: this wave's column block (sub) and its rows inside it; a full tile
  // is one sub-tile and the compiler sees the constants
  const int kc_shift = (FULL || NV > 1) ? 0 : o[0].kc_shift;  // several value tiles are never packed
  SubTile<RPT> sl;
  if constexpr (FULL) { sl.sub = 0; sl.rgl = rg; sl.ws = wave; }
  else sl = sub_tile<RPT>(kc_shift);
  const int rgl = sl.rgl;

  // A wave owns 4*RPT consecutive rows.  In a partial tile the waves whose rows all
  // lie beyond the last stored row (or whose column block does not exist) have nothing
  // to quantise: their values are zero, their row-wise outputs do not exist and their
  // bytes of the transposed tile are never stored, so they only keep the barriers company.
  const bool live = FULL || (sl.ws * (4 * RPT) < rows_valid && sl.sub < o[0].n_sub);

  // LEAN: the four output bases, which are the same in every lane, are moved to scalar
  // registers, so that each store is "scalar base + 32-bit lane offset" (a tile spans
  // at most 128 rows of at most 2^24 bytes) without 64-bit vector address arithmetic,
  // and the column maxima take the paired reduction: 10 % fewer vector instructions,
  // 3-9 % less time in every tile kernel but the plain blockwise quantiser.
  uint8_t* q_base[NV];
  uint8_t* t_base[NV];
  float* s_base[NV];
  float* st_base[NV];
  uint32_t q_ld = (uint32_t)o[0].q_ld, t_ld = (uint32_t)o[0].t_ld;
#pragma unroll
  for (int t = 0; t < NV; ++t) {
    q_base[t] = o[t].q + o[t].q_off;
    t_base[t] = o[t].qt + o[t].t_off;
    s_base[t] = o[t].s + o[t].s_off;
    st_base[t] = o[t].st + o[t].st_off;
    if constexpr (!FULL) {  // this wave's column block of a packed tile
      q_base[t] += sl.sub * kGroup;
      s_base[t] += sl.sub * o[t].s_cb;
      // t_base / st_base stay those of the first column block: the threads that store the
      // transposed rows and the column scales are not the ones that computed them
    }
    if constexpr (LEAN) {
      q_base[t] = (uint8_t*)uniform64((int64_t)q_base[t]);
      t_base[t] = (uint8_t*)uniform64((int64_t)t_base[t]);
      s_base[t] = (float*)uniform64((int64_t)s_base[t]);
      st_base[t] = (float*)uniform64((int64_t)st_base[t]);
    }
  }
  if constexpr (LEAN) {
    q_ld = (uint32_t)uniform32((int)q_ld);
    t_ld = (uint32_t)uniform32((int)t_ld);
  }

  // ------------------------------------------------------------- row-wise
  if ((MODE == 0 || MODE == 2) && live) {
    // every lane of a 16-lane row gets the amax of its RPT rows; lane cg < RPT then
    // turns ONE of them (row rg*RPT+cg) into its scale and divisor, stores the scale,
    // and hands the divisor to the other lanes through LDS.  The rows of a wave are
    // written and read by that wave only, so no barrier is needed.
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      float mine = 0.f;
#pragma unroll
      for (int s = 0; s < RPT; ++s) {
        float m = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) m = fmaxf(m, fabsf(v[t][s][j]));
        m = row16_max(m);
        if (cg == s) mine = m;
      }
      if (cg < RPT) {
        const float sc = make_scale<KIND, ROUND>(mine);
        const Quantum<ROUND> d = make_quantum<ROUND>(sc);
        const int i = rgl * RPT + cg;
        sh.rdiv[t][rg * RPT + cg] = make_float2(d.a, d.b);
        if (FULL || i < rows_valid) store_f32(s_base[t] + (uint32_t)i, sc);  // a wave writes 4*RPT consecutive floats
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int t = 0; t < NV; ++t) {
#pragma unroll
      for (int s = 0; s < RPT; ++s) {
        const float2 sr = sh.rdiv[t][rg * RPT + s];
        const Quantum<ROUND> d{sr.x, sr.y};
        const uint2 pk = quantize8<KIND, ROUND>(v[t][s], d);
        const int i = rgl * RPT + s;
        if (FULL || i < rows_valid) store8<(NT & 2) != 0>(q_base[t] + ((uint32_t)i * q_ld + (uint32_t)cg * 8u), pk);
      }
    }
  }

  // ---------------------------------------------------------- column-wise
  if constexpr (MODE == 1 || MODE == 2) {
#pragma unroll
    for (int t = 0; t < NV; ++t) {
      float cm[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) cm[j] = 0.f;
      if constexpr (LEAN) {
        float cm_lo = 0.f, cm_hi = 0.f;
        if (live) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            float m = 0.f;
#pragma unroll
            for (int s = 0; s < RPT; ++s) m = fmaxf(m, fabsf(v[t][s][j]));
            cm[j] = m;
          }
          wave_column_max(cm, cm_lo, cm_hi);
        }
        const int r = lane >> 4;
        float* dst = &sh.colmax[t][wave][cg * 8 + (((r & 1) << 1) | (r >> 1))];
        dst[0] = cm_lo;
        dst[4] = cm_hi;
      } else {
        if (live) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            float m = 0.f;
#pragma unroll
            for (int s = 0; s < RPT; ++s) m = fmaxf(m, fabsf(v[t][s][j]));
            cm[j] = max_across_rows(m);
          }
        }
        if (lane < 16) {
          float4* dst = (float4*)&sh.colmax[t][wave][cg * 8];
          dst[0] = make_float4(cm[0], cm[1], cm[2], cm[3]);
          dst[1] = make_float4(cm[4], cm[5], cm[6], cm[7]);
        }
      }
    }
    __syncthreads();
    if constexpr (FULL || NV > 1) {
      if (tid < NV * kGroup) {  // thread (t, c): the scale of column c of tile t
        const int t = tid / kGroup, c = tid % kGroup;
        float m = sh.colmax[t][0][c];
#pragma unroll
        for (int w = 1; w < Shape::kWaves; ++w) m = fmaxf(m, sh.colmax[t][w][c]);
        const float sc = make_scale<KIND, ROUND>(m);
        const Quantum<ROUND> d = make_quantum<ROUND>(sc);
        sh.cdiv[t][0][c] = make_float2(d.a, d.b);
        float* dst = st_base[0];
#pragma unroll
        for (int u = 1; u < NV; ++u) dst = (t == u) ? st_base[u] : dst;
        store_f32(dst + (uint32_t)c, sc);
      }
    } else {
      // thread (sb, c): the scale of column c of sub-tile sb, over that sub-tile's waves
      const int wps = Shape::kWaves >> kc_shift;
      for (int idx = tid; idx < o[0].n_sub * kGroup; idx += Shape::kThreads) {
        const int sb = idx / kGroup, c = idx % kGroup;
        float m = 0.f;
        for (int w = 0; w < wps; ++w) m = fmaxf(m, sh.colmax[0][sb * wps + w][c]);
        const float sc = make_scale<KIND, ROUND>(m);
        const Quantum<ROUND> d = make_quantum<ROUND>(sc);
        sh.cdiv[0][sb][c] = make_float2(d.a, d.b);
        store_f32(st_base[0] + (uint32_t)(sb * kGroup + c), sc);
      }
    }
    __syncthreads();
    if (live) {
#pragma unroll
      for (int t = 0; t < NV; ++t) {
        const float2* cdp = &sh.cdiv[t][FULL ? 0 : sl.sub][cg * 8];
        // transposed codes -> LDS; byte (c, i) lives at c*128 + ((i>>4) ^ ((c>>3)&7))*16 + (i&15)
        const int i0 = rg * RPT;
        const int chunk = (i0 >> 4) ^ Shape::swizzle(cg);
        uint8_t* base = sh.t[t] + chunk * 16 + (i0 & 15);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float2 c2 = cdp[j];
          const Quantum<ROUND> d{c2.x, c2.y};
          uint8_t* p = base + (cg * 8 + j) * Shape::kPitch;
          if constexpr (RPT == 8) {
            uint2 pk;
            pk.x = quantize4<KIND, ROUND>(v[t][0][j], v[t][1][j], v[t][2][j], v[t][3][j], d);
            pk.y = quantize4<KIND, ROUND>(v[t][4][j], v[t][5][j], v[t][6][j], v[t][7][j], d);
            *(uint2*)p = pk;
          } else {
            *(uint32_t*)p = quantize4<KIND, ROUND>(v[t][0][j], v[t][1][j], v[t][2][j], v[t][3][j], d);
          }
        }
      }
    }
    __syncthreads();
    // each transposed row (one column, 128 row-bytes) leaves as 8 x 16 bytes
    constexpr int kRowsPerPass = Shape::kThreads / 8;
    const int ch = tid & 7;
#pragma unroll
    for (int t = 0; t < NV; ++t) {
#pragma unroll
      for (int k = 0; k < kGroup / kRowsPerPass; ++k) {
        const int c = (tid >> 3) + k * kRowsPerPass;
        if constexpr (FULL) {
          const uint4 val = *(const uint4*)(sh.t[t] + c * Shape::kPitch + ((ch ^ Shape::swizzle(c >> 3)) * 16));
          store16_any<(NT & 1) != 0>(t_base[t] + ((uint32_t)c * t_ld + (uint32_t)ch * 16u), val);
        } else {
          // LDS row c holds, one after the other, the rows of column c of every sub-tile
          const int cps = 8 >> kc_shift;  // 16-byte chunks per sub-tile
          const int sb = ch / cps;
          const int len = sb < o[t].n_sub ? rows_valid : 0;
          store_t_row<(NT & 1) != 0>(sh.t[t] + c * Shape::kPitch, Shape::swizzle(c >> 3),
                                     t_base[t] + ((int64_t)sb * o[t].t_cb + (int64_t)((uint32_t)c * t_ld)), len, ch,
                                     ch & (cps - 1));
        }
      }
    }
    if constexpr (TAIL_SYNC) __syncthreads();  // LDS is reused by a following call
  }
}

// NT: bit 0 = transposed codes, bit 1 = row-wise codes leave with the non-temporal hint
// ALL_FULL: the launch has no partial tile (single matrix, M a multiple of 128): only the
// mask-free path is compiled.  The ragged path costs registers the full one does not need
// (SwiGLU forward: 77 against 62, i.e. three against four workgroups per CU).
template <int KIND, bool ROUND, int MODE, int RPT, int NT = 0, bool LEAN = true, int NV = 1, bool TAIL_SYNC = false,
          bool ALL_FULL = false>
__device__ __forceinline__ void quantize_tiles(const float (&v)[NV][RPT][8], const TileOut (&o)[NV],
                                               TileShared<RPT, NV>& sh) {
  if constexpr (ALL_FULL) {
    quantize_tiles_impl<KIND, ROUND, MODE, RPT, true, NT, LEAN, NV, TAIL_SYNC>(v, o, sh);
  } else {
    // workgroup-uniform choice of the mask-free path
    const bool full = o[0].rows_valid == kGroup;
    if (full) quantize_tiles_impl<KIND, ROUND, MODE, RPT, true, NT, LEAN, NV, TAIL_SYNC>(v, o, sh);
    else quantize_tiles_impl<KIND, ROUND, MODE, RPT, false, NT, LEAN, NV, TAIL_SYNC>(v, o, sh);
  }
}

// one tile
template <int KIND, bool ROUND, int MODE, int RPT, int NT = 0, bool LEAN = true, bool ALL_FULL = false>
__device__ __forceinline__ void quantize_tile(const float (&v)[RPT][8], const TileOut& o, TileShared<RPT>& sh) {
  const float (&vs)[1][RPT][8] = reinterpret_cast<const float (&)[1][RPT][8]>(v);
  const TileOut (&os)[1] = reinterpret_cast<const TileOut (&)[1]>(o);
  quantize_tiles<KIND, ROUND, MODE, RPT, NT, LEAN, 1, false, ALL_FULL>(vs, os, sh);
}

// ---------------------------------------------------------------------------
// per-expert tile lookup for the batched forms
// ---------------------------------------------------------------------------
struct ExpertTile {
  int expert;
  int count;            // rows of this expert
  int pcount;           // rows of its region in the outputs: count rounded up to a multiple of `pad`
  int rb;               // 128-row block inside the expert
  int cb;               // first 128-column block of the workgroup
  int kc_shift;         // the workgroup covers 1 << kc_shift column blocks (packed partial tile), 0 = one
  int64_t row_start;    // first global row of the expert's region (sum of the pcount before it)
  int64_t tblock_start; // sum over previous experts of ceil(count/128)
};

__device__ __forceinline__ int load_count(const void* counts, int is_i64, int e) {
  return is_i64 ? (int)((const long long*)counts)[e] : ((const int*)counts)[e];
}

// inclusive prefix sum over the 64 lanes of a wave with DPP row shifts and the two
// row broadcasts (no LDS traffic, ~6 dependent VALU steps)
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xf, 0xf, true);   // row_shr:1
  v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xf, 0xf, true);   // row_shr:2
  v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xf, 0xf, true);   // row_shr:4
  v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xf, 0xf, true);   // row_shr:8
  v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xa, 0xf, false);  // row_bcast:15 into rows 1, 3
  v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xc, 0xf, false);  // row_bcast:31 into rows 2, 3
  return v;
}

// How many neighbouring column blocks one workgroup takes in the LAST row block of an expert
// whose (padded) count leaves `last` rows there: a block of at most 64 (32) rows leaves half
// (three quarters) of a 128-row workgroup without rows, so the idle waves take the next column
// block(s) of the same rows instead: 1 << shift column blocks of 128 >> shift rows each.
// Column maxima stay per column, row maxima per row and column block: nothing else changes.
__device__ __forceinline__ int pack_shift(int last_rows) { return last_rows <= 32 ? 2 : last_rows <= 64 ? 1 : 0; }

// the 16-byte-chunk bookkeeping of an expert with `c` rows: padded rows, 128-row blocks, pack shift
// of the last block and workgroups
struct ExpertShape {
  int pc, nb, shift, nw;
};
__device__ __forceinline__ ExpertShape expert_shape(int c, int ncb, int pad) {
  ExpertShape e;
  e.pc = (c + pad - 1) & -pad;  // pad is a power of two (1 or 16)
  e.nb = (c + kGroup - 1) / kGroup;
  e.shift = pack_shift(e.pc - (e.nb - 1) * kGroup);
  e.nw = e.nb > 0 ? (e.nb - 1) * ncb + ((ncb + (1 << e.shift) - 1) >> e.shift) : 0;
  return e;
}

constexpr int kLookupSteps = 16;  // 64 experts per step: the counts of up to 1024 experts are fetched together
// No condition on the loads and one code path for both count types: a lane beyond the last expert
// fetches the last expert's count (the caller takes it as 0), an int64 count is read as its low half
// (little endian; a count is a number of rows and fits 31 bits).
__device__ __forceinline__ void load_counts(const void* counts, int is_i64, int n_experts, int base0, int steps,
                                            int (&cs)[kLookupSteps]) {
  const int lane = tile_tid() & 63;
  const int shift = is_i64 ? 3 : 2;
  const uint8_t* base = (const uint8_t*)counts;
#pragma unroll
  for (int k = 0; k < kLookupSteps; ++k) {
    cs[k] = 0;
    if (k < steps) {
      const int e = base0 + k * 64 + lane;
      cs[k] = *(const int*)(base + ((int64_t)(e < n_experts ? e : n_experts - 1) << shift));  // masked by the caller
    }
  }
}

// Which tile does workgroup `wg` of a per-expert launch own?  Workgroups are numbered expert
// after expert; an expert with nbk = ceil(count/128) row blocks takes (nbk - 1) * ncb workgroups
// for its full row blocks (row block after row block, ncb column blocks each) and
// ceil(ncb / kc) for its last one, kc = 1 << pack_shift(rows of the last block).  Computed from
// the device-side counts by a prefix scan that EVERY WAVE runs for itself, 64 experts per step
// with the loads of up to sixteen steps in flight together: no LDS, no barrier, and every
// thread of the workgroup ends with the same answer.  (A workgroup-wide scan with three
// barriers cost 13 % of the batched SwiGLU forward, one wave scanning for the others 6 %.)
// A workgroup beyond the last tile (the launch is sized for one workgroup per 128 x 128 tile,
// packing needs fewer) or counts that disagree with the host's yield expert = -1.
// `wg` is the tile's number in that order; which workgroup takes which number is the caller's
// choice (resolve_tile: grid order, or runs of neighbouring row blocks per XCD).  Numbering the
// tiles so that every XCD works on one contiguous eighth of the REAL tiles needs their number
// first, one more pass over the counts, and measured slower: 89.3 against 87.8 us for the
// per-expert SwiGLU backward at 65536 x 1024 with 256 experts, 59 against 51 us for
// gather+pad+quant.
// pad > 1: every expert's region starts at a multiple of pad rows (the reference's
// permute-and-pad layout, pad = 16); 128 is a multiple of pad, so the number of
// 128-row blocks of an expert does not change.
__device__ __forceinline__ ExpertTile find_expert_tile(const void* counts, int is_i64, int n_experts, int wg, int ncb,
                                                       int pad = 1) {
  ExpertTile t;
  t.expert = -1;
  t.count = 0;
  t.pcount = 0;
  t.rb = 0;
  t.cb = 0;
  t.kc_shift = 0;
  t.row_start = 0;
  t.tblock_start = 0;
  int run_rows = 0, run_blocks = 0, run_wgs = 0;
  constexpr int kSteps = kLookupSteps;
  int cs[kSteps];
  // one chunk of up to 1024 experts whose counts sit in cs: true when the tile was found
  auto scan_chunk = [&](int base0, int steps) -> bool {
#pragma unroll
    for (int k = 0; k < kSteps; ++k) {
      if (k < steps) {
        const int base = base0 + k * 64;
        const int c = base + (int)(tile_tid() & 63) < n_experts ? cs[k] : 0;
        const ExpertShape es = expert_shape(c, ncb, pad);
        const int pc = es.pc, nb = es.nb, shift = es.shift, nw = es.nw;
        const int rows = wave_inclusive_scan(pc);
        const int blocks = wave_inclusive_scan(nb);
        const int wgs = wave_inclusive_scan(nw);
        const int excl_wgs = run_wgs + wgs - nw;
        const bool hit = nw > 0 && wg >= excl_wgs && wg < excl_wgs + nw;
        const unsigned long long mask = __builtin_amdgcn_ballot_w64(hit);
        if (mask != 0) {
          const int src = __builtin_ctzll(mask);
          t.expert = base + src;
          t.count = __builtin_amdgcn_readlane(c, src);
          t.pcount = __builtin_amdgcn_readlane(pc, src);
          t.tblock_start = run_blocks + __builtin_amdgcn_readlane(blocks - nb, src);
          t.row_start = (int64_t)(run_rows + __builtin_amdgcn_readlane(rows - pc, src));
          const int local = wg - __builtin_amdgcn_readlane(excl_wgs, src);
          const int nbe = __builtin_amdgcn_readlane(nb, src);
          const int full = (nbe - 1) * ncb;  // workgroups of the expert's full row blocks
          if (local < full) {
            t.rb = local / ncb;
            t.cb = local - t.rb * ncb;
          } else {
            t.rb = nbe - 1;
            t.kc_shift = __builtin_amdgcn_readlane(shift, src);
            t.cb = (local - full) << t.kc_shift;
          }
          return true;
        }
        run_rows += __builtin_amdgcn_readlane(rows, 63);
        run_blocks += __builtin_amdgcn_readlane(blocks, 63);
        run_wgs += __builtin_amdgcn_readlane(wgs, 63);
      }
    }
    return false;
  };
  for (int base0 = 0; base0 < n_experts; base0 += 64 * kSteps) {
    const int left = n_experts - base0;
    const int steps = left >= 64 * kSteps ? kSteps : (left + 63) / 64;  // wave-uniform
    load_counts(counts, is_i64, n_experts, base0, steps, cs);
    if (scan_chunk(base0, steps)) return t;
  }
  return t;
}

}  // namespace fq
