// Where a 128x128 tile of a launch lives: its rows, its column block and the
// offsets of its four outputs, for the single-matrix and the per-expert forms.
#pragma once
#include "fq_tile.hpp"

namespace fq {

// ---------------------------------------------------------------------------
// tile geometry
// ---------------------------------------------------------------------------
struct TileGeom {
  int64_t row0;      // first global row of the tile
  int rows_valid;    // rows that exist in the input (and in the outputs unless padded)
  int rows_store;    // rows written to the outputs (>= rows_valid; the extra ones hold zeros)
  int cb;            // (first) 128-column block of the input
  int kc_shift;      // packed partial tile: 1 << kc_shift column blocks of at most 128 >> kc_shift rows
  int n_sub;         // of which exist (the run may end at the matrix edge)
  int64_t s_base, s_stride;
  int64_t t_base, t_stride;
  int64_t st_row;
  int expert;        // per-expert forms: the expert the tile belongs to
  bool valid;
};

struct BatchArgs {
  const void* counts;  // device, int32 or int64, [n_experts]
  int counts_i64;
  int n_experts;
  int pad;             // 0/1: experts packed back to back; 16: each expert's region padded to 16 rows
  const void* plan;    // device, PlanEntry per 128-row block (expert_plan_kernel), or NULL: scan the counts
  int plan_unpacked;   // records of row blocks that are worked on unpacked,
  int plan_packed2;    // of last blocks of 33..64 rows, and (behind them) of
  int plan_packed4;    // last blocks of at most 32 rows: the table's three sections, counted by the host
  int xcd_rows;        // > 0: every XCD works on runs of so many row blocks (xcd_runs)
  int plan_packed_first;  // order of a planned launch: the packed tiles before (1) or behind (0) the others
};

// What a workgroup of a per-expert launch needs to know about its 128-row block, written once per
// set of counts by expert_plan_kernel and read with one 16-byte load through the constant path
// instead of the prefix scan over all counts (which puts a dependent vector load and three wave
// scans in front of every workgroup's first tile load).  Three sections, each in expert order: the row blocks that are worked on
// unpacked (all but an expert's last one, and last ones of more than 64 rows), the last blocks of
// 33..64 rows (two column blocks to a workgroup), the last blocks of at most 32 rows (four).  The
// host knows the sizes of the sections from its copy of the counts, sizes the launch for exactly
// the workgroups that have a tile, and passes the sizes as kernel arguments: a workgroup finds its
// section and its record from its number alone.
// Records are small because they are read cold: every line of the table that a workgroup is the
// first of its XCD to touch costs it a trip to memory before its first tile load can leave.
struct PlanEntry {
  uint32_t row0;   // first global row of the row block (in the outputs: regions padded when BatchArgs::pad says so)
  int rb;          // row block inside the expert
  int count;       // rows of the expert
  uint32_t where;  // kind << 30 | row block in expert order over all experts (row of the transposed scales)
};
// behind the records: one int per record, the expert it belongs to (read only by the kernel that
// needs it, gather + pad + quant for its probabilities)
constexpr uint32_t kPlanEmpty = 0, kPlanUnpacked = 1, kPlanPacked2 = 2, kPlanPacked4 = 3;  // kinds
static_assert(sizeof(PlanEntry) == 16, "16-byte records");

// workgroups of a planned launch over ncb column blocks
__host__ __device__ inline int64_t plan_workgroups(int64_t unpacked, int64_t packed2, int64_t packed4, int ncb) {
  return unpacked * ncb + packed2 * ((ncb + 1) >> 1) + packed4 * ((ncb + 3) >> 2);
}

// Workgroup i runs on XCD i % 8, each with an L2 of its own.  Neighbouring row blocks of an expert
// share lines of the transposed outputs (a column's 128-byte run starts at any byte offset), which
// one L2 merges and two write out twice as partial lines.  This renumbering hands every XCD runs
// of `chunk` consecutive tiles (a few row blocks with all their column blocks) instead of every
// eighth tile, in rounds of 8 * chunk tiles so that the XCDs stay in step; the tiles behind the
// last full round keep their numbers.
__device__ __forceinline__ int xcd_runs(int id, int total, int chunk) {
  const int round_tiles = 8 * chunk;
  if (id < (total / round_tiles) * round_tiles) {
    const int xcd = id & 7, pos = id >> 3;
    const int round = pos / chunk;
    return (round * 8 + xcd) * chunk + (pos - round * chunk);
  }
  return id;
}

// out_w: width of the quantised matrix the tile belongs to (n, or 2n for the
// backward's dx1|dx2)
// remap: workgroup i runs on XCD i % 8; 1 = give every XCD one contiguous eighth of the
// tiles instead of every eighth tile (single-matrix kernels only).  Which order of the tiles the memory system likes
// better depends on the kernel and the shape (measured: the RMSNorm tile kernel 4-18 %
// faster with it at 16384 x 7168 and slower below ~2000 tiles or with narrow rows, the
// per-expert SwiGLU backward 5 % faster; gather+pad+quant 18 % slower, the blockwise
// quantisers 5-9 %, the forward SwiGLU kernels 2-4 %), so the caller decides.
template <bool BATCHED>
__device__ __forceinline__ TileGeom resolve_tile(int64_t M, int ncb, int64_t out_w, const BatchArgs& b,
                                                 int remap = 0) {
  TileGeom g;
  int id = wg_x();
  if (remap == 1) {  // workgroup-uniform
    const int G = (int)n_wg_x();
    const int per = (G + 7) >> 3;
    const int xcd = id & 7, slot = id >> 3;
    // the first (G % 8, or 8) XCDs hold `per` tiles, the others one fewer
    const int full = (G & 7) ? (G & 7) : 8;
    id = xcd < full ? xcd * per + slot : full * per + (xcd - full) * (per - 1) + slot;
  }
  g.kc_shift = 0;
  g.n_sub = 1;
  if constexpr (!BATCHED) {
    const int rbk = id / ncb;
    g.cb = id - rbk * ncb;
    g.row0 = (int64_t)rbk * kGroup;
    const int64_t left = M - g.row0;
    g.rows_valid = left < kGroup ? (int)left : kGroup;
    g.rows_store = g.rows_valid;
    g.s_base = g.row0;
    g.s_stride = M;
    g.t_base = g.row0;
    g.t_stride = M;
    g.st_row = rbk;
    g.expert = 0;
    g.valid = left > 0;
  } else if (b.plan != nullptr) {  // workgroup-uniform
    typedef const __attribute__((address_space(4))) uint32_t* const_u32;
    const int c1 = (ncb + 1) >> 1, c2 = (ncb + 3) >> 2;
    // Order of the launch: the packed tiles, which move few bytes for the time they take, before or
    // behind the unpacked row blocks (those in expert order: neighbouring row blocks of an expert
    // share lines of the transposed outputs, and a strided walk over them measured 20 % slower).
    // Which end is better differs by kernel, by about 1 us either way at 65536 rows in 256 experts.
    const int n1 = b.plan_packed2 * c1, n2 = b.plan_packed4 * c2;
    int idx, x;
    uint32_t kind = kPlanUnpacked;
    if (!b.plan_packed_first) {
      const int n0 = b.plan_unpacked * ncb;
      id = id < n0 ? id + n1 + n2 : id - n0;
    }
    if (id < n1) {
      const int q = id / c1;
      idx = b.plan_unpacked + q;
      x = id - q * c1;
      kind = kPlanPacked2;
    } else if (id < n1 + n2) {
      const int r = id - n1, q = r / c2;
      idx = b.plan_unpacked + b.plan_packed2 + q;
      x = r - q * c2;
      kind = kPlanPacked4;
    } else {
      int r = id - n1 - n2;
      if (b.xcd_rows > 0) r = xcd_runs(r, b.plan_unpacked * ncb, b.xcd_rows * ncb);
      idx = r / ncb;
      x = r - idx * ncb;
      if (b.xcd_rows < 0 && (ncb & 7) == 0) {
        // column sweeps: XCD X takes the column blocks X, X + 8, ... one after the other, each over all row
        // blocks (what an XCD reads while it works on one column block is a 256-byte-wide strip of the source)
        const int xcd = r & 7, pos = r >> 3;
        const int cbi = pos / b.plan_unpacked;
        idx = pos - cbi * b.plan_unpacked;
        x = xcd + 8 * cbi;
      }
    }
    const int n_records = b.plan_unpacked + b.plan_packed2 + b.plan_packed4;
    const_u32 e = (const_u32)((uintptr_t)b.plan + (uintptr_t)idx * sizeof(PlanEntry));
    const uint32_t row0 = e[0], where = e[3];
    const int rb = (int)e[1], count = (int)e[2];
    g.expert = 0;
    if (b.pad > 1)  // the one kernel that pads is the one that asks for the expert
      g.expert = (int)((const_u32)((uintptr_t)b.plan + (uintptr_t)n_records * sizeof(PlanEntry)))[idx];
    g.kc_shift = (int)kind - 1;
    const int pcount = b.pad > 1 ? (count + b.pad - 1) & -b.pad : count;
    const int64_t row_start = (int64_t)row0 - (int64_t)rb * kGroup;
    const int left = count - rb * kGroup;
    const int pleft = pcount - rb * kGroup;
    g.cb = x << g.kc_shift;
    const int cbs_left = ncb - g.cb;
    g.n_sub = cbs_left < (1 << g.kc_shift) ? cbs_left : (1 << g.kc_shift);
    // a record of another kind than its section's: the host's counts are not the device's
    g.valid = (where >> 30) == kind && idx < n_records;
    g.rows_valid = left < kGroup ? left : kGroup;
    g.rows_store = pleft < kGroup ? pleft : kGroup;
    g.row0 = (int64_t)row0;
    g.s_base = row_start * (out_w / kGroup) + (int64_t)rb * kGroup;
    g.s_stride = pcount;
    g.t_base = row_start * out_w + (int64_t)rb * kGroup;
    g.t_stride = pcount;
    g.st_row = (int64_t)(where & 0x3fffffffu);
    if (g.row0 + g.rows_store > M) g.valid = false;
  } else {
    if (b.xcd_rows > 0) id = xcd_runs(id, (int)n_wg_x(), b.xcd_rows * ncb);
    const ExpertTile et = find_expert_tile(b.counts, b.counts_i64, b.n_experts, id, ncb, b.pad > 1 ? b.pad : 1);
    // the lookup's answer is the same in every lane: keep it in scalar registers
    const int expert = uniform32(et.expert), count = uniform32(et.count), rb = uniform32(et.rb);
    const int pcount = uniform32(et.pcount);
    g.cb = uniform32(et.cb);
    g.kc_shift = uniform32(et.kc_shift);
    const int cbs_left = ncb - g.cb;
    g.n_sub = cbs_left < (1 << g.kc_shift) ? cbs_left : (1 << g.kc_shift);
    const int64_t row_start = uniform64(et.row_start), tblock_start = uniform64(et.tblock_start);
    g.valid = expert >= 0;
    g.expert = expert;
    const int left = count - rb * kGroup;
    const int pleft = pcount - rb * kGroup;
    g.rows_valid = left < kGroup ? left : kGroup;
    g.rows_store = pleft < kGroup ? pleft : kGroup;
    g.row0 = row_start + (int64_t)rb * kGroup;
    g.s_base = row_start * (out_w / kGroup) + (int64_t)rb * kGroup;
    g.s_stride = pcount;
    g.t_base = row_start * out_w + (int64_t)rb * kGroup;
    g.t_stride = pcount;
    g.st_row = tblock_start + rb;
    if (g.row0 + g.rows_store > M) g.valid = false;  // counts disagree with the matrix: write nothing
  }
  return g;
}

struct OutPtrs {
  uint8_t* q;
  float* s;
  uint8_t* qt;
  float* st;
};

// ocb: 128-column block index inside the quantised matrix of width out_w
__device__ __forceinline__ TileOut make_out(const OutPtrs& p, const TileGeom& g, int64_t out_w, int ocb) {
  TileOut o;
  o.q = p.q;
  o.q_off = g.row0 * out_w + (int64_t)ocb * kGroup;
  o.q_ld = out_w;
  o.s = p.s;
  o.s_off = g.s_base + (int64_t)ocb * g.s_stride;
  o.qt = p.qt;
  o.t_off = g.t_base + (int64_t)ocb * kGroup * g.t_stride;
  o.t_ld = g.t_stride;
  o.st = p.st;
  o.st_off = g.st_row * out_w + (int64_t)ocb * kGroup;
  o.rows_valid = g.rows_store;
  o.kc_shift = g.kc_shift;
  o.n_sub = g.n_sub;
  o.s_cb = g.s_stride;
  o.t_cb = (int64_t)kGroup * g.t_stride;
  return o;
}

// RPT rows x 8 bf16 columns of a row-major matrix; rows >= rows_valid read as 0
// STREAM: loads carry the non-temporal hint (the tile is not read again).
// SCALAR: the tile base, the same in every lane of a wave, is moved to scalar registers
// rgl: the thread's row group (rows rgl*RPT ..): tile_tid() >> 4 in an unpacked tile, the row
// group inside the wave's sub-tile in a packed one (then base points at that sub-tile's columns)
// The loads carry no condition: a row beyond rows_valid fetches row 0 of the tile again (`base`
// must be a valid address also when rows_valid is 0); the caller zeroes such rows with mask_rows
// once every load of the tile has been issued.  With the loads
// behind per-row branches, and a second, mask-free copy of them for full tiles, the compiler's
// wait insertion turned conservative where the paths meet: the per-expert SwiGLU forward waited
// for the whole x1 tile before it asked for x2.
template <int RPT, bool STREAM = false, bool SCALAR = true>
__device__ __forceinline__ void load_rows(const uint16_t* base, int64_t ld, int rows_valid, uint4 (&raw)[RPT],
                                          int rgl) {
  const int cg = tile_tid() & 15;
  // a tile spans at most 128 rows of at most 2^24 bytes (the widest input the entry
  // points accept), so lane offsets fit 32 bits
  const uint8_t* b = (const uint8_t*)base;
  uint32_t pitch = (uint32_t)ld * 2u;
  if constexpr (SCALAR) {
    b = (const uint8_t*)uniform64((int64_t)b);
    pitch = (uint32_t)uniform32((int)pitch);
  }
  const uint32_t col = (uint32_t)cg * 16u;
#pragma unroll
  for (int s = 0; s < RPT; ++s) {
    const int i = rgl * RPT + s;
    raw[s] = load16<STREAM>(b + ((uint32_t)(i < rows_valid ? i : 0) * pitch + col));
  }
}
// zero the rows that load_rows fetched from beyond rows_valid; called after ALL loads of a tile
// have been issued (it has to wait for the rows it touches)
template <int RPT>
__device__ __forceinline__ void mask_rows(int rows_valid, uint4 (&raw)[RPT], int rgl) {
  if (rows_valid != kGroup) {  // workgroup-uniform
#pragma unroll
    for (int s = 0; s < RPT; ++s)
      if (rgl * RPT + s >= rows_valid) raw[s] = make_uint4(0, 0, 0, 0);
  }
}
template <int RPT, bool STREAM = false, bool SCALAR = true>
__device__ __forceinline__ void load_rows(const uint16_t* base, int64_t ld, int rows_valid, uint4 (&raw)[RPT]) {
  load_rows<RPT, STREAM, SCALAR>(base, ld, rows_valid, raw, (int)(tile_tid() >> 4));
}

// The part of a (possibly packed) tile this thread's wave works on, and how many of its rows exist
template <int RPT>
struct TilePart {
  SubTile<RPT> sl;
  int rows;  // rows of this wave's sub-tile that exist (0: the column block lies beyond the matrix)
  int cb;    // its 128-column block
  int asub;  // column block inside the workgroup's run to LOAD from: sl.sub, or 0 when rows == 0 (a valid address)
};
template <int RPT>
__device__ __forceinline__ TilePart<RPT> tile_part(const TileGeom& g) {
  TilePart<RPT> p;
  p.sl = sub_tile<RPT>(g.kc_shift);
  p.rows = p.sl.sub < g.n_sub ? g.rows_valid : 0;
  p.cb = g.cb + p.sl.sub;
  p.asub = p.sl.sub < g.n_sub ? p.sl.sub : 0;
  return p;
}

#define FQ_DISPATCH_BOOL(flag, NAME, ...) \
  if (flag) { constexpr bool NAME = true; __VA_ARGS__ } else { constexpr bool NAME = false; __VA_ARGS__ }
#define FQ_DISPATCH_KIND(kind, NAME, ...) \
  if ((kind) == kE5M2) { constexpr int NAME = kE5M2; __VA_ARGS__ } else { constexpr int NAME = kE4M3; __VA_ARGS__ }
#define FQ_DISPATCH_MODE(mode, NAME, ...)                                    \
  if ((mode) == 0) { constexpr int NAME = 0; __VA_ARGS__ }                   \
  else if ((mode) == 1) { constexpr int NAME = 1; __VA_ARGS__ }              \
  else { constexpr int NAME = 2; __VA_ARGS__ }

}  // namespace fq
