// Tuning policy of the kernels: cache hints, rows per thread, tile order.  Every value here
// was chosen by measurement on MI355X with cold inputs (buffers rotated beyond the memory-side
// cache); results are identical whatever the values.  One table for the whole library.
//
// A sweep build may replace the table: compile with -DFQ_POLICY_HEADER='"my_policy.hpp"', a
// header that defines fq::Policy with the same members.
#pragma once

#ifdef FQ_POLICY_HEADER
#include FQ_POLICY_HEADER
#else
namespace fq {

struct Policy {
  // ---- which code stores carry the non-temporal hint (bit 0: transposed codes, bit 1: row-wise
  // codes).  With it the outputs do not displace inputs from L2 and the memory-side cache:
  // gather+pad+quant 75 -> 55 us, RMSNorm+quant after the statistic pass 25 -> 21 us
  // (8192 x 2048) and 146 -> 122 us (16384 x 7168).  The SwiGLU backward is 3-7 % slower when its
  // transposed stores carry it; the plain blockwise quantiser takes none (13.2 us at 8192 x 2048
  // against 14.2-16.1 with any), its per-expert form the transposed stores only (31.5 us against
  // 39.2 without, 32.7 with the row-wise codes only and 36.3 with both); the RMSNorm tile kernel
  // with the statistic given (transposed output only, x read once: nothing to protect) none
  // (16384 x 7168: 66.6 -> 59.5 us).  Transposed rows that do not start on 16-byte boundaries
  // (M or a per-expert count that is not a multiple of 16) are where the hint on the transposed
  // stores costs most: the SwiGLU forward takes 100 instead of 70 us at 16300 x 3584 with it (and
  // gains 3 % at 8192 x 2048), so it keeps the hint on the row-wise codes only; the RMSNorm tile
  // kernel gains 18 % from it on aligned rows and loses 8 % on unaligned ones.
  static constexpr int kStoreHintBlockwise = 0;
  static constexpr int kStoreHintBlockwiseBatched = 1;
  // ... and with its tiles read from a plan, numbered so that neighbouring row blocks share an XCD, the row-wise
  // codes only (the L2 then merges the partial lines of the transposed ones): 65536 x 512 in 256 experts
  // 33.2 / 29.8 / 27.8 / 33.5 us with 0 / 1 / 2 / 3
  static constexpr int kStoreHintBlockwisePlanned = 2;
  static constexpr int kStoreHintPermute = 3;
  static constexpr int kStoreHintSiluFwd = 2;        // both layouts, single matrix
  static constexpr int kStoreHintSiluFwdRows = 2;    // row-wise layout only
  static constexpr int kStoreHintSiluFwdCols = 1;    // transposed layout only
  static constexpr int kStoreHintSiluFwdBatched = 2;
  static constexpr int kStoreHintSiluBwd = 2;
  static constexpr int kStoreHintSiluBwdBatched = 2;
  static constexpr int kStoreHintRmsnorm = 3;        // both layouts (x is read again: protect it)
  static constexpr int kStoreHintRmsnormCols = 0;    // transposed output only, statistic given

  // ---- the bulk loads carry the hint (3-5 % on the SwiGLU kernels and the RMSNorm tile kernel,
  // 12 % on the plain blockwise quantiser, 6 % on its per-expert form; the gathered rows, which
  // several experts read, are 27 % slower with it)
  static constexpr bool kLoadHintBlockwise = true;
  static constexpr bool kLoadHintBlockwiseBatched = true;
  static constexpr bool kLoadHintPermute = false;
  static constexpr bool kLoadHintSiluFwd = true;
  static constexpr bool kLoadHintSiluFwdBatched = true;
  static constexpr bool kLoadHintSiluBwd = true;
  static constexpr bool kLoadHintSiluBwdBatched = true;
  static constexpr bool kLoadHintRmsnorm = true;

  // ---- the lean form of the quantiser and of the tile loads (scalar bases, paired
  // column-maximum reduction; every other tile kernel uses it, -3 to -9 %) in the PLAIN
  // blockwise quantiser, which is 7 % slower with it (48 -> 51 us at 65536 x 1024); the
  // per-expert form takes it (Zipf counts: 60.6 -> 57.9 us)
  static constexpr bool kLeanBlockwise = false;

  // ---- rows per thread (workgroup = 2048 / rows threads).  8 rows per thread spread the
  // per-thread overhead over twice the elements, 4 rows per thread put twice the waves on a CU.
  // The SwiGLU forward needs 135 registers with 8 and loses 5-9 %.  The RMSNorm tile kernel
  // measured 3-4 % ahead with 8 (93 registers, five 256-thread workgroups per CU) when its
  // division took three operations per element; with the current two it is level at
  // 16384 x 7168 (110.5 us either way, 58.9 / 58.5 us with the statistic given) and 2 % behind at
  // 8192 x 2048 (18.3 / 18.0 us), so it runs with 4.
  static constexpr int kRowsPerThreadSiluFwd = 4;
  // Rows of a 128x128 tile per thread in the plain blockwise quantiser: 8 (256 threads) for the
  // dense form (4 rows: 13.2 -> 13.9 us on 8192x4096), 4 (512 threads) for the per-expert form,
  // which waits on its lookup and gains from more waves per CU (31.3 -> 30.9 us, 32 experts).
  static constexpr int kRowsPerThreadBlockwise = 8;
  static constexpr int kRowsPerThreadBlockwiseBatched = 4;
  static constexpr int kRowsPerThreadRmsnorm = 4;
  // waves (one row each) per workgroup of the statistic pass: 18.10 / 18.00 / 18.00 / 18.04 us at 8192 x 2048 and
  // 107.8 / 108.0 / 107.4 / 107.6 at 16384 x 7168 with 1 / 2 / 4 / 8
  static constexpr int kRowstatWaves = 4;
  // per-expert launches that read their tiles from a plan: the packed tiles (last row blocks of at most 64
  // rows) before or behind the others.  65536 rows in 256 experts (Zipf counts), packed first / last:
  // SwiGLU forward 44.2 / 43.2 us, backward 77.7 / 77.4, blockwise quantiser 30.9 / 31.8
  static constexpr bool kPlanPackedFirstSiluFwd = false;
  static constexpr bool kPlanPackedFirstSiluBwd = false;
  static constexpr bool kPlanPackedFirstBlockwise = true;
  static constexpr bool kPlanPackedFirstPermute = false;  // 43.8 / 43.3 us first / last (33040 x 2048 gathered from 16384 rows)
  // row blocks per run that an XCD works on (xcd_runs; 0: every eighth tile).  Same sizes, planned launches with
  // 0 / 2 / 4 / 8 / 16: SwiGLU forward 43.4 / 41.2 / 40.8 / 40.7 / 40.8 us, backward 76.5 / 76.1 / 75.5 / 75.3 / 76.2,
  // blockwise quantiser 30.9 / 30.3 / 29.9 / 29.9 / 29.8.  Launches that scan the counts, 0 / 2 / 4 / 8: forward
  // 44.4 / 45.2 / 45.1 / 45.6, backward 80.4 / 78.4 / 78.4 / 79.4, blockwise 31.1 / 32.2 / 32.4 / 32.7,
  // gather + pad + quant 47.0 / 48.8 / 49.4 / 50.8: only the backward gains there
  static constexpr int kXcdRowsPlanned = 8;
  static constexpr int kXcdRowsSiluBwdCounts = 4;
  // gather + pad + quant with a plan: runs of 8 row blocks per XCD 50.6 us, grid order 44.8, column sweeps (-1:
  // XCD X takes the column blocks X, X + 8, .. one after the other, so that what it gathers from while it works
  // on one of them is a 256-byte strip of the source: 4.2 MB for 16384 source rows, the size of its L2) 43.8;
  // the launch that scans the counts 45.6
  static constexpr int kXcdRowsPermutePlanned = -1;
  static constexpr bool kStartPriorityRmsnorm = true;
  // RMSNorm + quant in two passes, both passes giving XCD X (workgroup number mod 8) the X-th eighth of the rows,
  // the statistic pass walking its eighth from the end and the tile kernel from the start: what the tile kernel
  // reads first is what the same XCD's L2 read last.  Rows a multiple of 1024 (the eighths are whole row blocks).
  // us without / with: 2048 x 2048 8.8 / 7.9, 4096 x 2048 11.7 / 10.6, 8192 x 2048 17.9 / 16.6, 3072 x 4096
  // 14.6 / 13.3, 4096 x 7168 30.2 / 27.9, 8192 x 4096 33.0 / 32.0, 16384 x 2048 33.2 / 31.7, 8192 x 7168
  // 55.8 / 52.9, 16384 x 4096 63.4 / 62.7, 32768 x 2048 63.6 / 63.3, 16384 x 7168 108.1 / 109.6: up to this
  // many bytes of input
  static constexpr long long kRmsnormByXcdMaxBytes = 160ll << 20;
  // 16-byte chunks per lane, matrix and step in the bf16 SwiGLU backward (three matrices are read):
  // 29.0 / 30.4 / 28.7 / 35.5 us with 2 / 3 / 4 / 8 at 8192 x 4096
  static constexpr int kSwigluBwdRowsUnroll = 4;
  // the wide-row (four waves per row) RMSNorm + row-wise quant kernel loads the next row while it works on
  // the current one (122 instead of 84 registers): 68.5 -> 65.5 us at 16384 x 7168
  static constexpr bool kPrefetchRowQuantWide = true;
  // workgroups per CU of that kernel's launch (it holds four at 122 registers): 64.0 / 65.4 / 64.8 / 64.6 /
  // 68.0 us with 4 / 5 / 6 / 8 / 12 at 16384 x 7168
  static constexpr int kRowQuantWideWgsPerCu = 4;
  // the same in the wide-row RMSNorm backward with one chunk per thread (2048 < n <= 4096: 70.4 -> 66.9 us at
  // 16384 x 3072, 78.5 -> 76.4 at 16384 x 4096); with two chunks the second register set spills
  static constexpr bool kPrefetchRowBwdWide = true;
  // 1x128 groups per thread and step of the plain group quantiser (their loads are in flight together):
  // 10.3 / 10.5 / 13.0 us with 1 / 2 / 4 at 8192 x 2048, where a thread has two groups in all
  static constexpr int kGroupQuantUnroll = 1;

  // ---- the SwiGLU backwards widen row s of their packed inputs after row s-1 is done (fence_values):
  // without it the per-expert form needed 136 registers under its cap of 128 and spilled; with it (and no
  // branch around the arithmetic) 105, the single-matrix form 100
  static constexpr bool kPinBwdRowsBatched = true;
  static constexpr bool kPinBwdRows = true;

  // ---- row kernels: the outputs are written once (-3 to -7 % with the hint on the RMSNorm
  // backward, the bf16 SwiGLU rows and the 128x128 block quantiser); the loads of rows that a
  // kernel reads once carry it too; RMSNorm + row-wise quant gives every XCD one contiguous
  // eighth of the rows (13.0 -> 12.4 us at 8192 x 2048)
  static constexpr bool kStoreHintRows = true;
  static constexpr bool kLoadHintRows = true;
  static constexpr bool kXcdContiguousRowQuant = true;

  // ---- router kernels: hint on the stores of y and the codes, and on the loads of x in the
  // register-resident kernel
  static constexpr bool kStoreHintRouter = true;
  static constexpr bool kLoadHintRouter = true;
};

}  // namespace fq
#endif
