// C-ABI layer: argument validation + dispatch to the kernel launchers.
// The only mutable state is the per-thread error message.
#include "../../include/fq_api.h"

#include <stdarg.h>
#include <stdio.h>

#include "fq_launch.h"

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(hipError_t e, const char* what) {
  if (e == hipSuccess) return FQ_OK;
  return fail(FQ_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define FQ_REQUIRE(cond, code, ...) \
  do { if (!(cond)) return fail(code, __VA_ARGS__); } while (0)

int check_common(const char* fn, int64_t M, int64_t width, int round_scale, int fp8_kind) {
  FQ_REQUIRE(M >= 0, FQ_ERR_SHAPE, "%s: negative row count", fn);
  FQ_REQUIRE(width > 0 && width % 128 == 0, FQ_ERR_SHAPE, "%s: width %lld is not a positive multiple of 128", fn,
             (long long)width);
  // lane offsets inside a tile are 32-bit: 128 rows of the widest input (2 * width bf16) and 128
  // transposed rows of M bytes must stay below 4 GB
  FQ_REQUIRE(width <= (1 << 22), FQ_ERR_SHAPE, "%s: width too large", fn);
  FQ_REQUIRE(M <= ((int64_t)1 << 24), FQ_ERR_SHAPE, "%s: too many rows", fn);
  FQ_REQUIRE(round_scale == 0 || round_scale == 1, FQ_ERR_ARG, "%s: round_scale must be 0 or 1", fn);
  FQ_REQUIRE(fp8_kind == FQ_E4M3 || fp8_kind == FQ_E5M2, FQ_ERR_ARG, "%s: unknown fp8_kind %d", fn, fp8_kind);
  return FQ_OK;
}

int check_mode_ptrs(const char* fn, int mode, const void* q, const void* s, const void* qt, const void* st) {
  FQ_REQUIRE(mode >= 0 && mode <= 2, FQ_ERR_ARG, "%s: output_mode must be 0, 1 or 2", fn);
  if (mode != 1) FQ_REQUIRE(q && s, FQ_ERR_ARG, "%s: row-wise outputs are NULL", fn);
  if (mode != 0) FQ_REQUIRE(qt && st, FQ_ERR_ARG, "%s: transposed outputs are NULL", fn);
  if (q) FQ_REQUIRE((reinterpret_cast<uintptr_t>(q) & 7u) == 0, FQ_ERR_ARG, "%s: q must be 8-byte aligned", fn);
  return FQ_OK;
}

int check_tiles(const char* fn, int64_t tiles) {
  FQ_REQUIRE(tiles < ((int64_t)1 << 31), FQ_ERR_SHAPE, "%s: too many tiles for one launch", fn);
  return FQ_OK;
}

}  // namespace

extern "C" {

int fq_version(void) { return 200; }  // 0.2.0: tile plans and the *_planned entry points

const char* fq_last_error(void) { return g_err; }

int fq_stream_rw_variant(const void* src, int64_t read_bytes, void* dst, int64_t write_bytes, void* sink,
                         int chunks_per_lane, int64_t workgroups, int order, int nt_loads, int nt_stores,
                         void* stream) {
  const char* fn = "fq_stream_rw_variant";
  FQ_REQUIRE(read_bytes >= 0 && write_bytes >= 0 && read_bytes % 16 == 0 && write_bytes % 16 == 0, FQ_ERR_SHAPE,
             "%s: byte counts must be non-negative multiples of 16", fn);
  FQ_REQUIRE((read_bytes == 0 || (src && aligned16(src))) && (write_bytes == 0 || (dst && aligned16(dst))) && sink &&
                 aligned16(sink),
             FQ_ERR_ARG, "%s: NULL or misaligned pointer", fn);
  FQ_REQUIRE(chunks_per_lane == 4 || chunks_per_lane == 8 || chunks_per_lane == 16, FQ_ERR_ARG,
             "%s: chunks_per_lane must be 4, 8 or 16", fn);
  FQ_REQUIRE(order >= 0 && order <= 3 && workgroups >= 0 && workgroups <= (1 << 24), FQ_ERR_ARG,
             "%s: order must be 0 .. 3 and workgroups 0 .. 2^24", fn);
  return check_launch(fq::launch_stream_rw(src, read_bytes, dst, write_bytes, sink, chunks_per_lane, workgroups, order,
                                           nt_loads != 0, nt_stores != 0, (hipStream_t)stream),
                      fn);
}

int fq_stream_rw(const void* src, int64_t read_bytes, void* dst, int64_t write_bytes, void* sink, int nontemporal,
                 void* stream) {
  // the plain form: 4 chunks per lane, at most 64 workgroups per CU, interleaved steps
  return fq_stream_rw_variant(src, read_bytes, dst, write_bytes, sink, 4, 256 * 64, 0, nontemporal, nontemporal,
                              stream);
}

int fq_blockwise_quant(const void* x, void* q, float* s, void* qt, float* st, int64_t M, int64_t N,
                       int round_scale, int output_mode, int fp8_kind, void* stream) {
  const char* fn = "fq_blockwise_quant";
  int rc = check_common(fn, M, N, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_mode_ptrs(fn, output_mode, q, s, qt, st))) return rc;
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && aligned16(x), FQ_ERR_ARG, "%s: x is NULL or not 16-byte aligned", fn);
  const int64_t rbs = (M + 127) / 128;
  if ((rc = check_tiles(fn, rbs * (N / 128)))) return rc;
  return check_launch(fq::launch_blockwise_quant(x, q, s, qt, st, M, (int)N, round_scale, output_mode, fp8_kind,
                                                 nullptr, 0, 0, rbs, (hipStream_t)stream),
                      fn);
}

}  // extern "C"

// The per-expert entry points come in two forms that differ only in where a workgroup learns its
// tile: from the device-side counts, or from a plan built from them (counts NULL, n_experts unused).
static int check_plan_shape(const char* fn, const int64_t* shape, int pad, fq::PlanShape* ps) {
  FQ_REQUIRE(shape != nullptr, FQ_ERR_ARG, "%s: plan shape NULL", fn);
  FQ_REQUIRE(shape[1] >= 0 && shape[2] >= 0 && shape[3] >= 0 && shape[0] == shape[1] + shape[2] + shape[3] &&
                 shape[0] <= (int64_t)0x3fffffff && (shape[4] == 1 || shape[4] == 16),
             FQ_ERR_SHAPE, "%s: not a plan shape (fq_expert_plan_shape fills it)", fn);
  // pad 0: any (the builder); otherwise the layout of the entry point that is given the plan
  FQ_REQUIRE(pad == 0 || shape[4] == pad, FQ_ERR_SHAPE, "%s: the plan was shaped for regions padded to %lld rows, not %d",
             fn, (long long)shape[4], pad);
  ps->unpacked = shape[1];
  ps->packed2 = shape[2];
  ps->packed4 = shape[3];
  ps->pad = (int)shape[4];
  return FQ_OK;
}

static int check_batch_source(const char* fn, const void* counts, int n_experts, const void* plan,
                              int64_t total_blocks, int64_t M) {
  FQ_REQUIRE(total_blocks >= 0, FQ_ERR_SHAPE, "%s: negative block count", fn);
  if (plan != nullptr) {
    FQ_REQUIRE(aligned16(plan), FQ_ERR_ARG, "%s: plan misaligned", fn);
    // every row block holds at least one row
    FQ_REQUIRE(total_blocks <= M, FQ_ERR_SHAPE, "%s: plan shape inconsistent with M", fn);
    FQ_REQUIRE(M <= (int64_t)0x7fffffff, FQ_ERR_SHAPE, "%s: a plan addresses at most 2^31 - 1 rows", fn);
    return FQ_OK;
  }
  FQ_REQUIRE(n_experts >= 0, FQ_ERR_SHAPE, "%s: negative expert count", fn);
  FQ_REQUIRE(counts != nullptr, FQ_ERR_ARG, "%s: counts NULL", fn);
  FQ_REQUIRE(total_blocks <= (M + 127) / 128 + n_experts, FQ_ERR_SHAPE, "%s: total_blocks inconsistent with M", fn);
  return FQ_OK;
}

static int batched_blockwise_quant(const char* fn, const void* x, const void* counts, int counts_is_i64,
                                   int n_experts, const void* plan, const fq::PlanShape* ps, int64_t total_blocks,
                                   void* q, float* s, void* qt, float* st, int64_t M, int64_t N, int round_scale,
                                   int fp8_kind, void* stream) {
  int rc = check_common(fn, M, N, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_mode_ptrs(fn, 2, q, s, qt, st))) return rc;
  FQ_REQUIRE((plan != nullptr || n_experts >= 0) && total_blocks >= 0, FQ_ERR_SHAPE,
             "%s: negative expert/block count", fn);
  if (M == 0 || total_blocks == 0) return FQ_OK;
  FQ_REQUIRE(x && aligned16(x), FQ_ERR_ARG, "%s: x NULL or misaligned", fn);
  if ((rc = check_batch_source(fn, counts, n_experts, plan, total_blocks, M))) return rc;
  if ((rc = check_tiles(fn, total_blocks * (N / 128)))) return rc;
  return check_launch(fq::launch_blockwise_quant(x, q, s, qt, st, M, (int)N, round_scale, 2, fp8_kind, counts,
                                                 counts_is_i64 != 0, n_experts, total_blocks, (hipStream_t)stream,
                                                 plan, ps),
                      fn);
}

extern "C" {

int fq_batched_blockwise_quant(const void* x, const void* counts, int counts_is_i64, int n_experts,
                               int64_t total_blocks, void* q, float* s, void* qt, float* st, int64_t M,
                               int64_t N, int round_scale, int fp8_kind, void* stream) {
  return batched_blockwise_quant("fq_batched_blockwise_quant", x, counts, counts_is_i64, n_experts, nullptr, nullptr,
                                 total_blocks, q, s, qt, st, M, N, round_scale, fp8_kind, stream);
}

int fq_batched_blockwise_quant_planned(const void* x, const void* plan, const int64_t* shape, void* q, float* s,
                                       void* qt, float* st, int64_t M, int64_t N, int round_scale, int fp8_kind,
                                       void* stream) {
  const char* fn = "fq_batched_blockwise_quant_planned";
  fq::PlanShape ps;
  int rc = check_plan_shape(fn, shape, 1, &ps);
  if (rc) return rc;
  FQ_REQUIRE(plan != nullptr || M == 0 || shape[0] == 0, FQ_ERR_ARG, "%s: plan NULL", fn);
  return batched_blockwise_quant(fn, x, nullptr, 0, 0, plan, &ps, shape[0], q, s, qt, st, M, N, round_scale, fp8_kind,
                                 stream);
}

int fq_expert_plan_shape(const int64_t* host_counts, int n_experts, int pad, int64_t* shape) {
  const char* fn = "fq_expert_plan_shape";
  FQ_REQUIRE(n_experts >= 0 && shape != nullptr && (host_counts != nullptr || n_experts == 0), FQ_ERR_ARG,
             "%s: NULL pointer or negative expert count", fn);
  FQ_REQUIRE(pad == 1 || pad == 16, FQ_ERR_ARG, "%s: pad is 1 (experts back to back) or 16", fn);
  const fq::PlanShape ps = fq::expert_plan_shape(host_counts, n_experts, pad);
  FQ_REQUIRE(ps.blocks() <= (int64_t)0x3fffffff, FQ_ERR_SHAPE, "%s: more than 2^30 - 1 row blocks", fn);
  shape[0] = ps.blocks();
  shape[1] = ps.unpacked;
  shape[2] = ps.packed2;
  shape[3] = ps.packed4;
  shape[4] = pad;
  return FQ_OK;
}

int64_t fq_expert_plan_bytes(const int64_t* shape) {
  return shape == nullptr || shape[0] < 0 ? 0 : shape[0] * 20;
}

int fq_build_expert_plan(const void* counts, int counts_is_i64, int n_experts, const int64_t* shape, void* plan,
                         void* stream) {
  const char* fn = "fq_build_expert_plan";
  fq::PlanShape ps;
  int rc = check_plan_shape(fn, shape, 0, &ps);
  if (rc) return rc;
  FQ_REQUIRE(n_experts >= 0, FQ_ERR_SHAPE, "%s: negative expert count", fn);
  if (shape[0] == 0) return FQ_OK;
  FQ_REQUIRE(plan && aligned16(plan) && (counts || n_experts == 0), FQ_ERR_ARG, "%s: NULL or misaligned pointer", fn);
  return check_launch(fq::launch_expert_plan(counts, counts_is_i64 != 0, n_experts, ps, plan, (hipStream_t)stream),
                      fn);
}

}  // extern "C"

static int batched_pad_permute_quant(const char* fn, const void* x, const void* counts, int counts_is_i64,
                                     int n_experts, const void* plan, const fq::PlanShape* ps, int64_t total_blocks,
                                     const void* indices, const void* probs, int probs_is_bf16, void* prob_out,
                                     void* q, float* s, void* qt, float* st, int64_t src_rows, int64_t M, int64_t N,
                                     int round_scale, int fp8_kind, void* stream) {
  int rc = check_common(fn, M, N, round_scale, fp8_kind);
  if (rc) return rc;
  if (M == 0) return FQ_OK;  // nothing routed: there is nothing to write (and empty outputs may be NULL)
  FQ_REQUIRE(n_experts >= 0 && total_blocks >= 0 && src_rows >= 0, FQ_ERR_SHAPE, "%s: negative count", fn);
  FQ_REQUIRE(src_rows <= ((int64_t)1 << 31) - 1, FQ_ERR_SHAPE, "%s: too many source rows for int32 indices", fn);
  FQ_REQUIRE(M % 16 == 0, FQ_ERR_SHAPE, "%s: M (%lld) must be the sum of the counts each rounded up to 16", fn,
             (long long)M);
  if ((rc = check_mode_ptrs(fn, 2, q, s, qt, st))) return rc;
  FQ_REQUIRE((probs == nullptr) == (prob_out == nullptr), FQ_ERR_ARG, "%s: probs and prob_out go together", fn);
  if (M == 0 || total_blocks == 0 || src_rows == 0) return FQ_OK;
  FQ_REQUIRE(x && aligned16(x) && indices && aligned16(indices), FQ_ERR_ARG, "%s: x/indices NULL or misaligned", fn);
  if ((rc = check_batch_source(fn, counts, n_experts, plan, total_blocks, M))) return rc;
  if ((rc = check_tiles(fn, total_blocks * (N / 128)))) return rc;
  return check_launch(fq::launch_pad_permute_quant(x, indices, probs, probs_is_bf16 != 0, prob_out, q, s, qt, st,
                                                   src_rows, M, (int)N, round_scale, fp8_kind, counts,
                                                   counts_is_i64 != 0, n_experts, total_blocks, (hipStream_t)stream,
                                                   plan, ps),
                      fn);
}

extern "C" {

int fq_batched_pad_permute_quant(const void* x, const void* counts, int counts_is_i64, int n_experts,
                                 int64_t total_blocks, const void* indices, const void* probs, int probs_is_bf16,
                                 void* prob_out, void* q, float* s, void* qt, float* st, int64_t src_rows,
                                 int64_t M, int64_t N, int round_scale, int fp8_kind, void* stream) {
  return batched_pad_permute_quant("fq_batched_pad_permute_quant", x, counts, counts_is_i64, n_experts, nullptr,
                                   nullptr, total_blocks, indices, probs, probs_is_bf16, prob_out, q, s, qt, st,
                                   src_rows, M, N, round_scale, fp8_kind, stream);
}

int fq_batched_pad_permute_quant_planned(const void* x, const void* plan, const int64_t* shape, int n_experts,
                                         const void* indices, const void* probs, int probs_is_bf16, void* prob_out,
                                         void* q, float* s, void* qt, float* st, int64_t src_rows, int64_t M,
                                         int64_t N, int round_scale, int fp8_kind, void* stream) {
  const char* fn = "fq_batched_pad_permute_quant_planned";
  fq::PlanShape ps;
  int rc = check_plan_shape(fn, shape, 16, &ps);
  if (rc) return rc;
  FQ_REQUIRE(plan != nullptr || M == 0 || shape[0] == 0, FQ_ERR_ARG, "%s: plan NULL", fn);
  return batched_pad_permute_quant(fn, x, nullptr, 0, n_experts, plan, &ps, shape[0], indices, probs, probs_is_bf16,
                                   prob_out, q, s, qt, st, src_rows, M, N, round_scale, fp8_kind, stream);
}

int fq_group_quant(const void* x, void* q, float* s, int64_t M, int64_t N, int round_scale, int fp8_kind,
                   void* stream) {
  const char* fn = "fq_group_quant";
  int rc = check_common(fn, M, N, round_scale, fp8_kind == FQ_E5M2_MAX448 ? FQ_E5M2 : fp8_kind);
  if (rc) return rc;
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && aligned16(x) && q && s, FQ_ERR_ARG, "%s: NULL or misaligned pointer", fn);
  FQ_REQUIRE((reinterpret_cast<uintptr_t>(q) & 7u) == 0, FQ_ERR_ARG, "%s: q must be 8-byte aligned", fn);
  return check_launch(fq::launch_group_quant(x, q, s, M * (N / 128), round_scale, fp8_kind, (hipStream_t)stream), fn);
}

static int check_norm_shape(const char* fn, int64_t M, int64_t n) {
  FQ_REQUIRE(M >= 0, FQ_ERR_SHAPE, "%s: negative row count", fn);
  FQ_REQUIRE(n > 0 && n % 8 == 0 && n <= 8192, FQ_ERR_SHAPE,
             "%s: hidden size %lld must be a multiple of 8 and at most 8192", fn, (long long)n);
  FQ_REQUIRE(M <= ((int64_t)1 << 31) - 256, FQ_ERR_SHAPE, "%s: too many rows", fn);
  return FQ_OK;
}

int fq_rmsnorm_fwd(const void* x, const void* gamma, void* out, float* rstd, int64_t M, int64_t n, float eps,
                   int reuse_rstd, void* stream) {
  const char* fn = "fq_rmsnorm_fwd";
  int rc = check_norm_shape(fn, M, n);
  if (rc) return rc;
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && gamma && out && rstd, FQ_ERR_ARG, "%s: NULL pointer", fn);
  FQ_REQUIRE(aligned16(x) && aligned16(gamma) && aligned16(out), FQ_ERR_ARG, "%s: misaligned pointer", fn);
  return check_launch(fq::launch_rmsnorm_fwd(x, gamma, out, nullptr, rstd, M, (int)n, eps, reuse_rstd != 0, 0, 0,
                                             FQ_E4M3, (hipStream_t)stream),
                      fn);
}

int64_t fq_rmsnorm_bwd_num_partials(int64_t M, int64_t n) {
  (void)n;
  return fq::rmsnorm_bwd_partials(M);
}

int fq_rmsnorm_bwd(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx, float* dgamma,
                   float* dgamma_partials, int64_t n_partials, int64_t M, int64_t n, float eps, void* stream) {
  const char* fn = "fq_rmsnorm_bwd";
  int rc = check_norm_shape(fn, M, n);
  if (rc) return rc;
  FQ_REQUIRE(dgamma, FQ_ERR_ARG, "%s: dgamma is NULL", fn);
  FQ_REQUIRE(n_partials == fq::rmsnorm_bwd_partials(M), FQ_ERR_SHAPE,
             "%s: n_partials must equal fq_rmsnorm_bwd_num_partials(M, n)", fn);
  if (M > 0) {  // with no rows only dgamma is touched (it is zeroed); the row kernel is not launched
    FQ_REQUIRE(dy && x && gamma && dx && dgamma_partials, FQ_ERR_ARG, "%s: NULL pointer", fn);
    FQ_REQUIRE(aligned16(dy) && aligned16(x) && aligned16(gamma) && aligned16(dx) && aligned16(dgamma_partials),
               FQ_ERR_ARG, "%s: misaligned pointer", fn);
  }
  return check_launch(fq::launch_rmsnorm_bwd(dy, x, gamma, rstd, dx, dgamma, dgamma_partials, n_partials, M, (int)n,
                                             eps, (hipStream_t)stream),
                      fn);
}

int fq_rmsnorm_bwd_noalloc(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx,
                           float* dgamma, int64_t M, int64_t n, float eps, void* stream) {
  const char* fn = "fq_rmsnorm_bwd_noalloc";
  int rc = check_norm_shape(fn, M, n);
  if (rc) return rc;
  FQ_REQUIRE(dgamma, FQ_ERR_ARG, "%s: dgamma is NULL", fn);
  const int64_t need = fq::rmsnorm_bwd_partials(M) * n * (int64_t)sizeof(float);
  FQ_REQUIRE(need <= fq::rmsnorm_bwd_static_scratch_bytes(), FQ_ERR_SHAPE,
             "%s: %lld bytes of dgamma partials exceed the library's fixed %lld-byte scratch array", fn,
             (long long)need, (long long)fq::rmsnorm_bwd_static_scratch_bytes());
  if (M > 0) {
    FQ_REQUIRE(dy && x && gamma && dx, FQ_ERR_ARG, "%s: NULL pointer", fn);
    FQ_REQUIRE(aligned16(dy) && aligned16(x) && aligned16(gamma) && aligned16(dx), FQ_ERR_ARG,
               "%s: misaligned pointer", fn);
  }
  return check_launch(fq::launch_rmsnorm_bwd_static(dy, x, gamma, rstd, dx, dgamma, M, (int)n, eps,
                                                    (hipStream_t)stream),
                      fn);
}

int fq_rmsnorm_quant_fwd(const void* x, const void* gamma, void* q, float* s, float* rstd, void* qt, float* st,
                         int64_t M, int64_t n, float eps, int round_scale, int output_mode, int fp8_kind,
                         void* stream) {
  const char* fn = "fq_rmsnorm_quant_fwd";
  int rc = check_common(fn, M, n, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_norm_shape(fn, M, n))) return rc;
  if ((rc = check_mode_ptrs(fn, output_mode, q, s, qt, st))) return rc;
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && gamma && rstd, FQ_ERR_ARG, "%s: NULL pointer", fn);
  FQ_REQUIRE(aligned16(x) && aligned16(gamma), FQ_ERR_ARG, "%s: misaligned pointer", fn);
  hipStream_t st_ = (hipStream_t)stream;
  if ((rc = check_tiles(fn, ((M + 127) / 128) * (n / 128)))) return rc;
  if (output_mode == 0) {
    return check_launch(fq::launch_rmsnorm_fwd(x, gamma, q, s, rstd, M, (int)n, eps, 0, 1, round_scale, fp8_kind, st_),
                        fn);
  }
  if (output_mode == 2) {  // two passes: the statistic alone, then the tile kernel with both outputs
    rc = check_launch(fq::launch_rmsnorm_fwd(x, gamma, nullptr, nullptr, rstd, M, (int)n, eps, 0, 2, 0, FQ_E4M3, st_),
                      fn);
    if (rc) return rc;
  }
  return check_launch(fq::launch_rmsnorm_quant_tile(x, gamma, rstd, q, s, qt, st, M, (int)n, round_scale, output_mode,
                                                    fp8_kind, st_),
                      fn);
}

int fq_block_quant(const void* x, void* q, float* s, int64_t M, int64_t N, int round_scale, int fp8_kind,
                   void* stream) {
  const char* fn = "fq_block_quant";
  int rc = check_common(fn, M, N, round_scale, fp8_kind);
  if (rc) return rc;
  FQ_REQUIRE(M % 128 == 0, FQ_ERR_SHAPE, "%s: M (%lld) is not a multiple of 128", fn, (long long)M);
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && q && s && aligned16(x), FQ_ERR_ARG, "%s: NULL or misaligned pointer", fn);
  FQ_REQUIRE((reinterpret_cast<uintptr_t>(q) & 7u) == 0, FQ_ERR_ARG, "%s: q must be 8-byte aligned", fn);
  if ((rc = check_tiles(fn, (M / 128) * (N / 128)))) return rc;
  return check_launch(fq::launch_block_quant(x, q, s, M, (int)N, round_scale, fp8_kind, (hipStream_t)stream), fn);
}

int fq_swiglu_fwd(const void* x, const void* weight, int weight_is_bf16, void* out, int64_t M, int64_t n,
                  void* stream) {
  const char* fn = "fq_swiglu_fwd";
  int rc = check_common(fn, M, n, 0, FQ_E4M3);
  if (rc) return rc;
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && out && aligned16(x) && aligned16(out), FQ_ERR_ARG, "%s: NULL or misaligned pointer", fn);
  return check_launch(fq::launch_swiglu_rows_fwd(x, weight, weight_is_bf16 != 0, out, M, (int)n, (hipStream_t)stream),
                      fn);
}

int fq_swiglu_bwd(const void* g, const void* x, const void* weight, int weight_is_bf16, void* dx, void* dw,
                  int64_t M, int64_t n, void* stream) {
  const char* fn = "fq_swiglu_bwd";
  int rc = check_common(fn, M, n, 0, FQ_E4M3);
  if (rc) return rc;
  FQ_REQUIRE((weight == nullptr) == (dw == nullptr), FQ_ERR_ARG, "%s: weight and dw go together", fn);
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(g && x && dx && aligned16(g) && aligned16(x) && aligned16(dx), FQ_ERR_ARG,
             "%s: NULL or misaligned pointer", fn);
  return check_launch(fq::launch_swiglu_rows_bwd(g, x, weight, weight_is_bf16 != 0, dx, dw, M, (int)n,
                                                 (hipStream_t)stream),
                      fn);
}

int64_t fq_rmsnorm_router_scratch_bytes(int64_t K, int64_t N, int weight_is_fp32) {
  if (K <= 0 || N <= 0 || K > 8192 || N > 8192) return 0;
  return fq::rmsnorm_router_scratch_bytes((int)K, (int)N, weight_is_fp32 != 0);
}

int fq_rmsnorm_router_quant_fwd(const void* x, const void* gamma, const void* route_weight, int weight_is_fp32,
                                void* weight_scratch, void* y, float* rstd, float* logits, void* q, float* s,
                                int64_t M, int64_t K, int64_t N, float eps, int round_scale, int fp8_kind,
                                void* stream) {
  const char* fn = "fq_rmsnorm_router_quant_fwd";
  int rc = check_common(fn, M, K, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_norm_shape(fn, M, K))) return rc;
  FQ_REQUIRE(M % 32 == 0, FQ_ERR_SHAPE, "%s: M (%lld) is not a multiple of 32", fn, (long long)M);
  FQ_REQUIRE(N > 0 && N % 128 == 0 && N <= 8192, FQ_ERR_SHAPE,
             "%s: %lld router outputs (supported: multiples of 128 up to 8192)", fn, (long long)N);
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && gamma && route_weight && weight_scratch && y && rstd && logits && q && s, FQ_ERR_ARG,
             "%s: NULL pointer", fn);
  FQ_REQUIRE(aligned16(x) && aligned16(gamma) && aligned16(route_weight) && aligned16(weight_scratch) && aligned16(y),
             FQ_ERR_ARG, "%s: misaligned pointer", fn);
  FQ_REQUIRE((reinterpret_cast<uintptr_t>(q) & 7u) == 0, FQ_ERR_ARG, "%s: q must be 8-byte aligned", fn);
  return check_launch(fq::launch_rmsnorm_router_quant(x, gamma, route_weight, weight_is_fp32 != 0, weight_scratch, y,
                                                      rstd, logits, q, s, M, (int)K, (int)N, eps, round_scale,
                                                      fp8_kind, (hipStream_t)stream),
                      fn);
}

int fq_pack_router_weight(const void* route_weight, int weight_is_fp32, void* packed, int64_t K, int64_t N,
                          void* stream) {
  const char* fn = "fq_pack_router_weight";
  FQ_REQUIRE(K > 0 && K % 128 == 0 && K <= 8192, FQ_ERR_SHAPE, "%s: K (%lld) must be a multiple of 128 up to 8192", fn,
             (long long)K);
  FQ_REQUIRE(N > 0 && N % 128 == 0 && N <= 8192, FQ_ERR_SHAPE,
             "%s: %lld router outputs (supported: multiples of 128 up to 8192)", fn, (long long)N);
  FQ_REQUIRE(route_weight && packed && aligned16(route_weight) && aligned16(packed), FQ_ERR_ARG,
             "%s: NULL or misaligned pointer", fn);
  return check_launch(fq::launch_pack_router_weight(route_weight, weight_is_fp32 != 0, packed, (int)K, (int)N,
                                                    (hipStream_t)stream),
                      fn);
}

int fq_rmsnorm_router_quant_fwd_packed(const void* x, const void* gamma, const void* packed_weight,
                                       int weight_is_fp32, void* y, float* rstd, float* logits, void* q, float* s,
                                       int64_t M, int64_t K, int64_t N, float eps, int round_scale, int fp8_kind,
                                       void* stream) {
  const char* fn = "fq_rmsnorm_router_quant_fwd_packed";
  int rc = check_common(fn, M, K, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_norm_shape(fn, M, K))) return rc;
  FQ_REQUIRE(M % 32 == 0, FQ_ERR_SHAPE, "%s: M (%lld) is not a multiple of 32", fn, (long long)M);
  FQ_REQUIRE(N > 0 && N % 128 == 0 && N <= 8192, FQ_ERR_SHAPE,
             "%s: %lld router outputs (supported: multiples of 128 up to 8192)", fn, (long long)N);
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && gamma && packed_weight && y && rstd && logits && q && s, FQ_ERR_ARG, "%s: NULL pointer", fn);
  FQ_REQUIRE(aligned16(x) && aligned16(gamma) && aligned16(packed_weight) && aligned16(y), FQ_ERR_ARG,
             "%s: misaligned pointer", fn);
  FQ_REQUIRE((reinterpret_cast<uintptr_t>(q) & 7u) == 0, FQ_ERR_ARG, "%s: q must be 8-byte aligned", fn);
  return check_launch(fq::launch_rmsnorm_router_quant_packed(x, gamma, packed_weight, weight_is_fp32 != 0, y, rstd,
                                                             logits, q, s, M, (int)K, (int)N, eps, round_scale,
                                                             fp8_kind, (hipStream_t)stream),
                      fn);
}

int fq_swiglu_quant_fwd(const void* x, void* q, float* s, void* qt, float* st, int64_t M, int64_t n,
                        int round_scale, int output_mode, int fp8_kind, void* stream) {
  const char* fn = "fq_swiglu_quant_fwd";
  int rc = check_common(fn, M, n, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_mode_ptrs(fn, output_mode, q, s, qt, st))) return rc;
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(x && aligned16(x), FQ_ERR_ARG, "%s: x is NULL or not 16-byte aligned", fn);
  const int64_t rbs = (M + 127) / 128;
  if ((rc = check_tiles(fn, rbs * (n / 128)))) return rc;
  return check_launch(fq::launch_silu_quant_fwd(x, nullptr, 0, q, s, qt, st, M, (int)n, round_scale, output_mode,
                                                fp8_kind, nullptr, 0, 0, rbs, (hipStream_t)stream),
                      fn);
}

int fq_swiglu_quant_bwd(const void* g, const void* x, void* dq, float* ds, void* dqt, float* dst, int64_t M,
                        int64_t n, int round_scale, int fp8_kind, void* stream) {
  const char* fn = "fq_swiglu_quant_bwd";
  int rc = check_common(fn, M, n, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_mode_ptrs(fn, 2, dq, ds, dqt, dst))) return rc;
  if (M == 0) return FQ_OK;
  FQ_REQUIRE(g && x && aligned16(g) && aligned16(x), FQ_ERR_ARG, "%s: NULL or misaligned input", fn);
  const int64_t rbs = (M + 127) / 128;
  if ((rc = check_tiles(fn, rbs * (n / 128)))) return rc;
  return check_launch(fq::launch_silu_quant_bwd(g, x, nullptr, 0, dq, ds, dqt, dst, nullptr, nullptr, M, (int)n,
                                                round_scale, fp8_kind, nullptr, 0, 0, rbs, (hipStream_t)stream),
                      fn);
}

}  // extern "C"

static int batched_swiglu_quant_fwd(const char* fn, const void* x, const void* weight, int weight_is_bf16,
                                    const void* counts, int counts_is_i64, int n_experts, const void* plan,
                                    const fq::PlanShape* ps, int64_t total_blocks, void* q, float* s, void* qt,
                                    float* st, int64_t M, int64_t n, int round_scale, int output_mode,
                                    int fp8_kind, void* stream) {
  int rc = check_common(fn, M, n, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_mode_ptrs(fn, output_mode, q, s, qt, st))) return rc;
  FQ_REQUIRE((plan != nullptr || n_experts >= 0) && total_blocks >= 0, FQ_ERR_SHAPE,
             "%s: negative expert/block count", fn);
  if (M == 0 || total_blocks == 0) return FQ_OK;
  FQ_REQUIRE(x && aligned16(x) && weight, FQ_ERR_ARG, "%s: NULL or misaligned input", fn);
  if ((rc = check_batch_source(fn, counts, n_experts, plan, total_blocks, M))) return rc;
  if ((rc = check_tiles(fn, total_blocks * (n / 128)))) return rc;
  return check_launch(fq::launch_silu_quant_fwd(x, weight, weight_is_bf16 != 0, q, s, qt, st, M, (int)n, round_scale,
                                                output_mode, fp8_kind, counts, counts_is_i64 != 0, n_experts,
                                                total_blocks, (hipStream_t)stream, plan, ps),
                      fn);
}

static int batched_swiglu_quant_bwd(const char* fn, const void* g, const void* x, const void* weight,
                                    int weight_is_bf16, const void* counts, int counts_is_i64, int n_experts,
                                    const void* plan, const fq::PlanShape* ps, int64_t total_blocks, void* dq,
                                    float* ds, void* dw, void* dqt, float* dst, float* dw_partials, int64_t M,
                                    int64_t n, int round_scale, int fp8_kind, void* stream) {
  int rc = check_common(fn, M, n, round_scale, fp8_kind);
  if (rc) return rc;
  if ((rc = check_mode_ptrs(fn, 2, dq, ds, dqt, dst))) return rc;
  FQ_REQUIRE((plan != nullptr || n_experts >= 0) && total_blocks >= 0, FQ_ERR_SHAPE,
             "%s: negative expert/block count", fn);
  if (M == 0 || total_blocks == 0) return FQ_OK;
  FQ_REQUIRE(g && x && aligned16(g) && aligned16(x) && weight && dw && dw_partials, FQ_ERR_ARG,
             "%s: NULL or misaligned pointer", fn);
  if ((rc = check_batch_source(fn, counts, n_experts, plan, total_blocks, M))) return rc;
  if ((rc = check_tiles(fn, total_blocks * (n / 128)))) return rc;
  return check_launch(fq::launch_silu_quant_bwd(g, x, weight, weight_is_bf16 != 0, dq, ds, dqt, dst, dw_partials, dw,
                                                M, (int)n, round_scale, fp8_kind, counts, counts_is_i64 != 0,
                                                n_experts, total_blocks, (hipStream_t)stream, plan, ps),
                      fn);
}

extern "C" {

int fq_batched_swiglu_quant_fwd(const void* x, const void* weight, int weight_is_bf16, const void* counts,
                                int counts_is_i64, int n_experts, int64_t total_blocks, void* q, float* s,
                                void* qt, float* st, int64_t M, int64_t n, int round_scale, int output_mode,
                                int fp8_kind, void* stream) {
  return batched_swiglu_quant_fwd("fq_batched_swiglu_quant_fwd", x, weight, weight_is_bf16, counts, counts_is_i64,
                                  n_experts, nullptr, nullptr, total_blocks, q, s, qt, st, M, n, round_scale,
                                  output_mode, fp8_kind, stream);
}

int fq_batched_swiglu_quant_fwd_planned(const void* x, const void* weight, int weight_is_bf16, const void* plan,
                                        const int64_t* shape, void* q, float* s, void* qt, float* st, int64_t M,
                                        int64_t n, int round_scale, int output_mode, int fp8_kind, void* stream) {
  const char* fn = "fq_batched_swiglu_quant_fwd_planned";
  fq::PlanShape ps;
  int rc = check_plan_shape(fn, shape, 1, &ps);
  if (rc) return rc;
  FQ_REQUIRE(plan != nullptr || M == 0 || shape[0] == 0, FQ_ERR_ARG, "%s: plan NULL", fn);
  return batched_swiglu_quant_fwd(fn, x, weight, weight_is_bf16, nullptr, 0, 0, plan, &ps, shape[0], q, s, qt, st, M,
                                  n, round_scale, output_mode, fp8_kind, stream);
}

int fq_batched_swiglu_quant_bwd(const void* g, const void* x, const void* weight, int weight_is_bf16,
                                const void* counts, int counts_is_i64, int n_experts, int64_t total_blocks,
                                void* dq, float* ds, void* dw, void* dqt, float* dst, float* dw_partials,
                                int64_t M, int64_t n, int round_scale, int fp8_kind, void* stream) {
  return batched_swiglu_quant_bwd("fq_batched_swiglu_quant_bwd", g, x, weight, weight_is_bf16, counts, counts_is_i64,
                                  n_experts, nullptr, nullptr, total_blocks, dq, ds, dw, dqt, dst, dw_partials, M, n,
                                  round_scale, fp8_kind, stream);
}

int fq_batched_swiglu_quant_bwd_planned(const void* g, const void* x, const void* weight, int weight_is_bf16,
                                        const void* plan, const int64_t* shape, void* dq, float* ds, void* dw,
                                        void* dqt, float* dst, float* dw_partials, int64_t M, int64_t n,
                                        int round_scale, int fp8_kind, void* stream) {
  const char* fn = "fq_batched_swiglu_quant_bwd_planned";
  fq::PlanShape ps;
  int rc = check_plan_shape(fn, shape, 1, &ps);
  if (rc) return rc;
  FQ_REQUIRE(plan != nullptr || M == 0 || shape[0] == 0, FQ_ERR_ARG, "%s: plan NULL", fn);
  return batched_swiglu_quant_bwd(fn, g, x, weight, weight_is_bf16, nullptr, 0, 0, plan, &ps, shape[0], dq, ds, dw, dqt,
                                  dst, dw_partials, M, n, round_scale, fp8_kind, stream);
}

}  // extern "C"
