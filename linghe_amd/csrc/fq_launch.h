// Internal launcher prototypes shared between the kernel translation units and
// the C-ABI layer.  Everything here takes raw device pointers and a stream and
// only enqueues work.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace fq {

// Sizes of the three sections of a per-expert tile plan: row blocks worked on unpacked, last blocks
// of 33..64 rows, last blocks of at most 32 rows (counted on the host from its copy of the counts)
struct PlanShape {
  int64_t unpacked, packed2, packed4;
  int pad;  // 1: experts back to back; 16: every expert's region of the outputs rounded up to 16 rows
  int64_t blocks() const { return unpacked + packed2 + packed4; }
};

hipError_t launch_blockwise_quant(const void* x, void* q, float* s, void* qt, float* st, int64_t M, int N,
                                  int round_scale, int mode, int kind, const void* counts, int counts_i64,
                                  int n_experts, int64_t row_blocks, hipStream_t stream, const void* plan = nullptr,
                                  const PlanShape* ps = nullptr);

hipError_t launch_pad_permute_quant(const void* x, const void* indices, const void* probs, int probs_bf16,
                                    void* prob_out, void* q, float* s, void* qt, float* st, int64_t src_rows,
                                    int64_t M, int N, int round_scale, int kind, const void* counts, int counts_i64,
                                    int n_experts, int64_t row_blocks, hipStream_t stream, const void* plan = nullptr,
                                    const PlanShape* ps = nullptr);

hipError_t launch_silu_quant_fwd(const void* x, const void* weight, int weight_bf16, void* q, float* s, void* qt,
                                 float* st, int64_t M, int n, int round_scale, int mode, int kind,
                                 const void* counts, int counts_i64, int n_experts, int64_t row_blocks,
                                 hipStream_t stream, const void* plan = nullptr, const PlanShape* ps = nullptr);

hipError_t launch_silu_quant_bwd(const void* g, const void* x, const void* weight, int weight_bf16, void* q,
                                 float* s, void* qt, float* st, float* dw_part, void* dw, int64_t M, int n,
                                 int round_scale, int kind, const void* counts, int counts_i64, int n_experts,
                                 int64_t row_blocks, hipStream_t stream, const void* plan = nullptr,
                                  const PlanShape* ps = nullptr);

// Per-expert launches with `plan` (expert_plan_bytes(ps) bytes of device memory filled by
// launch_expert_plan from the same counts) and its shape read their tile from it instead of
// scanning the counts; counts may then be NULL and row_blocks is not used.
PlanShape expert_plan_shape(const int64_t* host_counts, int n_experts, int pad);
int64_t expert_plan_bytes(const PlanShape& ps);
hipError_t launch_expert_plan(const void* counts, int counts_i64, int n_experts, const PlanShape& ps, void* plan,
                              hipStream_t stream);

// RMSNorm + quant with both outputs runs the statistic pass (launch_rmsnorm_fwd, quant = 2) and then
// the tile kernel (launch_rmsnorm_quant_tile, mode 2); for these shapes both hand XCD X the X-th
// eighth of the rows, so that the second pass finds in its XCD's L2 what the first one left there
bool rmsnorm_passes_by_xcd(int64_t M, int n);

hipError_t launch_rmsnorm_quant_tile(const void* x, const void* gamma, const float* rstd, void* q, float* s,
                                     void* qt, float* st, int64_t M, int n, int round_scale, int mode, int kind,
                                     hipStream_t stream);

hipError_t launch_rmsnorm_fwd(const void* x, const void* gamma, void* out, float* scale, float* rstd, int64_t M,
                              int n, float eps, int reuse_rstd, int quant, int round_scale, int kind,
                              hipStream_t stream);

int64_t rmsnorm_bwd_partials(int64_t M);

hipError_t launch_rmsnorm_bwd(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx,
                              float* dgamma, float* dg_part, int64_t n_partials, int64_t M, int n, float eps,
                              hipStream_t stream);

// the same with the dgamma partial rows in the library's own fixed device array
int64_t rmsnorm_bwd_static_scratch_bytes();
hipError_t launch_rmsnorm_bwd_static(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx,
                                     float* dgamma, int64_t M, int n, float eps, hipStream_t stream);

hipError_t launch_group_quant(const void* x, void* q, float* s, int64_t n_groups, int round_scale, int kind,
                              hipStream_t stream);

// bf16 SwiGLU rows (no quantisation) and the 128x128 weight block quantiser
hipError_t launch_swiglu_rows_fwd(const void* x, const void* weight, int weight_bf16, void* out, int64_t M, int n,
                                  hipStream_t stream);
hipError_t launch_swiglu_rows_bwd(const void* g, const void* x, const void* weight, int weight_bf16, void* dx,
                                  void* dw, int64_t M, int n, hipStream_t stream);
hipError_t launch_block_quant(const void* x, void* q, float* s, int64_t M, int N, int round_scale, int kind,
                              hipStream_t stream);

// RMSNorm + router GEMM + 1x128 quant; M a multiple of 32, N a multiple of 128, the router
// weight bf16 or fp32; wpacked: rmsnorm_router_scratch_bytes() bytes
int64_t rmsnorm_router_scratch_bytes(int K, int N, int weight_fp32);
hipError_t launch_rmsnorm_router_quant(const void* x, const void* gamma, const void* wr, int weight_fp32,
                                       void* wpacked, void* y, float* rstd, float* logits, void* q, float* s,
                                       int64_t M, int K, int N, float eps, int round_scale, int kind,
                                       hipStream_t stream);

// the two halves of launch_rmsnorm_router_quant: re-order the weight (once per weight update),
// run on the re-ordered weight
hipError_t launch_pack_router_weight(const void* wr, int weight_fp32, void* wpacked, int K, int N, hipStream_t stream);
hipError_t launch_rmsnorm_router_quant_packed(const void* x, const void* gamma, const void* wpacked,
                                              int weight_fp32, void* y, float* rstd, float* logits, void* q,
                                              float* s, int64_t M, int K, int N, float eps, int round_scale,
                                              int kind, hipStream_t stream);

// measurement aid: read read_bytes from src, write write_bytes to dst (both multiples of 16), no arithmetic;
// chunks_per_lane 4 / 8 / 16, workgroups (0: one step each), order 0 / 1 / 2, hint on loads / stores
hipError_t launch_stream_rw(const void* src, int64_t read_bytes, void* dst, int64_t write_bytes, void* sink,
                            int chunks_per_lane, int64_t workgroups, int order, int nt_loads, int nt_stores,
                            hipStream_t stream);

}  // namespace fq
