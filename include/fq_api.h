/* C ABI of libfq_gfx950.so: the MI355X (gfx950) fused blockwise-FP8 quantisation
 * kernels.  Each entry point replaces the Triton launch(es) made by one Python
 * wrapper of the reference (path:line of the wrapper is cited at each
 * declaration; paths are relative to the reference checkout).
 *
 * Conventions
 *  - every pointer is a DEVICE pointer on the current HIP device; the library
 *    never allocates or frees device memory and never synchronises;
 *  - `stream` is a hipStream_t passed as void* (NULL = the default stream);
 *    calls only enqueue work on it;
 *  - bf16 inputs are row-major and contiguous, 16-byte aligned;
 *  - fp8 outputs are raw bytes (OCP e4m3fn when fp8_kind == FQ_E4M3, OCP e5m2
 *    when FQ_E5M2); scales are fp32 "scale_inv": value ~= code * scale,
 *    scale = max(amax/fmax, 1e-30), rounded up to a power of two if round_scale;
 *  - output_mode: 0 = row-wise (1x128) outputs only, 1 = transposed (128x1)
 *    outputs only, 2 = both.  Outputs a mode does not produce may be NULL;
 *  - return value: FQ_OK or a negative FQ_ERR_* code; fq_last_error() gives
 *    the message of the calling thread's last failure.
 *
 * Layouts (nb = n/128, rb = r/128, b = c/128; element offsets):
 *   single matrix: q[r*n + c], s[b*M + r], qt[c*M + r], st[rb*n + c]
 *   per expert e (rows si..si+ce, tb = sum of ceil(c_e'/128) over e' < e):
 *     q[(si+i)*n + c], s[si*nb + b*ce + i], qt[si*n + c*ce + i],
 *     st[(tb + i/128)*n + c]
 */
#ifndef FQ_API_H_
#define FQ_API_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FQ_OK 0
#define FQ_ERR_ARG (-1)     /* null pointer, bad flag, misaligned pointer */
#define FQ_ERR_SHAPE (-2)   /* shape outside what the kernels support */
#define FQ_ERR_LAUNCH (-3)  /* HIP reported a launch failure */

#define FQ_E4M3 0
#define FQ_E5M2 1
/* fq_group_quant only: e5m2 codes, scale = amax/448 (what the reference's group
 * quantiser computes when its dtype argument is float8_e5m2,
 * linghe/quant/group.py:27,57) */
#define FQ_E5M2_MAX448 2

/* library version (major*10000 + minor*100 + patch) */
int fq_version(void);
/* message of this thread's last failing call ("" if none) */
const char* fq_last_error(void);

/* Measurement aid with no counterpart in the reference: a kernel that reads
 * read_bytes from src and writes write_bytes to dst (multiples of 16; the two
 * need not be equal, either may be 0) with the 16-byte accesses of the product
 * kernels and no arithmetic.  sink: 16 bytes of device memory that are never
 * written in practice (they keep the loads alive).  nontemporal != 0 puts the
 * streaming hint on loads and stores.  bench.py times it on each
 * configuration's own byte counts (the measured ceiling) and the profiler
 * counters are calibrated on it. */
int fq_stream_rw(const void* src, int64_t read_bytes, void* dst, int64_t write_bytes, void* sink, int nontemporal,
                 void* stream);
/* The same kernel in its variants (no counterpart in the reference either): chunks_per_lane = 16-byte
 * chunks in flight per lane (4, 8 or 16); workgroups = how many to launch (0: one step of
 * 256 * chunks_per_lane chunks per workgroup, else each walks several); order 0 = interleaved steps,
 * 1 = one contiguous run per workgroup, 2 = the same with one contiguous eighth of the buffers per XCD,
 * 3 = interleaved steps shaped as the tile kernels' accesses (a step is 16 * chunks_per_lane rows x 256 bytes
 * of a matrix with 4096-byte rows);
 * nt_loads / nt_stores put the streaming hint on loads / stores.  fq_stream_rw is
 * (4, 16384, 0, nontemporal, nontemporal).  The measured ceiling is the fastest variant. */
int fq_stream_rw_variant(const void* src, int64_t read_bytes, void* dst, int64_t write_bytes, void* sink,
                         int chunks_per_lane, int64_t workgroups, int order, int nt_loads, int nt_stores,
                         void* stream);

/* triton_blockwise_quant, linghe/quant/block.py:129-170.
 * x bf16 [M,N], N % 128 == 0.  q [M,N], s [N/128, M], qt [N, M], st [ceil(M/128), N]. */
int fq_blockwise_quant(const void* x, void* q, float* s, void* qt, float* st, int64_t M, int64_t N,
                       int round_scale, int output_mode, int fp8_kind, void* stream);

/* triton_batch_blockwise_quant, linghe/quant/block.py:251-297.
 * counts: device int32/int64 [n_experts]; total_blocks = sum ceil(count_e/128)
 * computed by the caller from its host-side copy of the counts. */
int fq_batched_blockwise_quant(const void* x, const void* counts, int counts_is_i64, int n_experts,
                               int64_t total_blocks, void* q, float* s, void* qt, float* st, int64_t M,
                               int64_t N, int round_scale, int fp8_kind, void* stream);

/* The per-expert entry points find every workgroup's tile by a prefix scan over
 * the device-side counts.  A caller that runs several of them on the same
 * counts (the forward, the backward and the quantiser of one MoE layer) can
 * have that scan done once, and the launches sized for exactly the workgroups
 * that have a tile:
 *  - fq_expert_plan_shape (host only, no GPU work) reads the caller's host-side
 *    copy of the counts - what the reference takes as `splits`
 *    (linghe/utils/silu.py:826, :838: "batch mode need splits to launch
 *    kernels") - and fills shape[0..4]: the number of 128-row blocks
 *    (= total_blocks of the other forms), how many of them are worked on
 *    whole, in halves and in quarters, and `pad`: 1 for the layouts in which
 *    the experts lie back to back (SwiGLU, blockwise quantiser), 16 for the
 *    gather + pad + quant layout (every expert's region rounded up to 16 rows);
 *  - fq_build_expert_plan writes one 20-byte record per row block from the
 *    DEVICE-side counts into `plan` (fq_expert_plan_bytes(shape) bytes of
 *    device memory, 16-byte aligned);
 *  - the *_planned forms of the entry points take plan and shape in place of
 *    counts, n_experts and total_blocks.  Their outputs are identical to those
 *    of the forms that take the counts.  A plan addresses at most 2^31 - 1 rows
 *    and serves the entry points of its own `pad` only.
 * Where host and device counts disagree the row blocks concerned are left out,
 * as in the other forms. */
int fq_expert_plan_shape(const int64_t* host_counts, int n_experts, int pad, int64_t* shape);
int64_t fq_expert_plan_bytes(const int64_t* shape);
int fq_build_expert_plan(const void* counts, int counts_is_i64, int n_experts, const int64_t* shape, void* plan,
                         void* stream);

/* fq_batched_blockwise_quant with the tiles read from a plan. */
int fq_batched_blockwise_quant_planned(const void* x, const void* plan, const int64_t* shape, void* q, float* s,
                                       void* qt, float* st, int64_t M, int64_t N, int round_scale, int fp8_kind,
                                       void* stream);

/* triton_batch_block_pad_permute_with_indices, linghe/utils/gather.py:960-1113
 * (kernel :840-957).  x bf16 [src_rows, N]; indices int32 [M], M = sum of the
 * counts each rounded up to 16: expert e's region of the outputs starts at the
 * sum of the rounded counts before it, holds x[indices[start + i]] for
 * i < count_e and zero rows up to its rounded count pc_e, and is laid out as
 * q[(start+i)*N + c], s[start*nb + b*pc_e + i], qt[start*N + c*pc_e + i],
 * st[(tb + i/128)*N + c].  probs (fp32 or bf16 [src_rows, n_experts], may be
 * NULL together with prob_out): prob_out[start + i] = probs[row, e], 0 in the
 * padding.  Indices outside [0, src_rows) read as zero rows. */
int fq_batched_pad_permute_quant(const void* x, const void* counts, int counts_is_i64, int n_experts,
                                 int64_t total_blocks, const void* indices, const void* probs, int probs_is_bf16,
                                 void* prob_out, void* q, float* s, void* qt, float* st, int64_t src_rows,
                                 int64_t M, int64_t N, int round_scale, int fp8_kind, void* stream);

/* fq_batched_pad_permute_quant with the tiles read from a plan of pad 16
 * (n_experts: the width of probs). */
int fq_batched_pad_permute_quant_planned(const void* x, const void* plan, const int64_t* shape, int n_experts,
                                         const void* indices, const void* probs, int probs_is_bf16, void* prob_out,
                                         void* q, float* s, void* qt, float* st, int64_t src_rows, int64_t M,
                                         int64_t N, int round_scale, int fp8_kind, void* stream);

/* triton_block_quant, linghe/quant/block.py:32-62 (kernel :11-29): one scale per
 * 128x128 block of a weight.  x bf16 [M,N], M and N multiples of 128;
 * q [M,N], s [M/128, N/128]. */
int fq_block_quant(const void* x, void* q, float* s, int64_t M, int64_t N, int round_scale, int fp8_kind,
                   void* stream);

/* triton_weighted_silu_forward, linghe/utils/silu.py:98-127 (kernel :63-94).
 * x bf16 [M, 2n] (gate | up), weight [M] fp32 or bf16 or NULL; out bf16 [M, n]. */
int fq_swiglu_fwd(const void* x, const void* weight, int weight_is_bf16, void* out, int64_t M, int64_t n,
                  void* stream);

/* triton_weighted_silu_backward, linghe/utils/silu.py:177-210 (kernel :130-174).
 * g bf16 [M,n], x bf16 [M,2n]; dx bf16 [M,2n] (dx1 | dx2); dw [M] in the weight's
 * dtype, NULL together with weight. */
int fq_swiglu_bwd(const void* g, const void* x, const void* weight, int weight_is_bf16, void* dx, void* dw,
                  int64_t M, int64_t n, void* stream);

/* triton_group_quant, linghe/quant/group.py:40-63.  s is [M, N/128] row-major. */
int fq_group_quant(const void* x, void* q, float* s, int64_t M, int64_t N, int round_scale, int fp8_kind,
                   void* stream);

/* triton_rms_norm_forward, linghe/utils/norm.py:58-93.  out bf16 [M,n].
 * reuse_rstd != 0: rstd [M] is an input, else it is written. */
int fq_rmsnorm_fwd(const void* x, const void* gamma, void* out, float* rstd, int64_t M, int64_t n, float eps,
                   int reuse_rstd, void* stream);

/* number of fp32 [n] partial rows fq_rmsnorm_bwd needs in dgamma_partials */
int64_t fq_rmsnorm_bwd_num_partials(int64_t M, int64_t n);

/* triton_rms_norm_backward, linghe/utils/norm.py:144-179.
 * rstd may be NULL (recomputed).  dx bf16 [M,n], dgamma fp32 [n],
 * dgamma_partials fp32 [n_partials, n] scratch (the reference's tmp_dw). */
int fq_rmsnorm_bwd(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx, float* dgamma,
                   float* dgamma_partials, int64_t n_partials, int64_t M, int64_t n, float eps, void* stream);

/* fq_rmsnorm_bwd for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has
 * no counterpart in the reference.  Same inputs, outputs and results as
 * fq_rmsnorm_bwd, but the dgamma partial rows live in a fixed 16 MiB array in
 * the library's own device memory (one copy per GPU, held until the process
 * ends) instead of a caller-provided buffer; the call allocates and frees
 * nothing.  n <= 8192 as for every RMSNorm entry point; anything whose partial
 * rows would not fit the array is refused with FQ_ERR_SHAPE.  Calls on one GPU
 * share that GPU's array: calls that may overlap in time (different streams
 * without ordering) race.  The array's device address is looked up on the first
 * call on each device. */
int fq_rmsnorm_bwd_noalloc(const void* dy, const void* x, const void* gamma, const float* rstd, void* dx,
                           float* dgamma, int64_t M, int64_t n, float eps, void* stream);

/* triton_rms_norm_and_block_quant_forward, linghe/utils/norm.py:343-502.
 * mode 0: writes q, s, rstd.  mode 1: reads rstd, writes qt, st.
 * mode 2: writes q, s, rstd, qt, st; runs as two launches on `stream` - the
 * row statistic (x read once, rstd written), then the 128x128 tile kernel that
 * reads x again (the second read is served by the memory-side cache when x fits
 * it) and emits both layouts. */
int fq_rmsnorm_quant_fwd(const void* x, const void* gamma, void* q, float* s, float* rstd, void* qt, float* st,
                         int64_t M, int64_t n, float eps, int round_scale, int output_mode, int fp8_kind,
                         void* stream);

/* bytes of weight_scratch fq_rmsnorm_router_quant_fwd needs: N*K*2 for a bf16 router
 * weight, N*K*4 for an fp32 one (0 for sizes the entry point refuses) */
int64_t fq_rmsnorm_router_scratch_bytes(int64_t K, int64_t N, int weight_is_fp32);

/* triton_rms_norm_fp32_gemm_block_quant_forward, output_mode 0,
 * linghe/utils/norm.py:690-784 (kernel :616-687).  x bf16 [M,K], gamma bf16 [K],
 * route_weight [N,K] bf16 or (weight_is_fp32) fp32, N a multiple of 128 up to
 * 8192, M a multiple of 32.  Writes y bf16 [M,K] (the normalised x), rstd [M],
 * logits fp32 [M,N] = y_fp32 @ route_weight^T, q [M,K] and s [K/128, M].
 * The product has fp32-GEMM accuracy: y, and an fp32 weight, enter the matrix
 * cores as two bf16 terms each (16 significant bits; the reference's tl.dot on
 * fp32 operands uses fewer).  weight_scratch: fq_rmsnorm_router_scratch_bytes()
 * bytes the call overwrites (the weight re-ordered for the matrix cores).
 * (output_mode 1 of the reference is fq_rmsnorm_quant_fwd with output_mode 1.) */
int fq_rmsnorm_router_quant_fwd(const void* x, const void* gamma, const void* route_weight, int weight_is_fp32,
                                void* weight_scratch, void* y, float* rstd, float* logits, void* q, float* s,
                                int64_t M, int64_t K, int64_t N, float eps, int round_scale, int fp8_kind,
                                void* stream);

/* The two halves of fq_rmsnorm_router_quant_fwd, for callers that keep the re-ordered weight
 * between weight updates (the reference re-reads route_weight on every call,
 * linghe/utils/norm.py:736-784; a router weight changes once per optimiser step).
 * fq_pack_router_weight re-orders route_weight [N,K] (bf16, or fp32 split into two bf16
 * planes) into `packed` (fq_rmsnorm_router_scratch_bytes() bytes);
 * fq_rmsnorm_router_quant_fwd_packed is fq_rmsnorm_router_quant_fwd on that buffer, with the
 * weight_is_fp32 it was packed with.  Results are bit-identical to the one-call form. */
int fq_pack_router_weight(const void* route_weight, int weight_is_fp32, void* packed, int64_t K, int64_t N,
                          void* stream);
int fq_rmsnorm_router_quant_fwd_packed(const void* x, const void* gamma, const void* packed_weight,
                                       int weight_is_fp32, void* y, float* rstd, float* logits, void* q, float* s,
                                       int64_t M, int64_t K, int64_t N, float eps, int round_scale, int fp8_kind,
                                       void* stream);

/* triton_silu_and_block_quant_forward, linghe/utils/silu.py:279-335.
 * x bf16 [M, 2n] (gate | up).  Outputs as fq_blockwise_quant with N = n. */
int fq_swiglu_quant_fwd(const void* x, void* q, float* s, void* qt, float* st, int64_t M, int64_t n,
                        int round_scale, int output_mode, int fp8_kind, void* stream);

/* triton_silu_and_block_quant_backward, linghe/utils/silu.py:424-464.
 * g bf16 [M,n], x bf16 [M,2n].  dq [M,2n] (dx1|dx2), ds [2n/128, M],
 * dqt [2n, M], dst [ceil(M/128), 2n]. */
int fq_swiglu_quant_bwd(const void* g, const void* x, void* dq, float* ds, void* dqt, float* dst, int64_t M,
                        int64_t n, int round_scale, int fp8_kind, void* stream);

/* triton_batch_weighted_silu_and_block_quant_forward, linghe/utils/silu.py:797-950.
 * weight [M] fp32 (or bf16 when weight_is_bf16), per-expert packed outputs. */
int fq_batched_swiglu_quant_fwd(const void* x, const void* weight, int weight_is_bf16, const void* counts,
                                int counts_is_i64, int n_experts, int64_t total_blocks, void* q, float* s,
                                void* qt, float* st, int64_t M, int64_t n, int round_scale, int output_mode,
                                int fp8_kind, void* stream);

/* triton_batch_weighted_silu_and_block_quant_backward, linghe/utils/silu.py:1293-1393.
 * dw [M] in the weight's dtype; dw_partials: M * n/128 floats of scratch (the
 * reference's dws; what it holds afterwards is not part of the interface). */
int fq_batched_swiglu_quant_bwd(const void* g, const void* x, const void* weight, int weight_is_bf16,
                                const void* counts, int counts_is_i64, int n_experts, int64_t total_blocks,
                                void* dq, float* ds, void* dw, void* dqt, float* dst, float* dw_partials,
                                int64_t M, int64_t n, int round_scale, int fp8_kind, void* stream);

/* The two entry points above with the tiles read from a plan
 * (fq_build_expert_plan). */
int fq_batched_swiglu_quant_fwd_planned(const void* x, const void* weight, int weight_is_bf16, const void* plan,
                                        const int64_t* shape, void* q, float* s, void* qt, float* st, int64_t M,
                                        int64_t n, int round_scale, int output_mode, int fp8_kind, void* stream);
int fq_batched_swiglu_quant_bwd_planned(const void* g, const void* x, const void* weight, int weight_is_bf16,
                                        const void* plan, const int64_t* shape, void* dq, float* ds, void* dw,
                                        void* dqt, float* dst, float* dw_partials, int64_t M, int64_t n,
                                        int round_scale, int fp8_kind, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FQ_API_H_ */
