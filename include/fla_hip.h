/*
 * fla_hip.h - C ABI of libfla_hip.so, the gfx950 (MI355X) linear-attention
 * operator library.
 *
 * Every operator of the reference's custom-op library is exposed there as a
 * two-phase pair
 *     aclnn<Op>GetWorkspaceSize(<inputs>, <attrs>, <outputs>, uint64_t *ws, aclOpExecutor **)
 *     aclnn<Op>(void *ws, uint64_t ws_size, aclOpExecutor *, aclrtStream)
 * bound from Python with ctypes
 * (torch_custom/fla_npu/fla_npu/ops/ascendc/_runtime.py:388-429).  This library
 * keeps the argument order of each aclnn prototype but is stateless: there is
 * no executor object, so phase two takes the operands again.
 *
 *     int fla_<op>_get_workspace_size(<operands>, uint64_t *workspace_size);
 *     int fla_<op>(<operands>, void *workspace, uint64_t workspace_size, void *stream);
 *
 * Contract (mirrors _runtime.py:191-207,413-428,463-482):
 *   - the caller owns every buffer: inputs, outputs and the workspace; the
 *     library never allocates or frees device memory and keeps no pointer
 *     after a call returns;
 *   - an absent optional tensor / int array is a NULL pointer;
 *   - host int arrays (cu_seqlens, chunk_indices, ...) are consumed before the
 *     call returns;
 *   - `stream` is a hipStream_t; kernels are enqueued on it and the call
 *     returns without synchronising;
 *   - return value 0 is success; any other value is an fla_status and
 *     fla_last_error() describes it (thread-local string);
 *   - all tensors of one call live on the current HIP device.
 */
#ifndef FLA_HIP_H_
#define FLA_HIP_H_

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLA_MAX_DIMS 8

typedef enum fla_dtype {
    FLA_F32 = 0,
    FLA_F16 = 1,
    FLA_BF16 = 2,
    FLA_I32 = 3,
    FLA_I64 = 4
} fla_dtype;

typedef enum fla_status {
    FLA_OK = 0,
    FLA_ERR_NULL = 1,        /* a required pointer is NULL                      */
    FLA_ERR_DTYPE = 2,       /* unsupported dtype or dtype combination          */
    FLA_ERR_SHAPE = 3,       /* rank / extent / stride violates the op contract */
    FLA_ERR_UNSUPPORTED = 4, /* valid request this build has no kernel for      */
    FLA_ERR_WORKSPACE = 5,   /* workspace missing or smaller than required      */
    FLA_ERR_LAUNCH = 6,      /* the HIP runtime refused the launch              */
    FLA_ERR_METADATA = 7,    /* cu_seqlens / chunk_indices are inconsistent     */
    FLA_ERR_HOST = 8         /* host-side failure (allocation, lock) in the call */
} fla_status;

/* Replaces the opaque aclTensor built by aclCreateTensor(shape, ndim, dtype,
 * strides, offset, format, storage_shape, n, storage_ptr) (_runtime.py:239-249).
 * `data` already includes the storage offset; strides are in elements. */
typedef struct fla_tensor {
    void *data;
    int32_t dtype; /* fla_dtype */
    int32_t ndim;
    int64_t shape[FLA_MAX_DIMS];
    int64_t stride[FLA_MAX_DIMS];
} fla_tensor;

/* Replaces aclIntArray (aclCreateIntArray, _runtime.py:259-273): host int64 values. */
typedef struct fla_int_array {
    const int64_t *data;
    uint64_t size;
} fla_int_array;

const char *fla_last_error(void);
/* ABI version of this header; bumped on any signature change. */
int fla_abi_version(void);

/* Per-kernel timing, no counterpart in the reference (it profiles from outside with msopprof,
 * fla/ops/ascendc/kda/KDA_FORWARD_VALIDATION_REPORT.md:77-84).  After fla_profile_enable(1) every kernel
 * launch is bracketed by two HIP events on its launch stream.  fla_profile_report waits for them, writes
 * one "name count total_ms" line per kernel name into buf (NUL-terminated, truncated to cap bytes),
 * clears the records and returns the number of kernel names.  Process-wide; not for use under stream
 * capture. */
void fla_profile_enable(int on);
int fla_profile_report(char *buf, uint64_t cap);

/* ------------------------------------------------------------------------
 * chunk_local_cumsum - replaces aclnnChunkLocalCumsum
 * (_aclnn_ctypes.py:875-904; chunk_local_cumsum/README.md:7-24).
 * g, out: [B,H,T] or [B,H,T,K] contiguous, head_first must be true.
 * ------------------------------------------------------------------------ */
int fla_chunk_local_cumsum_get_workspace_size(
    const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices_out,
    int64_t chunk_size, bool reverse, double scale, bool head_first, const char *output_dtype,
    const fla_tensor *out, uint64_t *workspace_size);
int fla_chunk_local_cumsum(
    const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices_out,
    int64_t chunk_size, bool reverse, double scale, bool head_first, const char *output_dtype,
    const fla_tensor *out, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * chunk_scaled_dot_kkt - replaces aclnnChunkScaledDotKkt (_aclnn_ctypes.py:907-936).
 * k [B,Hk,T,K] bf16; g, beta [B,Hv,T] f32; out A [B,Hv,T,C] f32.
 * ------------------------------------------------------------------------ */
int fla_chunk_scaled_dot_kkt_get_workspace_size(
    const fla_tensor *k, const fla_tensor *g, const fla_tensor *beta,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size,
    const fla_tensor *out, uint64_t *workspace_size);
int fla_chunk_scaled_dot_kkt(
    const fla_tensor *k, const fla_tensor *g, const fla_tensor *beta,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size,
    const fla_tensor *out, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * chunk_scaled_dot_kkt_inverse - no counterpart in the reference: the two operators above and below in one
 * launch, for callers that only want the inverse (the backward's recompute).  Same operands as
 * chunk_scaled_dot_kkt; out = (I + A)^-1 [B,Hv,T,64] in the element type of k, contiguous; 64-token chunks.
 * The result equals solve_tri(chunk_scaled_dot_kkt(...)) bit for bit.
 * ------------------------------------------------------------------------ */
int fla_chunk_scaled_dot_kkt_inverse_get_workspace_size(
    const fla_tensor *k, const fla_tensor *g, const fla_tensor *beta,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size,
    const fla_tensor *out, uint64_t *workspace_size);
int fla_chunk_scaled_dot_kkt_inverse(
    const fla_tensor *k, const fla_tensor *g, const fla_tensor *beta,
    const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, int64_t chunk_size,
    const fla_tensor *out, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * solve_tri - replaces aclnnSolveTri (_aclnn_ctypes.py:1786-1800):
 * out = (I + x)^-1 per C x C chunk block, x strictly lower triangular.
 * layout "bnsd": x [B,H,T,C]; "bsnd": x [B,T,H,C]; "tnd" / "ntd" without the batch
 * dimension; C (the last dimension) in {16, 32, 64, 128}; bf16 or fp16 in and out,
 * or f32 in (rounded to the dtype of out while it is loaded).
 * ------------------------------------------------------------------------ */
int fla_solve_tri_get_workspace_size(
    const fla_tensor *x, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    const char *layout, const fla_tensor *out, uint64_t *workspace_size);
int fla_solve_tri(
    const fla_tensor *x, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    const char *layout, const fla_tensor *out, void *workspace, uint64_t workspace_size,
    void *stream);

/* ------------------------------------------------------------------------
 * recompute_w_u_fwd - replaces aclnnRecomputeWUFwd (_aclnn_ctypes.py:618-651).
 * k [B,Hk,T,K], v [B,Hv,T,V] bf16; beta, g [B,Hv,T] f32; A [B,Hv,T,C] bf16;
 * gk must be NULL.  Outputs w [B,Hv,T,K], u [B,Hv,T,V] bf16.
 * ------------------------------------------------------------------------ */
int fla_recompute_w_u_fwd_get_workspace_size(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A,
    const fla_tensor *g, const fla_tensor *gk, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *w,
    const fla_tensor *u, uint64_t *workspace_size);
int fla_recompute_w_u_fwd(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A,
    const fla_tensor *g, const fla_tensor *gk, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *w,
    const fla_tensor *u, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * chunk_gated_delta_rule_fwd_h - replaces aclnnChunkGatedDeltaRuleFwdH
 * (_aclnn_ctypes.py:552-615).  k [B,Hk,T,K], w [B,Hv,T,K], u [B,Hv,T,V] bf16;
 * g [B,Hv,T] f32 (chunk-cumsummed, natural log) and / or gk [B,Hv,T,K] f32
 * (chunk-cumsummed per-channel gate, log2 units; k then already carries
 * 2^{gk_last - gk}; chunk_size 64); initial_state [N,Hv,K,V] f32 or NULL.  Outputs h [B,Hv,NT,K,V] bf16 (state at chunk
 * start), v_new [B,Hv,T,V] bf16, final_state [N,Hv,K,V] f32 (NULL unless
 * output_final_state).
 * ------------------------------------------------------------------------ */
int fla_chunk_gated_delta_rule_fwd_h_get_workspace_size(
    const fla_tensor *k, const fla_tensor *w, const fla_tensor *u, const fla_tensor *g,
    const fla_tensor *gk, const fla_tensor *initial_state, bool output_final_state,
    int64_t chunk_size, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    bool state_v_first, const fla_tensor *h, const fla_tensor *v_new,
    const fla_tensor *final_state, uint64_t *workspace_size);
int fla_chunk_gated_delta_rule_fwd_h(
    const fla_tensor *k, const fla_tensor *w, const fla_tensor *u, const fla_tensor *g,
    const fla_tensor *gk, const fla_tensor *initial_state, bool output_final_state,
    int64_t chunk_size, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    bool state_v_first, const fla_tensor *h, const fla_tensor *v_new,
    const fla_tensor *final_state, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * chunk_fwd_o - replaces aclnnChunkFwdO (_aclnn_ctypes.py:517-549).
 * q,k [B,Hk,T,K], v (= v_new) [B,Hv,T,V], h [B,Hv,NT,K,V] bf16; g [B,Hv,T] f32.
 * Output o [B,Hv,T,V] bf16.
 * ------------------------------------------------------------------------ */
int fla_chunk_fwd_o_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *h,
    const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    double scale, int64_t chunk_size, const fla_tensor *out, uint64_t *workspace_size);
int fla_chunk_fwd_o(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *h,
    const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    double scale, int64_t chunk_size, const fla_tensor *out, void *workspace,
    uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * gdn_chunk_fwd - the whole chunk forward in one call.  Replaces the Python
 * composition flash_chunk_gated_delta_rule_fwd
 * (examples/flash_gated_delta_rule.py:796-881), which issues the six ops
 * above plus transposes.  q,k [B,Hk,T,K], v [B,Hv,T,V] bf16 (any strides with
 * unit innermost stride); g (raw per-token log gate), beta [B,T,Hv] f32 as the
 * pipeline passes them; initial_state [N,Hv,K,V] f32 or NULL.
 * Outputs: o [B,T,Hv,V] bf16, g_cumsum [B,T,Hv] f32 (may be NULL),
 * final_state [N,Hv,K,V] f32 (NULL unless output_final_state).
 * use_qk_l2norm_in_kernel: q and k rows are scaled by 1/sqrt(sum x^2 + 1e-6)
 * while they are staged, as fla's l2norm_fwd does ahead of the chunk forward
 * (examples/flash_gated_delta_rule.py:1086-1089).
 * h [B,Hv,NT,K,V] (state at the start of every chunk), v_new [B,Hv,T,V] and
 * w [B,Hv,T,K], all bf16 and each NULL or given: what the reference's backward
 * recomputes with recompute_w_u_fwd and chunk_gated_delta_rule_fwd_h
 * (examples/flash_gated_delta_rule.py:913-951), written by the forward instead.
 * q_normalised [B,Hk,T,K], k_normalised [B,Hk,T,K] (element type of q, any
 * strides with unit innermost stride) and q_rstd, k_rstd [B,Hk,T] f32
 * (contiguous): all four given or all NULL, and only with
 * use_qk_l2norm_in_kernel.  The scaled rows and the factors they were scaled
 * by, which fla's l2norm_fwd returns to its autograd function
 * (examples/flash_gated_delta_rule.py:1086-1089) and a backward needs.
 * ------------------------------------------------------------------------ */
int fla_gdn_chunk_fwd_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
    const fla_tensor *beta, double scale, const fla_tensor *initial_state,
    bool output_final_state, const fla_int_array *cu_seqlens, int64_t chunk_size,
    bool use_qk_l2norm_in_kernel, const fla_tensor *o, const fla_tensor *g_cumsum,
    const fla_tensor *final_state, const fla_tensor *h, const fla_tensor *v_new,
    const fla_tensor *w, const fla_tensor *q_normalised, const fla_tensor *k_normalised,
    const fla_tensor *q_rstd, const fla_tensor *k_rstd, uint64_t *workspace_size);
int fla_gdn_chunk_fwd(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
    const fla_tensor *beta, double scale, const fla_tensor *initial_state,
    bool output_final_state, const fla_int_array *cu_seqlens, int64_t chunk_size,
    bool use_qk_l2norm_in_kernel, const fla_tensor *o, const fla_tensor *g_cumsum,
    const fla_tensor *final_state, const fla_tensor *h, const fla_tensor *v_new,
    const fla_tensor *w, const fla_tensor *q_normalised, const fla_tensor *k_normalised,
    const fla_tensor *q_rstd, const fla_tensor *k_rstd, void *workspace,
    uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * recurrent_gated_delta_rule - replaces aclnnRecurrentGatedDeltaRule
 * (recurrent_gated_delta_rule/README.md:46-70; _aclnn_ctypes.py:654-846).
 * query,key [T,Nk,Dk], value [T,Nv,Dv], beta [T,Nv] bf16; state
 * [Block,Nv,Dv,Dk] f32 or bf16, updated in place, may be strided over the
 * first two dims; actual_seq_lengths [B+1] i32 and ssm_state_indices [T] i32
 * are DEVICE tensors; g [T,Nv] f32, gk [T,Nv,Dk] f32, num_accepted_tokens
 * [B] i32 optional.  out [T,Nv,Dv] bf16.
 * ------------------------------------------------------------------------ */
int fla_recurrent_gated_delta_rule_get_workspace_size(
    const fla_tensor *query, const fla_tensor *key, const fla_tensor *value,
    const fla_tensor *beta, const fla_tensor *state, const fla_tensor *actual_seq_lengths,
    const fla_tensor *ssm_state_indices, const fla_tensor *g, const fla_tensor *gk,
    const fla_tensor *num_accepted_tokens, float scale, const fla_tensor *out,
    uint64_t *workspace_size);
int fla_recurrent_gated_delta_rule(
    const fla_tensor *query, const fla_tensor *key, const fla_tensor *value,
    const fla_tensor *beta, const fla_tensor *state, const fla_tensor *actual_seq_lengths,
    const fla_tensor *ssm_state_indices, const fla_tensor *g, const fla_tensor *gk,
    const fla_tensor *num_accepted_tokens, float scale, const fla_tensor *out,
    void *workspace, uint64_t workspace_size, void *stream);

/* gdn_chunk_fwd_state_pool and recurrent_gdn_prefill_plan: what recurrent_gated_delta_rule needs to run the long
 * sequences of a call (prefill) on the chunk kernels instead of token by token.  No counterpart in the reference.
 *
 * gdn_chunk_fwd_state_pool: gdn_chunk_fwd (operands as there) whose initial and final states are rows of one pool:
 * state_pool f32 [rows,Hv,K,V] with contiguous K x V or V x K blocks (the recurrent operator's V-first pool is passed
 * as its transposed view), state_indices i32 [N] on the device names the row of each sequence.  A sequence reads its
 * row before its first token and overwrites it after its last one; a negative index means no row (zero initial state,
 * final state dropped), an index past the pool is clamped into it.  Two sequences that name one row race.
 *
 * recurrent_gdn_prefill_plan: one launch over actual_seq_lengths i32 [B+1] and ssm_state_indices i32 [T] (device, as
 * the recurrent operator takes them) that writes slots i32 [B] (the pool row of each sequence's first token, -1 for an
 * empty or rejected sequence) and report i32 [2B+1] = {offset, length of each sequence, flag of each sequence}; a flag
 * is 1 when the lengths are inconsistent with T, when a token of the sequence names another row than its first token,
 * when that row is outside the pool (pool_rows) or when another sequence names it too.  B <= 8192. */
int fla_gdn_chunk_fwd_state_pool_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
    const fla_tensor *beta, double scale, const fla_tensor *state_pool, const fla_tensor *state_indices,
    const fla_int_array *cu_seqlens, int64_t chunk_size, bool use_qk_l2norm_in_kernel,
    const fla_tensor *o, uint64_t *workspace_size);
int fla_gdn_chunk_fwd_state_pool(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
    const fla_tensor *beta, double scale, const fla_tensor *state_pool, const fla_tensor *state_indices,
    const fla_int_array *cu_seqlens, int64_t chunk_size, bool use_qk_l2norm_in_kernel,
    const fla_tensor *o, void *workspace, uint64_t workspace_size, void *stream);
int fla_recurrent_gdn_prefill_plan(
    const fla_tensor *actual_seq_lengths, const fla_tensor *ssm_state_indices, int64_t pool_rows,
    const fla_tensor *slots, const fla_tensor *report, void *stream);

/* ------------------------------------------------------------------------
 * causal_conv1d - replaces aclnnCausalConv1d (docs/aclnnCausalConv1d.md:31-48;
 * _aclnn_ctypes.py:951-985).  x [B,S,D] or [T,D] bf16/f16; weight [W,D];
 * bias [D] optional; conv_states [N,>=W-1,D] optional, updated in place.
 * run_mode 0 (prefill) only.  out like x, or [B,head_num,S,D/head_num].
 * ------------------------------------------------------------------------ */
int fla_causal_conv1d_get_workspace_size(
    const fla_tensor *x, const fla_tensor *weight, const fla_tensor *bias,
    const fla_tensor *conv_states, const fla_int_array *query_start_loc,
    const fla_int_array *cache_indices, const fla_int_array *initial_state_mode,
    const fla_int_array *num_accepted_tokens, int64_t activation_mode, int64_t pad_slot_id,
    int64_t run_mode, int64_t head_num, const fla_tensor *out, uint64_t *workspace_size);
int fla_causal_conv1d(
    const fla_tensor *x, const fla_tensor *weight, const fla_tensor *bias,
    const fla_tensor *conv_states, const fla_int_array *query_start_loc,
    const fla_int_array *cache_indices, const fla_int_array *initial_state_mode,
    const fla_int_array *num_accepted_tokens, int64_t activation_mode, int64_t pad_slot_id,
    int64_t run_mode, int64_t head_num, const fla_tensor *out, void *workspace,
    uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * kda_gate_cumsum - replaces aclnnKdaGateCumsum (_aclnn_ctypes.py:1268-1296;
 * kda_gate_cumsum/op_kernel/kda_gate_cumsum_kernel.h:374-419,516-534).
 * g [B,Hv,T,K] f32/bf16 raw gate; A_log [Hv] f32 and dt_bias [Hv*K] f32 are
 * used when use_gate_in_kernel (softplus gate, or lower_bound * sigmoid when
 * safe_gate).  Output gk [B,Hv,T,K] f32 = chunk-local cumsum / ln 2.
 * ------------------------------------------------------------------------ */
int fla_kda_gate_cumsum_get_workspace_size(
    const fla_tensor *g, const fla_tensor *A_log, const fla_tensor *dt_bias,
    const fla_int_array *cu_seqlens, int64_t chunk_size, bool use_gate_in_kernel,
    bool safe_gate, double lower_bound, const fla_tensor *gk, uint64_t *workspace_size);
int fla_kda_gate_cumsum(
    const fla_tensor *g, const fla_tensor *A_log, const fla_tensor *dt_bias,
    const fla_int_array *cu_seqlens, int64_t chunk_size, bool use_gate_in_kernel,
    bool safe_gate, double lower_bound, const fla_tensor *gk, void *workspace,
    uint64_t workspace_size, void *stream);

/* kda_gate_bwd - gradient of the gate activation that chunk_kda_fwd / kda_gate_cumsum apply with use_gate_in_kernel.
 * No counterpart among the reference's kernels (its KDA backward is a third-party Triton package,
 * adapters/triton_ascend_kda.py:141-242); fla_hip.pipeline.chunk_kda uses it so that a training step with the gate in
 * the kernel needs no tensor-operation copy of the activation.  g: the raw gate, f32 or bf16, in `layout`
 * ("BSND", "BNSD", "TND", "NTD"; any outer strides); dgate: f32, gradient of the activated gate, same shape;
 * A_log f32 [Hv]; dt_bias f32 [Hv*K] or NULL.  Outputs: dg_raw (dtype and shape of g); partial sums over tiles of 256
 * tokens, contiguous f32: ddt_bias_partial [B*ceil(T/256), Hv, K] (NULL without dt_bias) and dA_log_partial
 * [B*ceil(T/256), Hv] - the caller adds them over the first dimension.  K in {32, 64, 128, 256}. */
int fla_kda_gate_bwd_get_workspace_size(
    const fla_tensor *g, const fla_tensor *dgate, const fla_tensor *A_log, const fla_tensor *dt_bias,
    const char *layout, bool safe_gate, double lower_bound, const fla_tensor *dg_raw,
    const fla_tensor *ddt_bias_partial, const fla_tensor *dA_log_partial, uint64_t *workspace_size);
int fla_kda_gate_bwd(
    const fla_tensor *g, const fla_tensor *dgate, const fla_tensor *A_log, const fla_tensor *dt_bias,
    const char *layout, bool safe_gate, double lower_bound, const fla_tensor *dg_raw,
    const fla_tensor *ddt_bias_partial, const fla_tensor *dA_log_partial, void *workspace,
    uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * chunk_gated_delta_rule_bwd_dhu - replaces aclnnChunkGatedDeltaRuleBwdDhu
 * (_aclnn_ctypes.py:324-394; chunk_gated_delta_rule_bwd_dhu/README.md:6-13).
 * q,k [B,Hk,T,K], w [B,Hv,T,K], d_o,dv [B,Hv,T,V] bf16.  Exactly one gate:
 * g [B,Hv,T] f32/bf16 (natural log, use_exp2 false) or gK [B,Hv,T,K] f32
 * (log2, use_exp2 true; q and k then already carry their gates).
 * h0 is only a presence flag for the caller; dht [N,Hv,K,V] f32 optional.
 * Outputs dh [B,Hv,NT,K,V] bf16, dv2 like dv, dh0 optional: either the
 * reference form (bf16, shape of dh, written at each sequence's first chunk)
 * or f32 [N,Hv,K,V].  Implemented: K in {64,128} (K = 256 with gK), V a
 * multiple of 64; chunk_size 64, and 128 with the scalar gate.
 * Extension: dv may be NULL (scalar gate, chunk_size 64).  The scan then forms
 * the intra-chunk part of dv itself, the result of chunk_bwd_dv_local on
 * (q, k, d_o, g, scale), from the tiles it stages anyway.
 * ------------------------------------------------------------------------ */
int fla_chunk_gated_delta_rule_bwd_dhu_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o,
    const fla_tensor *dv, const fla_tensor *g, const fla_tensor *gK, const fla_tensor *h0,
    const fla_tensor *dht, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    double scale, int64_t chunk_size, bool use_exp2, const fla_tensor *dh,
    const fla_tensor *dh0, const fla_tensor *dv2, uint64_t *workspace_size);
int fla_chunk_gated_delta_rule_bwd_dhu(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o,
    const fla_tensor *dv, const fla_tensor *g, const fla_tensor *gK, const fla_tensor *h0,
    const fla_tensor *dht, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    double scale, int64_t chunk_size, bool use_exp2, const fla_tensor *dh,
    const fla_tensor *dh0, const fla_tensor *dv2, void *workspace, uint64_t workspace_size,
    void *stream);

/* ------------------------------------------------------------------------
 * chunk_kda_fwd - replaces aclnnChunkKdaFwd (_aclnn_ctypes.py:1066-1265;
 * fla/ops/ascendc/kda/chunk_kda_fwd/docs/api.md).  layout is "BSND", "BNSD",
 * "TND" or "NTD" and applies to q,k [..H,K], v [..HV,V], g [..HV,K] (raw gate,
 * f32/bf16), beta [..HV] (f32/bf16) and attn_out (like v).  A_log [HV] and
 * dt_bias [HV*K] f32 are used when use_gate_in_kernel.  States are f32
 * [N,HV,K,V] ([N,HV,V,K] when state_v_first).  The remaining outputs are
 * head-major: gk f32 [..HV,T,K] (chunk-local cumulated gate, log2 units),
 * Aqk, Akk [..HV,T,chunk], w, qg, kg [..HV,T,K], u, v_new [..HV,T,V], and
 * h [B,NT,HV,K,V] (rank-3 layouts: [NT,HV,K,V]).  final_state, gk, w, u, qg,
 * kg, v_new and h may be null.  Implemented: bf16 or f16 q/k/v, chunk_size 64
 * and 128, K in {64,128} with V in {K, 2K}, and K = V = 256.  With bf16
 * inputs and K <= 128, qg and kg may also be f16 tensors (11-bit significands
 * for the reverse scan of a training step, see chunk_kda_bwd_dhu).
 * ------------------------------------------------------------------------ */
int fla_chunk_kda_fwd_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
    const fla_tensor *beta, const fla_tensor *A_log, const fla_tensor *dt_bias,
    const fla_tensor *initial_state, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const char *layout, double scale, int64_t chunk_size,
    bool safe_gate, double lower_bound, bool use_gate_in_kernel, bool state_v_first,
    const fla_tensor *attn_out, const fla_tensor *final_state, const fla_tensor *gk,
    const fla_tensor *Aqk, const fla_tensor *Akk, const fla_tensor *w, const fla_tensor *u,
    const fla_tensor *qg, const fla_tensor *kg, const fla_tensor *v_new, const fla_tensor *h,
    uint64_t *workspace_size);
int fla_chunk_kda_fwd(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
    const fla_tensor *beta, const fla_tensor *A_log, const fla_tensor *dt_bias,
    const fla_tensor *initial_state, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const char *layout, double scale, int64_t chunk_size,
    bool safe_gate, double lower_bound, bool use_gate_in_kernel, bool state_v_first,
    const fla_tensor *attn_out, const fla_tensor *final_state, const fla_tensor *gk,
    const fla_tensor *Aqk, const fla_tensor *Akk, const fla_tensor *w, const fla_tensor *u,
    const fla_tensor *qg, const fla_tensor *kg, const fla_tensor *v_new, const fla_tensor *h,
    void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * chunk_kda_fwd_noalloc - no counterpart in the reference.  For callers that cannot allocate
 * device memory around a call (code under HIP stream capture, serving loops and harnesses that
 * forbid hipMalloc): fla_chunk_kda_fwd with the same operands and results, minus the workspace
 * pair.  The per-chunk decay rows and whichever of w, u, qg, kg the caller passes as NULL live
 * in a fixed array of FLA_CHUNK_KDA_FWD_NOALLOC_SCRATCH_BYTES in device memory, one per GPU,
 * held until the process ends.  A call whose scratch need exceeds the array returns
 * FLA_ERR_WORKSPACE (with w, u, qg, kg supplied the need is B*NT*HV*K*4 bytes, plus, with bf16
 * elements, the fp16 copies of u and kg that the state scan reads: 2 bytes per element of each);
 * cu_seqlens and chunk_indices must be NULL (FLA_ERR_UNSUPPORTED otherwise).  The call performs no
 * hipMalloc / hipFree / hipHostMalloc.  All calls on one GPU share the array: calls that may
 * overlap in time on one GPU (different streams, different threads) race and must be serialised
 * by the caller.  The array's device address is resolved by the first call on a device, which
 * must not be made while `stream` is being captured (FLA_ERR_UNSUPPORTED then):
 * fla_chunk_kda_fwd_noalloc_init(), called once per device with that device current, resolves it
 * ahead of time; it launches nothing and allocates nothing.
 * ------------------------------------------------------------------------ */
#define FLA_CHUNK_KDA_FWD_NOALLOC_SCRATCH_BYTES (32u << 20)
int fla_chunk_kda_fwd_noalloc_init(void);
int fla_chunk_kda_fwd_noalloc(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g,
    const fla_tensor *beta, const fla_tensor *A_log, const fla_tensor *dt_bias,
    const fla_tensor *initial_state, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const char *layout, double scale, int64_t chunk_size,
    bool safe_gate, double lower_bound, bool use_gate_in_kernel, bool state_v_first,
    const fla_tensor *attn_out, const fla_tensor *final_state, const fla_tensor *gk,
    const fla_tensor *Aqk, const fla_tensor *Akk, const fla_tensor *w, const fla_tensor *u,
    const fla_tensor *qg, const fla_tensor *kg, const fla_tensor *v_new, const fla_tensor *h,
    void *stream);

/* ------------------------------------------------------------------------
 * chunk_kda_bwd_intra - replaces aclnnChunkKdaBwdIntra
 * (_aclnn_ctypes.py:1534-1768; golden test_npu_chunk_kda_bwd_intra.py:7-91).
 * layout "BSND", "BNSD" (dense) or "TND" (needs cu_seqlens).  q,k bf16 [..,K];
 * gk (chunk-local cumulated gate, log2 units), dq, dk, dg f32 like q; beta
 * bf16/f32 and db f32 [..]; dAqk, dAkk f32 [..,64].  All contiguous.
 * Outputs dq_out, dk_out, dg_out like dq and db_out like db hold the inputs
 * plus the intra-chunk terms.  K in {64,128,256}; chunk_size 64; safe_gate
 * must be true.
 * ------------------------------------------------------------------------ */
int fla_chunk_kda_bwd_intra_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta,
    const fla_tensor *dAqk, const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *db, const fla_tensor *dg, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate, const char *layout,
    const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, uint64_t *workspace_size);
int fla_chunk_kda_bwd_intra(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta,
    const fla_tensor *dAqk, const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *db, const fla_tensor *dg, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate, const char *layout,
    const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, void *workspace, uint64_t workspace_size, void *stream);

/* chunk_kda_bwd_intra followed by the reverse chunk-local running sum of dg_out.  No counterpart in the reference, whose
 * composition (and this build's, fla_hip.pipeline.chunk_kda_bwd) runs chunk_local_cumsum(reverse) over the gate gradient
 * right after this operator: here the workgroup that holds a chunk of dg takes the sum before it stores it.  Same
 * operands and rules as fla_chunk_kda_bwd_intra, except that dq_out and dk_out (both or neither) may be tensors of q's
 * element type with the strides of dq: dq and dk are final with this stage, and a training step would otherwise
 * convert them in a pass of its own. */
int fla_chunk_kda_bwd_intra_cumsum_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta,
    const fla_tensor *dAqk, const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *db, const fla_tensor *dg, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate, const char *layout,
    const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, uint64_t *workspace_size);
int fla_chunk_kda_bwd_intra_cumsum(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *gk, const fla_tensor *beta,
    const fla_tensor *dAqk, const fla_tensor *dAkk, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *db, const fla_tensor *dg, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, bool safe_gate, const char *layout,
    const fla_tensor *dq_out, const fla_tensor *dk_out, const fla_tensor *db_out,
    const fla_tensor *dg_out, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * KDA chunk backward, the stages around chunk_gated_delta_rule_bwd_dhu (gK) and chunk_kda_bwd_intra.
 * The reference has no operators for them: its deployment keeps them in a third-party Triton package
 * (torch_custom/fla_npu/fla_npu/adapters/triton_ascend_kda.py:1-8); they differentiate the forward of
 * tests/atk/chunk_kda_fwd/executor_chunk_kda_fwd.py:459-484.  All activations in [B,H,T,D] index order
 * through strides (unit innermost stride; a [B,T,H,D] tensor is passed as its transposed view).  gk is
 * the chunk-local cumulated gate in log2 units, f32 [B,Hv,T,K].  dq, dk, dg are f32 [B,Hv,T,K], one per
 * VALUE head; "dg" is the gradient with respect to ln2 * gk, as in chunk_kda_bwd_intra.  chunk_size 64.
 * ------------------------------------------------------------------------ */

/* chunk_kda_bwd_dav: dAqk = scale * tril(d_o v_new^T) (f32 [B,Hv,T,64], zero above the diagonal),
 * dv = Aqk^T d_o.  v_new, d_o, dv [B,Hv,T,V], Aqk [B,Hv,T,64] in the element type. */
int fla_chunk_kda_bwd_dav_get_workspace_size(
    const fla_tensor *v_new, const fla_tensor *d_o, const fla_tensor *Aqk, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dAqk, const fla_tensor *dv,
    uint64_t *workspace_size);
int fla_chunk_kda_bwd_dav(
    const fla_tensor *v_new, const fla_tensor *d_o, const fla_tensor *Aqk, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dAqk, const fla_tensor *dv,
    void *workspace, uint64_t workspace_size, void *stream);

/* chunk_kda_bwd_dqkwg: with h the state at each chunk start, dh the gradient of the state at each chunk
 * end and dv the total gradient of v_new (dh, dv: outputs of bwd_dhu), both [B,Hv,NT,K,V] with any outer strides:
 *   dq = scale (d_o h^T) 2^g,  dk = (v_new dh^T) 2^{g_last - g},  dw = -dv h^T (element type, [B,Hv,T,K]),
 *   dg = q dq - k dk, plus on the last token of a chunk  sum_j k_j dk_j + 2^{g_last} rowsum(h . dh).
 * dAqk (f32 [B,Hv,T,64], or NULL): also written, the first result of chunk_kda_bwd_dav (scale * tril(d_o v_new^T)),
 * from the d_o and v_new tiles this operator stages anyway. */
int fla_chunk_kda_bwd_dqkwg_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *dw, const fla_tensor *dg, const fla_tensor *dAqk, uint64_t *workspace_size);
int fla_chunk_kda_bwd_dqkwg(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk,
    const fla_tensor *dw, const fla_tensor *dg, const fla_tensor *dAqk, void *workspace, uint64_t workspace_size,
    void *stream);

/* chunk_kda_bwd_dhu: chunk_gated_delta_rule_bwd_dhu with the per-channel gate gK (log2 units, use_exp2) whose dv
 * operand, dv = Aqk^T d_o per chunk (the second result of chunk_kda_bwd_dav), is formed inside the scan from the
 * forward's score blocks Aqk [B,Hv,T,64] and the d_o tiles it stages anyway, so that dv never goes through memory.
 * No counterpart in the reference (see the note above); q, k are the gated qg, kg of the forward, in the element type
 * of w and d_o or both f16 beside bf16 w and d_o (the tensors chunk_kda_fwd writes when asked for f16 qg, kg).
 * chunk_size 64, K in {64,128}.  Outputs as chunk_gated_delta_rule_bwd_dhu. */
int fla_chunk_kda_bwd_dhu_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o, const fla_tensor *Aqk,
    const fla_tensor *gK, const fla_tensor *h0, const fla_tensor *dht, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dh, const fla_tensor *dh0,
    const fla_tensor *dv2, uint64_t *workspace_size);
int fla_chunk_kda_bwd_dhu(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *w, const fla_tensor *d_o, const fla_tensor *Aqk,
    const fla_tensor *gK, const fla_tensor *h0, const fla_tensor *dht, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, double scale, int64_t chunk_size, const fla_tensor *dh, const fla_tensor *dh0,
    const fla_tensor *dv2, void *workspace, uint64_t workspace_size, void *stream);

/* chunk_kda_bwd_wy: backward of w = Akk (k beta 2^g), u = Akk (v beta), Akk = (I + M)^-1 given dw, du:
 *   x = Akk^T dw, y = Akk^T du;  dk += x beta 2^g;  dg += (x beta 2^g) k   (dk, dg are read and added to);
 *   dv = y beta (element type);  db = <x, k 2^g> + <y, v> (f32 [B,Hv,T], written);
 *   dAkk = -strict_lower(Akk^T (dw (k beta 2^g)^T + du (v beta)^T) Akk^T)  (f32 [B,Hv,T,64], written). */
int fla_chunk_kda_bwd_wy_get_workspace_size(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *gk, const fla_tensor *Akk,
    const fla_tensor *dw, const fla_tensor *du, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dg,
    const fla_tensor *dAkk, uint64_t *workspace_size);
int fla_chunk_kda_bwd_wy(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *gk, const fla_tensor *Akk,
    const fla_tensor *dw, const fla_tensor *du, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dg,
    const fla_tensor *dAkk, void *workspace, uint64_t workspace_size, void *stream);

/* chunk_kda_bwd_dqkwg_wy: chunk_kda_bwd_dqkwg (with dAqk) and chunk_kda_bwd_wy of the same chunks in one launch, for
 * the composition of the KDA backward: dw = -dv2 h^T passes from the first stage to the second through on-chip memory
 * and dk, dg leave once, complete (as two operators they are written, read back, added to and written again).  dv2 is
 * the total gradient of v_new (the dv2 of chunk_kda_bwd_dhu; du of the second stage), v and beta the forward's inputs,
 * Akk its inverse blocks.  Results: dq, dk, dg f32 [B,Hv,T,K]; dAqk, dAkk f32 [B,Hv,T,64]; dv (element type,
 * [B,Hv,T,V]); db f32 [B,Hv,T].  (K,V) in (128,128), (64,64), (64,128); chunk_size 64.  No counterpart in the reference. */
int fla_chunk_kda_bwd_dqkwg_wy_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dAqk,
    const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dAkk, uint64_t *workspace_size);
int fla_chunk_kda_bwd_dqkwg_wy(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dAqk,
    const fla_tensor *dv, const fla_tensor *db, const fla_tensor *dAkk, void *workspace, uint64_t workspace_size,
    void *stream);

/* chunk_kda_bwd_dqkwg_wy_intra: the same two stages followed by chunk_kda_bwd_intra_cumsum in the same launch, i.e.
 * everything of the KDA backward after the reverse scan.  dAqk and dAkk stay on chip (the intra-chunk stage reads them
 * as fp32 tiles, masked as that operator masks them), its increments are added to dq, dk, dg in registers (same fp32
 * products and order of additions as the separate operators), dg leaves as its reverse chunk-local running sum and
 * dbeta complete.  dq and dk (one dtype for both): f32 [B,Hv,T,K], or the element type, which is meant for Hv == Hk
 * where they are final; with grouped value heads the caller adds the fp32 results of the heads of a group.  Other
 * operands, head sizes and chunk size as chunk_kda_bwd_dqkwg_wy.  No counterpart in the reference. */
int fla_chunk_kda_bwd_dqkwg_wy_intra_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dv,
    const fla_tensor *db, uint64_t *workspace_size);
int fla_chunk_kda_bwd_dqkwg_wy_intra(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v_new, const fla_tensor *gk, const fla_tensor *h,
    const fla_tensor *d_o, const fla_tensor *dh, const fla_tensor *dv2, const fla_tensor *v, const fla_tensor *beta,
    const fla_tensor *Akk, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dg, const fla_tensor *dv,
    const fla_tensor *db, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * l2norm_fwd / l2norm_bwd - the q/k normalisation of the chunk pipelines, which the reference
 * runs as Triton kernels (fla/ops/triton/triton_core/l2norm.py:131-224; called from
 * examples/flash_gated_delta_rule.py:1047-1049,1104-1106).  Rank 2..4 bf16/f16 tensors with
 * arbitrary outer strides, last extent 64, 128 or 256; rstd fp32, contiguous, one per row.
 *   fwd: y = x rstd, rstd = 1/sqrt(sum x^2 + eps) (rstd may be NULL);  bwd: dx = (dy - sum(dy y) y) rstd.
 * ------------------------------------------------------------------------ */
int fla_l2norm_fwd_get_workspace_size(const fla_tensor *x, double eps, const fla_tensor *y, const fla_tensor *rstd,
                                      uint64_t *workspace_size);
int fla_l2norm_fwd(const fla_tensor *x, double eps, const fla_tensor *y, const fla_tensor *rstd, void *workspace,
                   uint64_t workspace_size, void *stream);
int fla_l2norm_bwd_get_workspace_size(const fla_tensor *y, const fla_tensor *rstd, const fla_tensor *dy, double eps,
                                      const fla_tensor *dx, uint64_t *workspace_size);
int fla_l2norm_bwd(const fla_tensor *y, const fla_tensor *rstd, const fla_tensor *dy, double eps, const fla_tensor *dx,
                   void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * recurrent_kda - replaces aclnnRecurrentKda (kda/recurrent_kda/docs/api.md:56-88;
 * _aclnn_ctypes.py:1298-1503).  layout "BSND": q,k [B,T,H,K], v,out [B,T,HV,V],
 * g [B,T,HV,K], beta [B,T,HV]; "TND": the same without B.  q,k,v,out bf16; g, beta
 * f32/bf16/f16.  initial_state: pool [capacity,HV,V,K] (state_v_first) or
 * [capacity,HV,K,V], f32 or bf16, slot and head axes may be strided.  cu_seqlens
 * [seq_num+1], ssm_state_indices (packed [>=T] or [seq_num,max_step]) and
 * num_accepted_tokens [seq_num] are DEVICE tensors, int32 or int64; their values are
 * read by the kernel only.  A_log [HV], dt_bias [HV*K] f32 with use_gate_in_kernel.
 * final_state: the pool the states are written to when inplace_final_state is false.
 * ------------------------------------------------------------------------ */
int fla_recurrent_kda_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
    const fla_tensor *initial_state, const fla_tensor *cu_seqlens, const fla_tensor *ssm_state_indices, const fla_tensor *A_log,
    const fla_tensor *dt_bias, const fla_tensor *num_accepted_tokens, const char *layout, double scale, bool output_final_state,
    bool inplace_final_state, bool use_qk_l2norm_in_kernel, bool use_gate_in_kernel, bool use_beta_sigmoid_in_kernel,
    bool allow_neg_eigval, bool safe_gate, double lower_bound, bool state_v_first, const fla_tensor *attn_out,
    const fla_tensor *final_state, uint64_t *workspace_size);
int fla_recurrent_kda(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *beta,
    const fla_tensor *initial_state, const fla_tensor *cu_seqlens, const fla_tensor *ssm_state_indices, const fla_tensor *A_log,
    const fla_tensor *dt_bias, const fla_tensor *num_accepted_tokens, const char *layout, double scale, bool output_final_state,
    bool inplace_final_state, bool use_qk_l2norm_in_kernel, bool use_gate_in_kernel, bool use_beta_sigmoid_in_kernel,
    bool allow_neg_eigval, bool safe_gate, double lower_bound, bool state_v_first, const fla_tensor *attn_out,
    const fla_tensor *final_state, void *workspace, uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * causal_conv1d_bwd - replaces aclnnCausalConv1dBwd (_aclnn_ctypes.py:988-1037;
 * causal_conv1d_bwd/README.md:54-118).  x, dx: logical [B,T,D] or packed [T,D];
 * y (pre-activation, needed when activation is 1 or 2) and dy in input_layout
 * "BSND"/"BSH" [B,T,D], "BNSD" [B,N,T,D/N], "TND" [T,D], "NTD" [N,T,D/N] (the packed
 * layouts need query_start_loc).  initial_state, dht, dh0: [N,W,D], rows 1..W-1 hold
 * the last W-1 inputs.  dw [W,D], db [D] and dh0 are optional outputs.  bf16 or f16.
 * ------------------------------------------------------------------------ */
int fla_causal_conv1d_bwd_get_workspace_size(
    const fla_tensor *x, const fla_tensor *y, const fla_tensor *weight, const fla_tensor *dy, const fla_tensor *initial_state,
    const fla_tensor *dht, const fla_int_array *query_start_loc, int64_t activation, const char *input_layout,
    const fla_tensor *dx, const fla_tensor *dw, const fla_tensor *db, const fla_tensor *dh0, uint64_t *workspace_size);
int fla_causal_conv1d_bwd(
    const fla_tensor *x, const fla_tensor *y, const fla_tensor *weight, const fla_tensor *dy, const fla_tensor *initial_state,
    const fla_tensor *dht, const fla_int_array *query_start_loc, int64_t activation, const char *input_layout,
    const fla_tensor *dx, const fla_tensor *dw, const fla_tensor *db, const fla_tensor *dh0, void *workspace,
    uint64_t workspace_size, void *stream);

/* ------------------------------------------------------------------------
 * Gated-delta-rule backward chain (examples/flash_gated_delta_rule.py:884-1008).
 * All activations head-first: q, k, dq, dk [B,Hk,T,K]; v, d_o, dv, du [B,Hv,T,V];
 * w, dw [B,Hv,T,K] bf16; g (chunk-cumsummed) and beta [B,Hv,T] f32 or bf16;
 * A, dA [B,Hv,T,C] bf16; h, dh [B,Hv,NT,K,V] bf16.  Hv may be a multiple of Hk:
 * dq and dk are then summed over the value heads of a key head.
 * ------------------------------------------------------------------------ */

/* chunk_bwd_dv_local - replaces aclnnChunkBwdDvLocal (_aclnn_ctypes.py:397-427):
 * out = triu(k q^T e^{G_j - G_i}) * scale . d_o per chunk.  g_gamma must be NULL; A is
 * accepted and not read (as in the reference). */
int fla_chunk_bwd_dv_local_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *d_o, const fla_tensor *g, const fla_tensor *g_gamma,
    const fla_tensor *A, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *out, uint64_t *workspace_size);
int fla_chunk_bwd_dv_local(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *d_o, const fla_tensor *g, const fla_tensor *g_gamma,
    const fla_tensor *A, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices, double scale,
    int64_t chunk_size, const fla_tensor *out, void *workspace, uint64_t workspace_size, void *stream);

/* chunk_bwd_dqkwg - replaces aclnnChunkBwdDqkwg (_aclnn_ctypes.py:463-510).  v is v_new of the
 * forward scan, h the state at each chunk start, dh / dv the outputs of bwd_dhu; dg [B,Hv,T] f32 is the
 * gradient of the cumsummed gate.  w and g_gamma must be NULL or are ignored as in the reference;
 * use_exp2 and transpose_state_layout must be false.  h and dh: K x V blocks whose rows may be wider than V (a column
 * slab of wider blocks), 16-byte aligned.  chunk_size 128 with V = 256 (also in prepare_wy_repr_bwd_da / _full and
 * prepare_wy_repr_bwd): the launcher runs the 128-column kernels over the two halves of the value dimension and adds
 * the second pass, which lands in the workspace (reported by the size query), to the first; each pass rounds its part
 * to the element type. */
int fla_chunk_bwd_dqkwg_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *w, const fla_tensor *g_gamma, float scale, int64_t chunk_size,
    bool use_exp2, bool transpose_state_layout, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dw,
    const fla_tensor *dg, uint64_t *workspace_size);
int fla_chunk_bwd_dqkwg(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *w, const fla_tensor *g_gamma, float scale, int64_t chunk_size,
    bool use_exp2, bool transpose_state_layout, const fla_tensor *dq, const fla_tensor *dk, const fla_tensor *dw,
    const fla_tensor *dg, void *workspace, uint64_t workspace_size, void *stream);

/* chunk_bwd_dqkwg_l2norm - no counterpart in the reference, whose entry normalises q and k ahead of the forward and runs
 * l2norm_bwd over dq and dk after the backward (examples/flash_gated_delta_rule.py:1047-1049, 1104-1106).  q is the
 * normalised tensor; q_rstd (f32 [B,Hk,T], contiguous: the second result of l2norm_fwd) lets the kernel return dq as the
 * gradient of the un-normalised q, dq <- (dq - q <q, dq>) rstd per row, instead of a pass of its own over dq.  dk is
 * not final here (prepare_wy_repr_bwd_full_accumulate takes k_rstd for it).  Other operands as chunk_bwd_dqkwg. */
int fla_chunk_bwd_dqkwg_l2norm_get_workspace_size(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *q_rstd, float scale, int64_t chunk_size, const fla_tensor *dq,
    const fla_tensor *dk, const fla_tensor *dw, const fla_tensor *dg, uint64_t *workspace_size);
int fla_chunk_bwd_dqkwg_l2norm(
    const fla_tensor *q, const fla_tensor *k, const fla_tensor *v, const fla_tensor *g, const fla_tensor *h,
    const fla_tensor *dox, const fla_tensor *dh, const fla_tensor *dv, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, const fla_tensor *q_rstd, float scale, int64_t chunk_size, const fla_tensor *dq,
    const fla_tensor *dk, const fla_tensor *dw, const fla_tensor *dg, void *workspace, uint64_t workspace_size,
    void *stream);

/* prepare_wy_repr_bwd_da - replaces aclnnPrepareWyReprBwdDa (_aclnn_ctypes.py:430-460): gradient of
 * the strictly-lower chunk matrix, stored TRANSPOSED (upper triangular) as the reference does. */
int fla_prepare_wy_repr_bwd_da_get_workspace_size(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dA, uint64_t *workspace_size);
int fla_prepare_wy_repr_bwd_da(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dA, void *workspace, uint64_t workspace_size, void *stream);

/* prepare_wy_repr_bwd - replaces aclnnPrepareWyReprBwd (_aclnn_ctypes.py:284-321): bwd_da followed by
 * bwd_full in one call; the intermediate dA (bf16, [B,Hv,T,C]) lives in the workspace. */
int fla_prepare_wy_repr_bwd_get_workspace_size(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg,
    uint64_t *workspace_size);
int fla_prepare_wy_repr_bwd(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dw,
    const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens, const fla_int_array *chunk_indices,
    int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg,
    void *workspace, uint64_t workspace_size, void *stream);

/* prepare_wy_repr_bwd_full - replaces aclnnPrepareWyReprBwdFull (_aclnn_ctypes.py:242-279):
 * dk [B,Hk,T,K], dv [B,Hv,T,V] bf16; dbeta, dg [B,Hv,T] f32; dA as written by bwd_da. */
int fla_prepare_wy_repr_bwd_full_get_workspace_size(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv,
    const fla_tensor *dbeta, const fla_tensor *dg, uint64_t *workspace_size);
int fla_prepare_wy_repr_bwd_full(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *dk, const fla_tensor *dv,
    const fla_tensor *dbeta, const fla_tensor *dg, void *workspace, uint64_t workspace_size, void *stream);

/* prepare_wy_repr_bwd_full_accumulate - no counterpart in the reference, whose composition adds the two
 * key gradients with a separate elementwise pass (examples/flash_gated_delta_rule.py:994-1010, dk.add_(dk2)).
 * Same operands as prepare_wy_repr_bwd_full; dk and dg are read, the operator's results added in fp32, and
 * written back in place (dk rounded once).  dv and dbeta are written as usual.  k_rstd (f32 [B,Hk,T] contiguous, or
 * NULL): k is the l2-normalised tensor and the completed dk leaves as the gradient of the un-normalised k,
 * dk <- (dk - k <k, dk>) rstd per row (what l2norm_bwd would do in a pass of its own).
 * dA may be NULL (chunk_size 64): the kernel then forms the result of prepare_wy_repr_bwd_da on the same operands
 * itself, from the tiles it stages anyway, and dA never goes through memory.  With dA NULL, A may be NULL too: each
 * chunk's (I + strict_lower(beta k k^T e^{g_i - g_j}))^-1 is rebuilt in the kernel from k, g and beta, by the arithmetic
 * of fla_chunk_scaled_dot_kkt_inverse (bit-identical to the matrix that operator stores). */
int fla_prepare_wy_repr_bwd_full_accumulate_get_workspace_size(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *k_rstd, const fla_tensor *dk,
    const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg, uint64_t *workspace_size);
int fla_prepare_wy_repr_bwd_full_accumulate(
    const fla_tensor *k, const fla_tensor *v, const fla_tensor *beta, const fla_tensor *A, const fla_tensor *dA,
    const fla_tensor *dw, const fla_tensor *du, const fla_tensor *g, const fla_int_array *cu_seqlens,
    const fla_int_array *chunk_indices, int64_t chunk_size, const fla_tensor *k_rstd, const fla_tensor *dk,
    const fla_tensor *dv, const fla_tensor *dbeta, const fla_tensor *dg, void *workspace, uint64_t workspace_size,
    void *stream);

#ifdef __cplusplus
}
#endif
#endif /* FLA_HIP_H_ */
