/*
 * dataflow_amd_ops.h -- operator interface of the MoE layer: skeleton setters and submit wrappers.
 *
 * The first two groups keep the names, argument order and argument meaning of the reference's
 * libdataflowops (libdataflowops/include/dataflow_ops.h, set_op_skeletons.h) so a caller written
 * against that library links against this one unchanged. Each wrapper builds an Op on the stack
 * (op_args[i] = address of argument i) and calls handle->submit_op.
 *
 * The last group ("amd_") are additions: one-launch grouped forms of work the reference issues as a
 * host loop over experts. They exist only in this backend.
 */
#ifndef DATAFLOW_AMD_OPS_H
#define DATAFLOW_AMD_OPS_H

#include "dataflow_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* ---------- skeleton setters (libdataflowops/src/set_ops/set_op_skeletons.c) ---------- */

/* :160-225, nickname "default_matmul", 19 args */
void dataflow_set_matmul_skeleton(Op_Skeleton * skeleton);
/* :885-914, "default_swiglu_<DT>", 5 args */
void dataflow_set_default_swiglu_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_datatype);
/* :916-950, "default_swiglu_bwd_x_<DT>_<DT>", 7 args */
void dataflow_set_default_swiglu_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_datatype, DataflowDatatype bwd_datatype);
/* :1087-1122, "default_select_experts_<DT>", 9 args */
void dataflow_set_default_select_experts_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_datatype);
/* :1124-1157, "default_build_expert_mapping", 7 args */
void dataflow_set_default_build_expert_mapping_skeleton(Op_Skeleton * skeleton);
/* :1159-1192, "default_prepare_expert_zone_<DT>_<DT>", 7 args */
void dataflow_set_default_prepare_expert_zone_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);
/* :1194-1225, "default_prepare_experts_<DT>_<DT>", 6 args */
void dataflow_set_default_prepare_experts_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);
/* :1227-1263, "default_merge_expert_result_<DT>_<DT>", 10 args */
void dataflow_set_default_merge_expert_result_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);
/* :1265-1297, "default_merge_experts_<DT>_<DT>", 7 args */
void dataflow_set_default_merge_experts_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);
/* :1299-1338, "default_router_bwd_x_<DT>_<DT>", 13 args */
void dataflow_set_default_router_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);
/* :1340-1371, "default_router_gate_bwd_x_<DT>_<DT>", 6 args */
void dataflow_set_default_router_gate_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);

/* ---------- submit wrappers with a counterpart in the reference ---------- */

/* libdataflowops/src/submit_ops/matmul_op.c:11-66.
 * Column-major BLAS view: D[M,N] = alpha * op(A)[M,K] * op(B)[K,N] + beta * C[M,N], leading dimensions
 * implied (A: K if to_trans_a else M; B: N if to_trans_b else K; C,D: M). Read as row-major arrays:
 *   to_trans_a=1: A is [M][K]      to_trans_a=0: A is [K][M]
 *   to_trans_b=0: B is [N][K]      to_trans_b=1: B is [K][N]
 *   C, D are [N][M].
 * C is ignored when c_dt == DATAFLOW_NONE, C == NULL or beta == 0. C may equal D.
 * This backend computes bf16 inputs/outputs with fp32 accumulation (compute_dt FP32 or BF16 both map
 * to that); with compute_dt FP32 also A, B fp32 -> D fp32; A, B fp16 -> D fp16 or fp32; A, B bf16 -> D fp32, a used C
 * having D's type (matmul_helper.c:168-296). Any other combination returns -1 (fp8, fp16 accumulation, the
 * reduced-precision compute types on fp32 operands). workspace holds the partial sums of a split along K (bf16 only). */
int dataflow_submit_matmul(Dataflow_Handle * handle, int stream_id,
					DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
					DataflowDatatype compute_dt,
					int to_trans_a, int to_trans_b,
					int M, int K, int N,
					float alpha, float beta,
					void * A, void * B, void * C, void * D,
					uint64_t workspaceBytes, void * workspace);

/* mlp_misc_ops.c:3-30. out = bf16(silu(x_w1) * x_w3), fp32 math. out may alias an input. num_cols % 8 == 0. */
int dataflow_submit_default_swiglu(Dataflow_Handle * handle, int stream_id,
						DataflowDatatype fwd_dt,
						int num_rows, int num_cols,
						void * x_w1, void * x_w3, void * out);

/* mlp_misc_ops.c:32-61 */
int dataflow_submit_default_swiglu_bwd_x(Dataflow_Handle * handle, int stream_id,
						DataflowDatatype fwd_dt, DataflowDatatype bwd_dt,
						int num_rows, int num_cols,
						void * x_w1, void * x_w3,
						void * upstream_dX, void * dX_w1, void * dX_w3);

/* moe_ops.c:4-37. Caller zeroes expert_counts[0..n_experts] (n_experts+1 ints; the last is a launch ticket)
 * and expert_counts_cumsum[0..n_experts) first. Leaves the EXCLUSIVE prefix sum in expert_counts_cumsum and
 * a copy of the counts in host_expert_counts (device-visible host memory), valid after sync_stream. */
int dataflow_submit_default_select_experts(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype fwd_dt,
								int total_tokens, int n_experts, int top_k_experts,
								void * X_routed, float * token_expert_weights,
								uint16_t * chosen_experts, int * expert_counts,
								int * expert_counts_cumsum,
								int * host_expert_counts);

/* moe_ops.c:40-69. expert_counts_cumsum must hold the exclusive prefix sum of the per-expert counts of
 * chosen_experts on entry and holds the INCLUSIVE prefix sum on return. Slots inside one expert are in
 * ascending token order (the reference leaves that order to atomics timing). */
int dataflow_submit_default_build_expert_mapping(Dataflow_Handle * handle, int stream_id,
								int total_tokens, int num_routed_experts, int num_selected_experts,
								uint16_t * chosen_experts, int * expert_counts_cumsum,
								int * expert_mapping, int * token_mapping);

/* moe_ops.c:71-99. expert_zone[token_mapping[t,k], :] = X[t, :]. model_dim % 8 == 0. */
int dataflow_submit_default_prepare_experts(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int total_tokens, int model_dim, int num_selected_experts, void * X,
								int * token_mapping,
								void * expert_zone);

/* moe_ops.c:101-131. Gather of one expert's rows through expert_mapping (inclusive cumsum expected). */
int dataflow_submit_default_prepare_expert_zone(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int model_dim, void * X,
								int expert_id, int * expert_counts, int * expert_counts_cumsum,
								int * expert_mapping,
								void * expert_zone);

/* moe_ops.c:133-164. X_combined[t,:] = bf16(float(X_combined[t,:]) + sum_k w[t,k] * expert_zones[token_mapping[t,k],:]),
 * k ascending, fp32. token_expert_weights == NULL means weight 1. */
int dataflow_submit_default_merge_experts(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int model_dim, int top_k_experts,
								void * expert_zones,
								int * token_mapping,
								float * token_expert_weights,
								void * X_combined);

/* moe_ops.c:166-202. Per-expert read-modify-write combine; num_tokens is this expert's row count. */
int dataflow_submit_default_merge_expert_result(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int model_dim, int top_k_experts,
								void * expert_zone, int expert_id,
								int * expert_counts_cumsum,
								int * expert_mapping,
								float * token_expert_weights,
								uint16_t * chosen_experts,
								void * X_combined);

/* moe_ops.c:204-245. num_tokens is this expert's row count; dX_expert_out may alias expert_out. */
int dataflow_submit_router_bwd_x(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
							int num_tokens, int model_dim, int num_routed_experts, int top_k_active,
							int expert_id,
							int * expert_counts_cumsum,
							int * expert_mapping,
							uint16_t * chosen_experts,
							float * token_expert_weights,
							void * expert_out, void * upstream_dX,
							void * dX_routed,
							void * dX_expert_out);

/* moe_ops.c:247-276 */
int dataflow_submit_router_gate_bwd_x(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int num_routed_experts, int top_k_active,
								uint16_t * chosen_experts,
								float * token_expert_weights,
								void * dX_routed);

/* ---------- RMS norm around the layer (libdataflowops/include/dataflow_ops.h:148-176) ---------- */

/* set_op_skeletons.c:522-556, "default_rms_norm_<DT>" (the reference lists eight tags for its seven arguments) */
void dataflow_set_default_rms_norm_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_datatype);
/* :558-590, "default_rms_norm_recompute_<DT>", 6 args */
void dataflow_set_default_rms_norm_recompute_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_datatype);
/* :592-627, "default_rms_norm_bwd_x_<DT>_<DT>", 9 args */
void dataflow_set_default_rms_norm_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_datatype, DataflowDatatype bwd_datatype);
/* :629-669, "default_rms_norm_bwd_w_<DT>_<DT>", count 8 with a ninth tag for the workspace size */
void dataflow_set_default_rms_norm_bwd_w_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_datatype, DataflowDatatype bwd_datatype);
/* :671-705, "default_rms_norm_bwd_w_combine_<DT>", 4 args */
void dataflow_set_default_rms_norm_bwd_w_combine_skeleton(Op_Skeleton * skeleton, DataflowDatatype bwd_datatype);

/* norm_ops.c:3-26.  rms_vals[row] = rsqrt(mean(X[row]^2) + eps) (nullable), out = bf16((X * rms_val) * rms_weight) */
int dataflow_submit_default_rms_norm(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
						int n_rows, int n_cols, float eps,
						void * rms_weight, void * X, void * out, float * rms_vals);
/* norm_ops.c:28-50.  the same output from saved rms_vals */
int dataflow_submit_default_rms_norm_recompute(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
						int n_rows, int n_cols,
						void * rms_weight, float * rms_vals, void * X, void * out);
/* norm_ops.c:52-80.  accumulates into dX; X_out (nullable) receives the recomputed forward output */
int dataflow_submit_default_rms_norm_bwd_x(Dataflow_Handle * handle, int stream_id,
						DataflowDatatype fwd_dt, DataflowDatatype bwd_dt,
						int n_rows, int n_cols, float eps, float * fwd_rms_vals,
						void * rms_weight, void * X_inp, void * upstream_dX, void * dX, void * X_out);
/* norm_ops.c:82-120.  accumulates into dW; workspace: 256 bytes + (work-groups * n_cols) floats, at least one row */
int dataflow_submit_default_rms_norm_bwd_w(Dataflow_Handle * handle, int stream_id,
						DataflowDatatype fwd_dt, DataflowDatatype bwd_dt,
						int n_rows, int n_cols, float eps, float * fwd_rms_vals,
						void * X_inp, void * upstream_dX, void * dW,
						uint64_t workspaceBytes, void * workspace);

/* ---------- optimizer step for the layer's weights (libdataflowops/include/dataflow_ops.h:310-315) ---------- */

/* set_op_skeletons.c:1045-1080, "default_adamw_step_<DT>_<DT>_<DT>_<DT>", 11 args */
void dataflow_set_default_adamw_step_skeleton(Op_Skeleton * skeleton, DataflowDatatype param_dt, DataflowDatatype grad_dt,
						DataflowDatatype mean_dt, DataflowDatatype var_dt);
/* optimizer_ops.c:3-40.  AdamW in place on param, mean and var; step_num counts from 1.  BF16 for all four arrays. */
int dataflow_submit_default_adamw_step(Dataflow_Handle * handle, int stream_id,
						DataflowDatatype param_dt, DataflowDatatype grad_dt,
						DataflowDatatype mean_dt, DataflowDatatype var_dt,
						uint64_t num_els, int step_num,
						float lr, float beta1, float beta2, float weight_decay, float epsilon,
						void * param, void * grad, void * mean, void * var);

/* ---------- casts (libdataflowops/include/dataflow_ops.h:7-13; registered at register_ops.c:168-177) ---------- */

/* set_op_skeletons.c:92-122, "default_cast", 3 args (count, src, dst); C_dt is accepted and ignored as there */
void dataflow_set_default_cast_skeleton(Op_Skeleton * skeleton, DataflowDatatype A_dt, DataflowDatatype B_dt, DataflowDatatype C_dt);
/* set_op_skeletons.c:124-156, "default_cast_and_add", 6 args */
void dataflow_set_default_cast_and_add_skeleton(Op_Skeleton * skeleton, DataflowDatatype A_dt, DataflowDatatype B_dt, DataflowDatatype C_dt);
/* cast_ops.c:3-23.  dst[i] = src[i]; BF16 -> FP32 only (the one combination the reference registers) */
int dataflow_submit_cast(Dataflow_Handle * handle, int stream_id, DataflowDatatype src_dt, DataflowDatatype dst_dt,
						uint64_t num_elements, void * src, void * dst);
/* cast_ops.c:25-52 (kernel cast.cu:61-113).  C[i] = bf16(alpha * A[i]) + bf16(beta) * B[i] with the product and the sum
 * rounded to bf16; A FP32, B and C BF16 (the one combination the reference registers); C may alias B */
int dataflow_submit_cast_and_add(Dataflow_Handle * handle, int stream_id,
						DataflowDatatype A_dt, DataflowDatatype B_dt, DataflowDatatype C_dt,
						uint64_t num_els, float alpha, void * A, float beta, void * B, void * C);

/* ---------- additions: grouped one-launch forms (no counterpart in the reference) ---------- */

#define AMD_GROUPED_RAGGED_N 0   /* the N dimension of group g is n_g rows of the packed B and D */
#define AMD_GROUPED_RAGGED_K 1   /* the K dimension of group g is n_g rows of the packed A and B */

void dataflow_set_amd_grouped_matmul_skeleton(Op_Skeleton * skeleton);
void dataflow_set_amd_router_bwd_x_all_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);

/* For every group g in [0, num_groups) with n_g > 0 this does what dataflow_submit_matmul would do
 * with the ragged dimension set to n_g, in one launch, reading n_g from the device:
 *   n_g = group_rows_cumsum[g] - (g ? group_rows_cumsum[g-1] : 0)   (inclusive prefix sum, int[num_groups])
 *   base_g = group_rows_cumsum[g] - n_g
 * ragged_dim == AMD_GROUPED_RAGGED_N (requires to_trans_b == 0): N_g = n_g;
 *   A_g = A + g*strideA_bytes (a weight matrix), B_g = B + base_g*K elements, C_g/D_g = C/D + base_g*M elements.
 *   The N argument is an upper bound of sum n_g (used to size the launch).
 * ragged_dim == AMD_GROUPED_RAGGED_K (requires to_trans_a == 0, to_trans_b == 1): K_g = n_g;
 *   A_g = A + base_g*M elements, B_g = B + base_g*N elements, C_g/D_g = C/D + g*strideD_bytes.
 *   The K argument is ignored.
 *   Groups with n_g == 0 leave D untouched when a C operand is given (the accumulating form, C == D), as the reference's
 *   loop does by skipping experts without tokens; without a C operand (c_dt DATAFLOW_NONE) their D_g is written as zeros,
 *   the value of alpha times a sum over no rows, so that D never needs clearing beforehand.
 * Groups never need a host round trip: this replaces the sync + per-expert loop of
 * libdataflowmodels/src/transformer/src/dataflow_transformer.c:2789-2940. */
int dataflow_submit_amd_grouped_matmul(Dataflow_Handle * handle, int stream_id,
					DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
					DataflowDatatype compute_dt,
					int to_trans_a, int to_trans_b, int ragged_dim,
					int M, int K, int N,
					int num_groups, int * group_rows_cumsum,
					float alpha, float beta,
					void * A, uint64_t strideA_bytes, void * B, void * C, void * D, uint64_t strideD_bytes);

/* The grouped matmul with the token rows gathered on the fly.  The operand whose rows are the groups' rows -- B for
 * AMD_GROUPED_RAGGED_N (a row is K elements), A for AMD_GROUPED_RAGGED_K (a row is M elements) -- is not a packed
 * copy: row i of group g is row row_map[base_g + i] of an array of source_rows rows (below 4 GiB in all), passed in
 * that operand's place.  With the layer input X [T][D] and row_map = expert_mapping (routed row -> token) this is the
 * up-projection of dataflow_transformer.c:2859-2880 without the dispatch copy of :2804 (default_prepare_experts) in
 * front of it, and the dW1 / dW3 GEMMs of :4112-4132 without the re-dispatch of :4062.  The values that reach the
 * multiplies are those of the packed copy, so the result equals copy + dataflow_submit_amd_grouped_matmul bit for
 * bit.  The other ragged operand (A's counterpart in ragged K: B) stays packed. */
void dataflow_set_amd_grouped_matmul_gathered_skeleton(Op_Skeleton * skeleton);
int dataflow_submit_amd_grouped_matmul_gathered(Dataflow_Handle * handle, int stream_id,
					DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
					DataflowDatatype compute_dt,
					int to_trans_a, int to_trans_b, int ragged_dim,
					int M, int K, int N,
					int num_groups, int * group_rows_cumsum,
					float alpha, float beta,
					void * A, uint64_t strideA_bytes, void * B, void * C, void * D, uint64_t strideD_bytes,
					int * row_map, int source_rows);

/* router_bwd_x for all experts in one launch, token-major: for every token t and slot k with
 * r = token_mapping[t,k], e = chosen_experts[t,k]:
 *   dX_routed[t,e] = bf16(<expert_out[r,:], upstream_dX[t,:]>)   (fp32 accumulation)
 *   dX_expert_out[r,:] = bf16(upstream_dX[t,:] * bf16(token_expert_weights[t,k]))
 * which is what E calls of dataflow_submit_router_bwd_x produce. dX_expert_out may alias expert_out. */
int dataflow_submit_amd_router_bwd_x_all(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
							int num_tokens, int model_dim, int num_routed_experts, int top_k_active,
							int * token_mapping,
							uint16_t * chosen_experts,
							float * token_expert_weights,
							void * expert_out, void * upstream_dX,
							void * dX_routed,
							void * dX_expert_out);

/* default_merge_experts into a row that counts as zero: X_combined[t,:] = bf16(0 + sum_k w[t,k] * expert_zones[
 * token_mapping[t,k],:]) with the same fp32 order.  Equal, bit for bit, to clearing X_combined and calling
 * dataflow_submit_default_merge_experts (what dataflow_transformer.c:3666-3678 does for the gradient of the layer input),
 * without the fill and without reading the zeros back. */
void dataflow_set_amd_merge_experts_fresh_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);
int dataflow_submit_amd_merge_experts_fresh(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int model_dim, int top_k_experts,
								void * expert_zones, int * token_mapping, float * token_expert_weights, void * X_combined);

/* default_swiglu for inputs whose rows are not packed: row r of x_w1 / x_w3 starts x_row_stride elements after row r-1
 * (a multiple of 8, >= num_cols); out is packed.  x_w3 = x_w1 + num_cols with x_row_stride = 2 * num_cols reads the two
 * up-projections of a row side by side, as one GEMM over the stacked w1 / w3 matrices writes them. */
void dataflow_set_amd_swiglu_strided_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_dt);
int dataflow_submit_amd_swiglu_strided(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
							int num_rows, int num_cols, int x_row_stride, void * x_w1, void * x_w3, void * out);

/* prepare_experts with the row scaled by the slot's routing weight on the way:
 *   expert_zones[token_mapping[t,k], :] = bf16(X[t,:] * bf16(token_expert_weights[t,k]))
 * Run on the upstream gradient it gives the rows that router_bwd_x writes (router_bwd_x.cu:83-86) without reading the
 * expert outputs. */
void dataflow_set_amd_prepare_experts_scaled_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn_datatype, DataflowDatatype expert_datatype);
int dataflow_submit_amd_prepare_experts_scaled(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
							int total_tokens, int model_dim, int num_selected_experts,
							void * X, int * token_mapping, float * token_expert_weights, void * expert_zones);

/* The expert-side backward between the hidden-gradient GEMM and the input-gradient GEMMs when the expert outputs are
 * not recomputed (the reference recomputes them to form the router gradient, dataflow_transformer.c:3494-3535).
 * dh [num_rows][num_cols] is the hidden gradient of the w-scaled upstream rows, dh_r = (wb * dY_t) W2.  For routed
 * row r (t = expert_mapping[r], slot k with token_mapping[t,k] == r, e = chosen_experts[t,k],
 * wb = bf16(token_expert_weights[t,k])):
 *   h_out[r,:] = bf16(silu(x_w1[r,:]) * x_w3[r,:])          (what default_swiglu writes)
 *   dX_routed[t,e] = bf16(<h_out[r,:], dh[r,:]> / wb)       (= <h W2^T, dY_t>, what router_bwd_x computes from the
 *                                                            recomputed expert output; 0 where wb == 0)
 *   dX_w1[r,:], dX_w3[r,:] = swiglu_bwd_x(x_w1[r,:], x_w3[r,:], dh[r,:])    (what default_swiglu_bwd_x writes)
 * Rows of x_w1 / x_w3 start x_row_stride elements apart, rows of dX_w1 / dX_w3 dx_row_stride elements apart (multiples of
 * 8, >= num_cols); dh and h_out are packed.  With dx_row_stride == num_cols dX_w1 may alias dh.  top_k_active <= 64.
 * A deliberate difference from router_bwd_x: where the routing weight rounds to zero in bf16 (wb == 0) this op writes 0,
 * the reference a finite <y, dY> (dh carries the factor wb, so the quotient is 0 / 0 there).  The softmax-gate backward
 * that follows, p_k (d_k - sum_j p_j d_j), multiplies that entry by p_k = 0 and enters it into the sum with weight 0, so
 * nothing downstream differs; softmax weights are never zero in any case.  Likewise dataflow_submit_amd_prepare_experts_scaled
 * writes a row of zeros for such a weight where router_bwd_x writes bf16(dY * 0), the same zeros. */
void dataflow_set_amd_swiglu_bwd_x_routed_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd_dt, DataflowDatatype bwd_dt);
int dataflow_submit_amd_swiglu_bwd_x_routed(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype fwd_dt, DataflowDatatype bwd_dt,
							int num_rows, int num_cols, int num_routed_experts, int top_k_active,
							int x_row_stride, int dx_row_stride,
							int * expert_mapping, int * token_mapping,
							uint16_t * chosen_experts, float * token_expert_weights,
							void * x_w1, void * x_w3, void * dh,
							void * dX_routed, void * dX_w1, void * dX_w3, void * h_out);

#ifdef __cplusplus
}
#endif

#endif
