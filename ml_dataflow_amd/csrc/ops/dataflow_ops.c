/*
 * dataflow_ops.c -- op skeletons and submit wrappers of the MoE layer (see include/dataflow_amd_ops.h).
 *
 * A skeleton is (nickname, argument count, argument type tags); its SHA-256 is the key under which a
 * backend registers the implementation.  The tables below restate, op by op, the tags listed in
 * libdataflowops/src/set_ops/set_op_skeletons.c (line ranges per op in the header), so fingerprints
 * computed here equal the ones the reference computes.  The wrappers restate
 * libdataflowops/src/submit_ops/{moe_ops.c, matmul_op.c, mlp_misc_ops.c}.
 */
#include "dataflow_amd_ops.h"

#include <stdio.h>
#include <string.h>

#define I_S DATAFLOW_INT_SCALAR
#define F_S DATAFLOW_FP32_SCALAR

static void fill_skeleton(Op_Skeleton * skeleton, const char * base, DataflowDatatype dt0, DataflowDatatype dt1,
						  int num_args, const DataflowDatatype * arg_dtypes) {
	Op_Skeleton_Header * header = &(skeleton->header);
	/* the nickname field is hashed in full, so everything after the text must be zero */
	memset(header->op_nickname, 0, sizeof(header->op_nickname));
	if (dt0 == DATAFLOW_NONE) {
		snprintf(header->op_nickname, MAX_OP_NICKNAME_SIZE, "%s", base);
	} else if (dt1 == DATAFLOW_NONE) {
		snprintf(header->op_nickname, MAX_OP_NICKNAME_SIZE, "%s_%s", base, dataflow_datatype_as_string(dt0));
	} else {
		snprintf(header->op_nickname, MAX_OP_NICKNAME_SIZE, "%s_%s_%s", base, dataflow_datatype_as_string(dt0), dataflow_datatype_as_string(dt1));
	}
	header->num_args = num_args;
	for (int i = 0; i < MAX_OP_ARGS; i++) {
		header->arg_dtypes[i] = (i < num_args) ? arg_dtypes[i] : DATAFLOW_NONE;
	}
	dataflow_do_fingerprinting(header, sizeof(Op_Skeleton_Header), skeleton->identifier.fingerprint);
}

/* for the one skeleton whose tag list is longer than its argument count: `listed` tags are set, then hashed */
static void fill_skeleton_listed(Op_Skeleton * skeleton, const char * base, DataflowDatatype dt0, DataflowDatatype dt1,
								 int num_args, int listed, const DataflowDatatype * arg_dtypes) {
	fill_skeleton(skeleton, base, dt0, dt1, listed, arg_dtypes);
	skeleton->header.num_args = num_args;
	dataflow_do_fingerprinting(&(skeleton->header), sizeof(Op_Skeleton_Header), skeleton->identifier.fingerprint);
}

void dataflow_set_matmul_skeleton(Op_Skeleton * skeleton) {
	/* num_procs, 5 dtype tags, 2 transpose flags, M K N, alpha beta, A B C D, workspace bytes, workspace */
	const DataflowDatatype t[19] = {I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, F_S, F_S,
									DATAFLOW_VOID, DATAFLOW_VOID, DATAFLOW_VOID, DATAFLOW_VOID, DATAFLOW_UINT64, DATAFLOW_VOID};
	fill_skeleton(skeleton, "default_matmul", DATAFLOW_NONE, DATAFLOW_NONE, 19, t);
}

void dataflow_set_default_swiglu_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd) {
	const DataflowDatatype t[5] = {I_S, I_S, fwd, fwd, fwd};
	fill_skeleton(skeleton, "default_swiglu", fwd, DATAFLOW_NONE, 5, t);
}

void dataflow_set_default_swiglu_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd, DataflowDatatype bwd) {
	const DataflowDatatype t[7] = {I_S, I_S, fwd, fwd, bwd, bwd, bwd};
	fill_skeleton(skeleton, "default_swiglu_bwd_x", fwd, bwd, 7, t);
}

void dataflow_set_default_select_experts_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd) {
	const DataflowDatatype t[9] = {I_S, I_S, I_S, fwd, DATAFLOW_FP32, DATAFLOW_UINT16, DATAFLOW_INT, DATAFLOW_INT, DATAFLOW_INT};
	fill_skeleton(skeleton, "default_select_experts", fwd, DATAFLOW_NONE, 9, t);
}

void dataflow_set_default_build_expert_mapping_skeleton(Op_Skeleton * skeleton) {
	const DataflowDatatype t[7] = {I_S, I_S, I_S, DATAFLOW_UINT16, DATAFLOW_INT, DATAFLOW_INT, DATAFLOW_INT};
	fill_skeleton(skeleton, "default_build_expert_mapping", DATAFLOW_NONE, DATAFLOW_NONE, 7, t);
}

void dataflow_set_default_prepare_expert_zone_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[7] = {I_S, attn, I_S, DATAFLOW_INT, DATAFLOW_INT, DATAFLOW_INT, expert};
	fill_skeleton(skeleton, "default_prepare_expert_zone", attn, expert, 7, t);
}

void dataflow_set_default_prepare_experts_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[6] = {I_S, I_S, I_S, attn, DATAFLOW_INT, expert};
	fill_skeleton(skeleton, "default_prepare_experts", attn, expert, 6, t);
}

void dataflow_set_default_merge_expert_result_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[10] = {I_S, I_S, I_S, expert, I_S, DATAFLOW_INT, DATAFLOW_INT, DATAFLOW_FP32, DATAFLOW_UINT16, attn};
	fill_skeleton(skeleton, "default_merge_expert_result", attn, expert, 10, t);
}

void dataflow_set_default_merge_experts_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[7] = {I_S, I_S, I_S, expert, DATAFLOW_INT, DATAFLOW_FP32, attn};
	fill_skeleton(skeleton, "default_merge_experts", attn, expert, 7, t);
}

void dataflow_set_default_router_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[13] = {I_S, I_S, I_S, I_S, I_S, DATAFLOW_INT, DATAFLOW_INT, DATAFLOW_UINT16, DATAFLOW_FP32,
									expert, attn, attn, expert};
	fill_skeleton(skeleton, "default_router_bwd_x", attn, expert, 13, t);
}

void dataflow_set_default_router_gate_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[6] = {I_S, I_S, I_S, DATAFLOW_UINT16, DATAFLOW_FP32, attn};
	fill_skeleton(skeleton, "default_router_gate_bwd_x", attn, expert, 6, t);
}

/* ---- RMS norm (set_op_skeletons.c:522-705).  The tag lists are the reference's, including the forward
 * skeleton's eight tags for seven arguments and the ninth tag of bwd_w behind its count of eight: the
 * fingerprint is taken over whatever the reference writes. ---- */

void dataflow_set_default_rms_norm_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd) {
	const DataflowDatatype t[8] = {I_S, I_S, I_S, fwd, DATAFLOW_FP32, DATAFLOW_UINT16, DATAFLOW_INT, DATAFLOW_INT};
	fill_skeleton(skeleton, "default_rms_norm", fwd, DATAFLOW_NONE, 8, t);
}

void dataflow_set_default_rms_norm_recompute_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd) {
	const DataflowDatatype t[6] = {I_S, I_S, fwd, DATAFLOW_FP32, fwd, fwd};
	fill_skeleton(skeleton, "default_rms_norm_recompute", fwd, DATAFLOW_NONE, 6, t);
}

void dataflow_set_default_rms_norm_bwd_x_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd, DataflowDatatype bwd) {
	const DataflowDatatype t[9] = {I_S, I_S, F_S, DATAFLOW_FP32, fwd, fwd, bwd, bwd, fwd};
	fill_skeleton(skeleton, "default_rms_norm_bwd_x", fwd, bwd, 9, t);
}

void dataflow_set_default_rms_norm_bwd_w_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd, DataflowDatatype bwd) {
	const DataflowDatatype t[9] = {I_S, I_S, F_S, DATAFLOW_FP32, fwd, bwd, DATAFLOW_FP32, DATAFLOW_INT, DATAFLOW_UINT64_SCALAR};
	fill_skeleton_listed(skeleton, "default_rms_norm_bwd_w", fwd, bwd, 8, 9, t);
}

void dataflow_set_default_rms_norm_bwd_w_combine_skeleton(Op_Skeleton * skeleton, DataflowDatatype bwd) {
	const DataflowDatatype t[4] = {DATAFLOW_INT, I_S, DATAFLOW_FP32, bwd};
	fill_skeleton(skeleton, "default_rms_norm_bwd_w_combine", bwd, DATAFLOW_NONE, 4, t);
}

/* ---- AdamW (set_op_skeletons.c:1045-1080): "default_adamw_step_<param>_<grad>_<mean>_<var>", 11 args ---- */

void dataflow_set_default_adamw_step_skeleton(Op_Skeleton * skeleton, DataflowDatatype param_dt, DataflowDatatype grad_dt,
											  DataflowDatatype mean_dt, DataflowDatatype var_dt) {
	const DataflowDatatype t[11] = {DATAFLOW_UINT64_SCALAR, I_S, F_S, F_S, F_S, F_S, F_S, param_dt, grad_dt, mean_dt, var_dt};
	char base[MAX_OP_NICKNAME_SIZE];
	snprintf(base, sizeof(base), "default_adamw_step_%s_%s", dataflow_datatype_as_string(param_dt), dataflow_datatype_as_string(grad_dt));
	fill_skeleton(skeleton, base, mean_dt, var_dt, 11, t);
}

/* ---- casts (set_op_skeletons.c:92-156): the nicknames carry no dtype suffix, the argument tags do ---- */

void dataflow_set_default_cast_skeleton(Op_Skeleton * skeleton, DataflowDatatype A_dt, DataflowDatatype B_dt, DataflowDatatype C_dt) {
	(void) C_dt;                                  /* part of the reference's signature, not of the op's identity */
	const DataflowDatatype t[3] = {DATAFLOW_UINT64_SCALAR, A_dt, B_dt};
	fill_skeleton(skeleton, "default_cast", DATAFLOW_NONE, DATAFLOW_NONE, 3, t);
}

void dataflow_set_default_cast_and_add_skeleton(Op_Skeleton * skeleton, DataflowDatatype A_dt, DataflowDatatype B_dt, DataflowDatatype C_dt) {
	const DataflowDatatype t[6] = {DATAFLOW_UINT64_SCALAR, F_S, A_dt, F_S, B_dt, C_dt};
	fill_skeleton(skeleton, "default_cast_and_add", DATAFLOW_NONE, DATAFLOW_NONE, 6, t);
}

/* ---- additions ---- */

void dataflow_set_amd_grouped_matmul_skeleton(Op_Skeleton * skeleton) {
	/* num_procs, 5 dtype tags, transa, transb, ragged_dim, M K N, num_groups, cumsum, alpha beta,
	 * A strideA B C D strideD */
	const DataflowDatatype t[22] = {I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, DATAFLOW_INT, F_S, F_S,
									DATAFLOW_VOID, DATAFLOW_UINT64_SCALAR, DATAFLOW_VOID, DATAFLOW_VOID, DATAFLOW_VOID, DATAFLOW_UINT64_SCALAR};
	fill_skeleton(skeleton, "amd_grouped_matmul", DATAFLOW_NONE, DATAFLOW_NONE, 22, t);
}

void dataflow_set_amd_grouped_matmul_gathered_skeleton(Op_Skeleton * skeleton) {
	/* the grouped matmul's 22 arguments, then the row map and the number of rows the gathered operand has */
	const DataflowDatatype t[24] = {I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, I_S, DATAFLOW_INT, F_S, F_S,
									DATAFLOW_VOID, DATAFLOW_UINT64_SCALAR, DATAFLOW_VOID, DATAFLOW_VOID, DATAFLOW_VOID, DATAFLOW_UINT64_SCALAR,
									DATAFLOW_INT, I_S};
	fill_skeleton(skeleton, "amd_grouped_matmul_gathered", DATAFLOW_NONE, DATAFLOW_NONE, 24, t);
}

void dataflow_set_amd_router_bwd_x_all_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[11] = {I_S, I_S, I_S, I_S, DATAFLOW_INT, DATAFLOW_UINT16, DATAFLOW_FP32, expert, attn, attn, expert};
	fill_skeleton(skeleton, "amd_router_bwd_x_all", attn, expert, 11, t);
}

void dataflow_set_amd_prepare_experts_scaled_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[7] = {I_S, I_S, I_S, attn, DATAFLOW_INT, DATAFLOW_FP32, expert};
	fill_skeleton(skeleton, "amd_prepare_experts_scaled", attn, expert, 7, t);
}

void dataflow_set_amd_swiglu_bwd_x_routed_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd, DataflowDatatype bwd) {
	const DataflowDatatype t[17] = {I_S, I_S, I_S, I_S, I_S, I_S, DATAFLOW_INT, DATAFLOW_INT, DATAFLOW_UINT16, DATAFLOW_FP32, fwd, fwd, bwd, bwd, bwd, bwd, fwd};
	fill_skeleton(skeleton, "amd_swiglu_bwd_x_routed", fwd, bwd, 17, t);
}

void dataflow_set_amd_merge_experts_fresh_skeleton(Op_Skeleton * skeleton, DataflowDatatype attn, DataflowDatatype expert) {
	const DataflowDatatype t[7] = {I_S, I_S, I_S, expert, DATAFLOW_INT, DATAFLOW_FP32, attn};
	fill_skeleton(skeleton, "amd_merge_experts_fresh", attn, expert, 7, t);
}

void dataflow_set_amd_swiglu_strided_skeleton(Op_Skeleton * skeleton, DataflowDatatype fwd) {
	const DataflowDatatype t[6] = {I_S, I_S, I_S, fwd, fwd, fwd};
	fill_skeleton(skeleton, "amd_swiglu_strided", fwd, DATAFLOW_NONE, 6, t);
}

/* ------------------------------------------------------------------ submit wrappers */

static int submit(Dataflow_Handle * handle, Op * op, int stream_id, const char * what) {
	if (!handle || !handle->submit_op) {
		fprintf(stderr, "Error: %s submitted to a handle with no submit_op...\n", what);
		return -1;
	}
	if ((handle->submit_op)(handle, op, stream_id)) {
		fprintf(stderr, "Error: failed to submit %s op...\n", what);
		return -1;
	}
	return 0;
}

int dataflow_submit_matmul(Dataflow_Handle * handle, int stream_id,
					DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
					DataflowDatatype compute_dt,
					int to_trans_a, int to_trans_b,
					int M, int K, int N,
					float alpha, float beta,
					void * A, void * B, void * C, void * D,
					uint64_t workspaceBytes, void * workspace) {
	Op op;
	dataflow_set_matmul_skeleton(&op.op_skeleton);
	int num_procs = (handle->get_num_procs)(handle);
	void ** a = op.op_args;
	a[0] = &num_procs;
	a[1] = &a_dt; a[2] = &b_dt; a[3] = &c_dt; a[4] = &d_dt; a[5] = &compute_dt;
	a[6] = &to_trans_a; a[7] = &to_trans_b;
	a[8] = &M; a[9] = &K; a[10] = &N;
	a[11] = &alpha; a[12] = &beta;
	a[13] = &A; a[14] = &B; a[15] = &C; a[16] = &D;
	a[17] = &workspaceBytes; a[18] = &workspace;
	return submit(handle, &op, stream_id, "matmul");
}

int dataflow_submit_default_swiglu(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
						int num_rows, int num_cols, void * x_w1, void * x_w3, void * out) {
	Op op;
	dataflow_set_default_swiglu_skeleton(&op.op_skeleton, fwd_dt);
	void ** a = op.op_args;
	a[0] = &num_rows; a[1] = &num_cols; a[2] = &x_w1; a[3] = &x_w3; a[4] = &out;
	return submit(handle, &op, stream_id, "swiglu");
}

int dataflow_submit_default_swiglu_bwd_x(Dataflow_Handle * handle, int stream_id,
						DataflowDatatype fwd_dt, DataflowDatatype bwd_dt, int num_rows, int num_cols,
						void * x_w1, void * x_w3, void * upstream_dX, void * dX_w1, void * dX_w3) {
	Op op;
	dataflow_set_default_swiglu_bwd_x_skeleton(&op.op_skeleton, fwd_dt, bwd_dt);
	void ** a = op.op_args;
	a[0] = &num_rows; a[1] = &num_cols; a[2] = &x_w1; a[3] = &x_w3; a[4] = &upstream_dX; a[5] = &dX_w1; a[6] = &dX_w3;
	return submit(handle, &op, stream_id, "swiglu bwd x");
}

int dataflow_submit_default_select_experts(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
								int total_tokens, int n_experts, int top_k_experts,
								void * X_routed, float * token_expert_weights,
								uint16_t * chosen_experts, int * expert_counts,
								int * expert_counts_cumsum, int * host_expert_counts) {
	Op op;
	dataflow_set_default_select_experts_skeleton(&op.op_skeleton, fwd_dt);
	void ** a = op.op_args;
	a[0] = &total_tokens; a[1] = &n_experts; a[2] = &top_k_experts;
	a[3] = &X_routed; a[4] = &token_expert_weights; a[5] = &chosen_experts;
	a[6] = &expert_counts; a[7] = &expert_counts_cumsum; a[8] = &host_expert_counts;
	return submit(handle, &op, stream_id, "select experts");
}

int dataflow_submit_default_build_expert_mapping(Dataflow_Handle * handle, int stream_id,
								int total_tokens, int num_routed_experts, int num_selected_experts,
								uint16_t * chosen_experts, int * expert_counts_cumsum,
								int * expert_mapping, int * token_mapping) {
	Op op;
	dataflow_set_default_build_expert_mapping_skeleton(&op.op_skeleton);
	void ** a = op.op_args;
	a[0] = &total_tokens; a[1] = &num_routed_experts; a[2] = &num_selected_experts;
	a[3] = &chosen_experts; a[4] = &expert_counts_cumsum; a[5] = &expert_mapping; a[6] = &token_mapping;
	return submit(handle, &op, stream_id, "build expert mapping");
}

int dataflow_submit_default_prepare_experts(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int total_tokens, int model_dim, int num_selected_experts, void * X,
								int * token_mapping, void * expert_zone) {
	Op op;
	dataflow_set_default_prepare_experts_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &total_tokens; a[1] = &model_dim; a[2] = &num_selected_experts; a[3] = &X; a[4] = &token_mapping; a[5] = &expert_zone;
	return submit(handle, &op, stream_id, "prepare experts");
}

int dataflow_submit_default_prepare_expert_zone(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int model_dim, void * X,
								int expert_id, int * expert_counts, int * expert_counts_cumsum,
								int * expert_mapping, void * expert_zone) {
	Op op;
	dataflow_set_default_prepare_expert_zone_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &model_dim; a[1] = &X; a[2] = &expert_id; a[3] = &expert_counts; a[4] = &expert_counts_cumsum;
	a[5] = &expert_mapping; a[6] = &expert_zone;
	return submit(handle, &op, stream_id, "prepare expert zone");
}

int dataflow_submit_default_merge_experts(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int model_dim, int top_k_experts,
								void * expert_zones, int * token_mapping, float * token_expert_weights, void * X_combined) {
	Op op;
	dataflow_set_default_merge_experts_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &num_tokens; a[1] = &model_dim; a[2] = &top_k_experts; a[3] = &expert_zones;
	a[4] = &token_mapping; a[5] = &token_expert_weights; a[6] = &X_combined;
	return submit(handle, &op, stream_id, "merge experts");
}

int dataflow_submit_default_merge_expert_result(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int model_dim, int top_k_experts,
								void * expert_zone, int expert_id,
								int * expert_counts_cumsum, int * expert_mapping,
								float * token_expert_weights, uint16_t * chosen_experts, void * X_combined) {
	Op op;
	dataflow_set_default_merge_expert_result_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &num_tokens; a[1] = &model_dim; a[2] = &top_k_experts; a[3] = &expert_zone; a[4] = &expert_id;
	a[5] = &expert_counts_cumsum; a[6] = &expert_mapping; a[7] = &token_expert_weights; a[8] = &chosen_experts;
	a[9] = &X_combined;
	return submit(handle, &op, stream_id, "merge expert result");
}

int dataflow_submit_router_bwd_x(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
							int num_tokens, int model_dim, int num_routed_experts, int top_k_active,
							int expert_id, int * expert_counts_cumsum, int * expert_mapping,
							uint16_t * chosen_experts, float * token_expert_weights,
							void * expert_out, void * upstream_dX, void * dX_routed, void * dX_expert_out) {
	Op op;
	dataflow_set_default_router_bwd_x_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &num_tokens; a[1] = &model_dim; a[2] = &num_routed_experts; a[3] = &top_k_active; a[4] = &expert_id;
	a[5] = &expert_counts_cumsum; a[6] = &expert_mapping; a[7] = &chosen_experts; a[8] = &token_expert_weights;
	a[9] = &expert_out; a[10] = &upstream_dX; a[11] = &dX_routed; a[12] = &dX_expert_out;
	return submit(handle, &op, stream_id, "router bwd x");
}

int dataflow_submit_router_gate_bwd_x(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int num_routed_experts, int top_k_active,
								uint16_t * chosen_experts, float * token_expert_weights, void * dX_routed) {
	Op op;
	dataflow_set_default_router_gate_bwd_x_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &num_tokens; a[1] = &num_routed_experts; a[2] = &top_k_active;
	a[3] = &chosen_experts; a[4] = &token_expert_weights; a[5] = &dX_routed;
	return submit(handle, &op, stream_id, "router gate bwd x");
}

int dataflow_submit_amd_grouped_matmul(Dataflow_Handle * handle, int stream_id,
					DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
					DataflowDatatype compute_dt,
					int to_trans_a, int to_trans_b, int ragged_dim,
					int M, int K, int N,
					int num_groups, int * group_rows_cumsum,
					float alpha, float beta,
					void * A, uint64_t strideA_bytes, void * B, void * C, void * D, uint64_t strideD_bytes) {
	Op op;
	dataflow_set_amd_grouped_matmul_skeleton(&op.op_skeleton);
	int num_procs = (handle->get_num_procs)(handle);
	void ** a = op.op_args;
	a[0] = &num_procs;
	a[1] = &a_dt; a[2] = &b_dt; a[3] = &c_dt; a[4] = &d_dt; a[5] = &compute_dt;
	a[6] = &to_trans_a; a[7] = &to_trans_b; a[8] = &ragged_dim;
	a[9] = &M; a[10] = &K; a[11] = &N;
	a[12] = &num_groups; a[13] = &group_rows_cumsum;
	a[14] = &alpha; a[15] = &beta;
	a[16] = &A; a[17] = &strideA_bytes; a[18] = &B; a[19] = &C; a[20] = &D; a[21] = &strideD_bytes;
	return submit(handle, &op, stream_id, "grouped matmul");
}

int dataflow_submit_amd_grouped_matmul_gathered(Dataflow_Handle * handle, int stream_id,
					DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
					DataflowDatatype compute_dt,
					int to_trans_a, int to_trans_b, int ragged_dim,
					int M, int K, int N,
					int num_groups, int * group_rows_cumsum,
					float alpha, float beta,
					void * A, uint64_t strideA_bytes, void * B, void * C, void * D, uint64_t strideD_bytes,
					int * row_map, int source_rows) {
	Op op;
	dataflow_set_amd_grouped_matmul_gathered_skeleton(&op.op_skeleton);
	int num_procs = (handle->get_num_procs)(handle);
	void ** a = op.op_args;
	a[0] = &num_procs;
	a[1] = &a_dt; a[2] = &b_dt; a[3] = &c_dt; a[4] = &d_dt; a[5] = &compute_dt;
	a[6] = &to_trans_a; a[7] = &to_trans_b; a[8] = &ragged_dim;
	a[9] = &M; a[10] = &K; a[11] = &N;
	a[12] = &num_groups; a[13] = &group_rows_cumsum;
	a[14] = &alpha; a[15] = &beta;
	a[16] = &A; a[17] = &strideA_bytes; a[18] = &B; a[19] = &C; a[20] = &D; a[21] = &strideD_bytes;
	a[22] = &row_map; a[23] = &source_rows;
	return submit(handle, &op, stream_id, "gathered grouped matmul");
}

int dataflow_submit_amd_router_bwd_x_all(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
							int num_tokens, int model_dim, int num_routed_experts, int top_k_active,
							int * token_mapping, uint16_t * chosen_experts, float * token_expert_weights,
							void * expert_out, void * upstream_dX, void * dX_routed, void * dX_expert_out) {
	Op op;
	dataflow_set_amd_router_bwd_x_all_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &num_tokens; a[1] = &model_dim; a[2] = &num_routed_experts; a[3] = &top_k_active;
	a[4] = &token_mapping; a[5] = &chosen_experts; a[6] = &token_expert_weights;
	a[7] = &expert_out; a[8] = &upstream_dX; a[9] = &dX_routed; a[10] = &dX_expert_out;
	return submit(handle, &op, stream_id, "router bwd x (all experts)");
}

int dataflow_submit_amd_prepare_experts_scaled(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
							int total_tokens, int model_dim, int num_selected_experts,
							void * X, int * token_mapping, float * token_expert_weights, void * expert_zones) {
	Op op;
	dataflow_set_amd_prepare_experts_scaled_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &total_tokens; a[1] = &model_dim; a[2] = &num_selected_experts;
	a[3] = &X; a[4] = &token_mapping; a[5] = &token_expert_weights; a[6] = &expert_zones;
	return submit(handle, &op, stream_id, "prepare experts (scaled)");
}

int dataflow_submit_amd_swiglu_bwd_x_routed(Dataflow_Handle * handle, int stream_id,
							DataflowDatatype fwd_dt, DataflowDatatype bwd_dt,
							int num_rows, int num_cols, int num_routed_experts, int top_k_active,
							int x_row_stride, int dx_row_stride,
							int * expert_mapping, int * token_mapping, uint16_t * chosen_experts, float * token_expert_weights,
							void * x_w1, void * x_w3, void * dh, void * dX_routed, void * dX_w1, void * dX_w3, void * h_out) {
	Op op;
	dataflow_set_amd_swiglu_bwd_x_routed_skeleton(&op.op_skeleton, fwd_dt, bwd_dt);
	void ** a = op.op_args;
	a[0] = &num_rows; a[1] = &num_cols; a[2] = &num_routed_experts; a[3] = &top_k_active; a[4] = &x_row_stride; a[5] = &dx_row_stride;
	a[6] = &expert_mapping; a[7] = &token_mapping; a[8] = &chosen_experts; a[9] = &token_expert_weights;
	a[10] = &x_w1; a[11] = &x_w3; a[12] = &dh; a[13] = &dX_routed; a[14] = &dX_w1; a[15] = &dX_w3; a[16] = &h_out;
	return submit(handle, &op, stream_id, "swiglu bwd x (routed)");
}

int dataflow_submit_amd_merge_experts_fresh(Dataflow_Handle * handle, int stream_id,
								DataflowDatatype attn_datatype, DataflowDatatype expert_datatype,
								int num_tokens, int model_dim, int top_k_experts,
								void * expert_zones, int * token_mapping, float * token_expert_weights, void * X_combined) {
	Op op;
	dataflow_set_amd_merge_experts_fresh_skeleton(&op.op_skeleton, attn_datatype, expert_datatype);
	void ** a = op.op_args;
	a[0] = &num_tokens; a[1] = &model_dim; a[2] = &top_k_experts; a[3] = &expert_zones;
	a[4] = &token_mapping; a[5] = &token_expert_weights; a[6] = &X_combined;
	return submit(handle, &op, stream_id, "merge experts (fresh)");
}

int dataflow_submit_amd_swiglu_strided(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
							int num_rows, int num_cols, int x_row_stride, void * x_w1, void * x_w3, void * out) {
	Op op;
	dataflow_set_amd_swiglu_strided_skeleton(&op.op_skeleton, fwd_dt);
	void ** a = op.op_args;
	a[0] = &num_rows; a[1] = &num_cols; a[2] = &x_row_stride; a[3] = &x_w1; a[4] = &x_w3; a[5] = &out;
	return submit(handle, &op, stream_id, "swiglu (strided)");
}

/* ---- RMS norm wrappers (libdataflowops/src/submit_ops/norm_ops.c:3-120) ---- */

int dataflow_submit_default_rms_norm(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
									 int n_rows, int n_cols, float eps,
									 void * rms_weight, void * X, void * out, float * rms_vals) {
	Op op;
	dataflow_set_default_rms_norm_skeleton(&op.op_skeleton, fwd_dt);
	void ** a = op.op_args;
	a[0] = &n_rows; a[1] = &n_cols; a[2] = &eps; a[3] = &rms_weight; a[4] = &X; a[5] = &out; a[6] = &rms_vals;
	return submit(handle, &op, stream_id, "rms norm");
}

int dataflow_submit_default_rms_norm_recompute(Dataflow_Handle * handle, int stream_id, DataflowDatatype fwd_dt,
											   int n_rows, int n_cols,
											   void * rms_weight, float * rms_vals, void * X, void * out) {
	Op op;
	dataflow_set_default_rms_norm_recompute_skeleton(&op.op_skeleton, fwd_dt);
	void ** a = op.op_args;
	a[0] = &n_rows; a[1] = &n_cols; a[2] = &rms_weight; a[3] = &rms_vals; a[4] = &X; a[5] = &out;
	return submit(handle, &op, stream_id, "rms norm recompute");
}

int dataflow_submit_default_rms_norm_bwd_x(Dataflow_Handle * handle, int stream_id,
										   DataflowDatatype fwd_dt, DataflowDatatype bwd_dt,
										   int n_rows, int n_cols, float eps, float * fwd_rms_vals,
										   void * rms_weight, void * X_inp, void * upstream_dX, void * dX, void * X_out) {
	Op op;
	dataflow_set_default_rms_norm_bwd_x_skeleton(&op.op_skeleton, fwd_dt, bwd_dt);
	void ** a = op.op_args;
	a[0] = &n_rows; a[1] = &n_cols; a[2] = &eps; a[3] = &fwd_rms_vals; a[4] = &rms_weight; a[5] = &X_inp;
	a[6] = &upstream_dX; a[7] = &dX; a[8] = &X_out;
	return submit(handle, &op, stream_id, "rms norm bwd x");
}

/* two submissions, as in the reference: partial sums per work-group into the workspace (a 256-byte header with
 * the work-group count, then fp32 rows), then the reduction into dW */
int dataflow_submit_default_rms_norm_bwd_w(Dataflow_Handle * handle, int stream_id,
										   DataflowDatatype fwd_dt, DataflowDatatype bwd_dt,
										   int n_rows, int n_cols, float eps, float * fwd_rms_vals,
										   void * X_inp, void * upstream_dX, void * dW,
										   uint64_t workspaceBytes, void * workspace) {
	if (!workspace) {
		fprintf(stderr, "Error: rms norm bwd w needs a workspace...\n");
		return -1;
	}
	int * ret_num_blocks_launched = (int *) workspace;
	float * dW_workspace = (float *) ((char *) workspace + 256);
	Op op;
	dataflow_set_default_rms_norm_bwd_w_skeleton(&op.op_skeleton, fwd_dt, bwd_dt);
	void ** a = op.op_args;
	a[0] = &n_rows; a[1] = &n_cols; a[2] = &eps; a[3] = &fwd_rms_vals; a[4] = &X_inp; a[5] = &upstream_dX;
	a[6] = &dW_workspace; a[7] = &ret_num_blocks_launched; a[8] = &workspaceBytes;
	if (submit(handle, &op, stream_id, "rms norm bwd w")) {
		return -1;
	}
	Op combine;
	dataflow_set_default_rms_norm_bwd_w_combine_skeleton(&combine.op_skeleton, bwd_dt);
	a = combine.op_args;
	a[0] = &ret_num_blocks_launched; a[1] = &n_cols; a[2] = &dW_workspace; a[3] = &dW;
	return submit(handle, &combine, stream_id, "rms norm bwd w combine");
}

/* ---- AdamW wrapper (libdataflowops/src/submit_ops/optimizer_ops.c:3-40) ---- */

int dataflow_submit_default_adamw_step(Dataflow_Handle * handle, int stream_id,
									   DataflowDatatype param_dt, DataflowDatatype grad_dt, DataflowDatatype mean_dt, DataflowDatatype var_dt,
									   uint64_t num_els, int step_num,
									   float lr, float beta1, float beta2, float weight_decay, float epsilon,
									   void * param, void * grad, void * mean, void * var) {
	Op op;
	dataflow_set_default_adamw_step_skeleton(&op.op_skeleton, param_dt, grad_dt, mean_dt, var_dt);
	void ** a = op.op_args;
	a[0] = &num_els; a[1] = &step_num; a[2] = &lr; a[3] = &beta1; a[4] = &beta2; a[5] = &weight_decay; a[6] = &epsilon;
	a[7] = &param; a[8] = &grad; a[9] = &mean; a[10] = &var;
	return submit(handle, &op, stream_id, "adamw step");
}

/* ---- cast wrappers (libdataflowops/src/submit_ops/cast_ops.c:3-52) ---- */

int dataflow_submit_cast(Dataflow_Handle * handle, int stream_id, DataflowDatatype src_dt, DataflowDatatype dst_dt,
						 uint64_t num_elements, void * src, void * dst) {
	Op op;
	dataflow_set_default_cast_skeleton(&op.op_skeleton, src_dt, dst_dt, DATAFLOW_NONE);
	void ** a = op.op_args;
	a[0] = &num_elements; a[1] = &src; a[2] = &dst;
	return submit(handle, &op, stream_id, "cast");
}

/* The reference's wrapper stores A, B and C themselves in the argument slots (cast_ops.c:39-42) where every other
 * wrapper stores the address of the argument; a launch would then read the kernel's pointer parameters out of the
 * device buffers.  It has no caller in the reference.  This wrapper passes the addresses, like all the others. */
int dataflow_submit_cast_and_add(Dataflow_Handle * handle, int stream_id,
								 DataflowDatatype A_dt, DataflowDatatype B_dt, DataflowDatatype C_dt,
								 uint64_t num_els, float alpha, void * A, float beta, void * B, void * C) {
	Op op;
	dataflow_set_default_cast_and_add_skeleton(&op.op_skeleton, A_dt, B_dt, C_dt);
	void ** a = op.op_args;
	a[0] = &num_els; a[1] = &alpha; a[2] = &A; a[3] = &beta; a[4] = &B; a[5] = &C;
	return submit(handle, &op, stream_id, "cast and add");
}
