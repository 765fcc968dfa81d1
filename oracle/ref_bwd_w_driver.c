/*
 * ref_bwd_w_driver.c -- TEST INFRASTRUCTURE, built only where the reference tree is mounted (oracle/Makefile, target
 * `ref`, output oracle/_ref/libref_models.so).  Nothing in the product links or loads it.
 *
 * It is compiled against the reference's own headers together with the reference's own
 * libdataflowmodels/src/transformer/src/dataflow_transformer.c and prep_seq_batch.c and its submit wrappers, and does
 * one thing: fill the reference's structs (Transformer_Block, Seq_Batch, Seq_Batch_Saved_Activations,
 * Seq_Batch_Activation_Workspace, as declared in libdataflowmodels/include/transformer/*.h) from flat arguments and call
 * the reference's dataflow_submit_transformer_moe_block_bwd_w (dataflow_transformer.c:3970-4247) on whatever
 * Dataflow_Handle it is given.  The per-expert x_1 / x_3 pointers come from the reference's own
 * set_moe_working_activations_offsets (prep_seq_batch.c:370-397).  A ctypes caller cannot fill those structs safely;
 * this file is the stub a C caller would write.
 */
#include <stdlib.h>
#include <string.h>

#include "dataflow_transformer.h"

typedef struct ref_bwd_w_args {
	/* shape */
	int total_q, model_dim, attn_dim, kv_dim, ffn_dim;
	int num_routed_experts, top_k_experts;
	int block_dt, compute_dt;                       /* DataflowDatatype values */
	int * host_expert_counts;                       /* [num_routed_experts], host */
	/* saved forward activations (device) */
	int * token_mapping;                            /* [total_q][top_k] */
	void * x_attn_out;                              /* [total_q][attn_dim] */
	/* backward working activations (device) */
	void * recomputed_ffn_norm;                     /* [total_q][model_dim]: the layer input X */
	void * recomputed_attn_norm;                    /* [total_q][model_dim] */
	void * dx1_base, * dx3_base;                    /* [total_q*top_k][ffn_dim] each: gradients of x1 / x3, expert-major rows */
	void * d_routed;                                /* [total_q][num_routed_experts] router-logit gradients */
	void * d_o, * d_q, * d_k_local, * d_v_local;    /* upstream gradients of the attention projections */
	/* workspace (device) */
	void * expert_zones;                            /* [total_q*top_k][model_dim] */
	void * kernel_workspace;
	uint64_t kernel_workspace_bytes;
	/* weight gradients (device): expert e's dW1 / dW3 at base + e * expert_stride_bytes */
	void * dw1_base, * dw3_base;
	uint64_t expert_stride_bytes;
	void * dw_router, * dw_o, * dw_q, * dw_k, * dw_v;
} Ref_Bwd_W_Args;

int ref_moe_block_bwd_w(Dataflow_Handle * handle, int compute_stream_id, int secondary_compute_stream_id, const Ref_Bwd_W_Args * a) {
	const int E = a->num_routed_experts;

	Transformer_Block grad_weights;
	memset(&grad_weights, 0, sizeof(grad_weights));
	grad_weights.config.block_dt = (DataflowDatatype) a->block_dt;
	grad_weights.config.compute_dt = (DataflowDatatype) a->compute_dt;
	grad_weights.config.model_dim = a->model_dim;
	grad_weights.config.attn_dim = a->attn_dim;
	grad_weights.config.kv_dim = a->kv_dim;
	grad_weights.config.ffn_dim = a->ffn_dim;
	grad_weights.config.moe_config.top_k_experts = a->top_k_experts;
	grad_weights.config.moe_config.num_shared_experts = 0;
	grad_weights.config.moe_config.num_global_routed_experts = E;
	grad_weights.config.moe_config.num_local_experts = E;
	grad_weights.layer_id = 0;
	grad_weights.w_router = a->dw_router;
	grad_weights.w_o = a->dw_o;
	grad_weights.w_q = a->dw_q;
	grad_weights.w_k = a->dw_k;
	grad_weights.w_v = a->dw_v;
	void ** w_1 = (void **) calloc((size_t) E, sizeof(void *));
	void ** w_3 = (void **) calloc((size_t) E, sizeof(void *));
	void ** x_1 = (void **) calloc((size_t) E, sizeof(void *));
	void ** x_3 = (void **) calloc((size_t) E, sizeof(void *));
	if (!w_1 || !w_3 || !x_1 || !x_3) {
		free(w_1); free(w_3); free(x_1); free(x_3);
		return -1;
	}
	for (int e = 0; e < E; e++) {
		w_1[e] = (char *) a->dw1_base + (uint64_t) e * a->expert_stride_bytes;
		w_3[e] = (char *) a->dw3_base + (uint64_t) e * a->expert_stride_bytes;
	}
	grad_weights.w_1 = w_1;
	grad_weights.w_3 = w_3;

	Seq_Batch seq_batch;
	memset(&seq_batch, 0, sizeof(seq_batch));
	seq_batch.attention_config.num_seqs = 1;
	seq_batch.attention_config.total_q = a->total_q;
	seq_batch.attention_config.total_k = a->total_q;
	seq_batch.moe_config.host_expert_counts = a->host_expert_counts;       /* layer 0: offset 0 */

	Transformer_Block_Transition grad_stream;
	memset(&grad_stream, 0, sizeof(grad_stream));
	grad_stream.seq_batch = &seq_batch;

	Seq_Batch_Saved_Activations fwd_activations;
	memset(&fwd_activations, 0, sizeof(fwd_activations));
	fwd_activations.seq_batch = &seq_batch;
	fwd_activations.token_mapping = a->token_mapping;
	fwd_activations.x_attn_out = a->x_attn_out;

	Seq_Batch_Recomputed_Activations recomputed;
	memset(&recomputed, 0, sizeof(recomputed));
	recomputed.recomputed_ffn_norm = a->recomputed_ffn_norm;
	recomputed.recomputed_attn_norm = a->recomputed_attn_norm;

	Seq_Batch_Saved_Activations bwd_activations;
	memset(&bwd_activations, 0, sizeof(bwd_activations));
	bwd_activations.seq_batch = &seq_batch;
	bwd_activations.recomputed_activations = &recomputed;
	bwd_activations.x_routed = a->d_routed;
	bwd_activations.x_o = a->d_o;
	bwd_activations.x_q = a->d_q;
	bwd_activations.x_k_local = a->d_k_local;
	bwd_activations.x_v_local = a->d_v_local;
	bwd_activations.x_1 = x_1;
	bwd_activations.x_3 = x_3;
	x_1[0] = a->dx1_base;
	x_3[0] = a->dx3_base;
	/* the reference's own partitioning of the x_1 / x_3 workspace by the host-side expert counts */
	int routed = set_moe_working_activations_offsets(&bwd_activations, a->total_q, a->model_dim, a->ffn_dim, 0, E, a->host_expert_counts,
													 dataflow_sizeof_element((DataflowDatatype) a->block_dt));
	int ret = -1;
	if (routed == a->total_q * a->top_k_experts) {
		Seq_Batch_Activation_Workspace workspace;
		memset(&workspace, 0, sizeof(workspace));
		workspace.x_expert_zones = a->expert_zones;
		workspace.kernelWorkspace = a->kernel_workspace;
		workspace.kernelWorkspaceBytes = a->kernel_workspace_bytes;

		Transformer_Block_Activations grad_activations;
		memset(&grad_activations, 0, sizeof(grad_activations));
		grad_activations.working_activations = &bwd_activations;
		grad_activations.activation_workspace = &workspace;

		ret = dataflow_submit_transformer_moe_block_bwd_w(handle, compute_stream_id, secondary_compute_stream_id, &grad_stream,
														  &fwd_activations, &grad_activations, &grad_weights);
	}
	free(w_1); free(w_3); free(x_1); free(x_3);
	return ret;
}
