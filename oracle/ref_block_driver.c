/*
 * ref_block_driver.c -- TEST INFRASTRUCTURE, built only where the reference tree is mounted (oracle/Makefile, target
 * `ref`, output oracle/_ref/libref_models.so).  Nothing in the product links or loads it.
 *
 * Compiled against the reference's own headers together with the reference's own dataflow_transformer.c,
 * prep_seq_batch.c and submit wrappers.  It fills the reference's structs (Transformer_Block, Seq_Batch, Seq_Batch_Context,
 * Seq_Batch_Saved_Activations, Seq_Batch_Activation_Workspace, as declared in libdataflowmodels/include/transformer/*.h)
 * from flat arguments and calls, unmodified,
 *     dataflow_submit_transformer_moe_block        (dataflow_transformer.c:2197-2986)   ref_moe_block_forward
 *     dataflow_submit_transformer_moe_block_bwd_x  (dataflow_transformer.c:3326-3968)   ref_moe_block_bwd_x
 * on whatever Dataflow_Handle it is given: the reference's host sync after routing, its host-side expert counts and its
 * per-expert loop over two streams then drive the backend under test.
 *
 * Those two functions also submit four ops of the attention half of the block, which is outside the MoE path: rope,
 * attention forward, attention backward, rope backward.  ref_register_noop_ops registers, through the handle's public
 * register_external_code and with the reference's own skeletons (set_op_skeletons.c), an op that does nothing for each
 * of them: ops of the backend under test, not edits of the reference.  The attention output, dQ and the context
 * gradients are then whatever the caller put into those buffers, which the test does on purpose.
 */
#include <stdlib.h>
#include <string.h>

#include "dataflow_transformer.h"

int ref_noop_op(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra) {
	(void) dataflow_handle; (void) stream_id; (void) op; (void) op_extra;
	return 0;
}

/* this_library: path of the shared object that holds ref_noop_op (this one); block_dt: the element type of the block */
int ref_register_noop_ops(Dataflow_Handle * handle, char * this_library, int block_dt) {
	enum { N = 4 };
	Op_Skeleton skeletons[N];
	dataflow_set_default_rope_skeleton(&skeletons[0], (DataflowDatatype) block_dt);
	dataflow_set_flash_attention_fwd_skeleton(&skeletons[1]);
	dataflow_set_flash_attention_bwd_skeleton(&skeletons[2]);
	dataflow_set_default_rope_bwd_x_skeleton(&skeletons[3], (DataflowDatatype) block_dt);
	char * symbols[N] = {"ref_noop_op", "ref_noop_op", "ref_noop_op", "ref_noop_op"};
	char * init_symbols[N] = {NULL, NULL, NULL, NULL};
	return (handle->register_external_code)(handle, this_library, N, skeletons, symbols, init_symbols);
}

typedef struct ref_block_args {
	/* shape */
	int total_q, model_dim, attn_dim, kv_dim, ffn_dim;
	int num_routed_experts, top_k_experts;
	int num_q_heads, num_kv_heads, head_dim;
	int block_dt, compute_dt;                       /* DataflowDatatype values */
	float eps;
	int * host_expert_counts;                       /* [num_routed_experts], pinned host memory the device can write */
	/* weights (device): expert e's w1 / w3 / w2 at base + e * expert_stride_bytes */
	void * w_attn_norm, * w_q, * w_k, * w_v, * w_o, * w_ffn_norm, * w_router;
	void * w1_base, * w3_base, * w2_base;
	uint64_t expert_stride_bytes;
	/* forward activations (device) */
	void * x_inp;
	float * attn_norm_rms_vals, * ffn_norm_rms_vals;
	void * x_q, * x_k_local, * x_v_local, * x_attn_out;
	float * softmax_lse;
	void * x_o, * x_routed;
	float * token_expert_weights;
	uint16_t * chosen_experts;
	int * expert_counts, * expert_counts_cumsum, * expert_mapping, * token_mapping;
	void * x1_base, * x3_base;
	void * ctx_k, * ctx_v;                          /* the forward context: [total_q][kv_dim] each */
	/* workspace (device) */
	void * x_temp, * x_temp_mlp, * expert_zones, * kernel_workspace;
	uint64_t kernel_workspace_bytes;
	/* block input and output (forward); upstream and downstream gradient (bwd_x) */
	void * X_in, * X_out;
	/* backward working activations (device) */
	void * g_x_routed, * g_x_q, * g_x_k_local, * g_x_v_local, * g_x_o;
	void * g_x1_base, * g_x3_base;
	void * recomputed_ffn_norm, * recomputed_attn_norm;
	void * g_ctx_k, * g_ctx_v;                      /* the gradient context */
	/* weight gradients that bwd_x accumulates (device) */
	void * dw2_base, * dw_ffn_norm, * dw_attn_norm;
} Ref_Block_Args;

typedef struct block_state {
	Transformer_Block block, grad_weights;
	Seq_Batch seq_batch;
	Seq_Batch_Context fwd_context, bwd_context;
	Seq_Batch_Saved_Activations fwd, bwd;
	Seq_Batch_Recomputed_Activations recomputed;
	Seq_Batch_Activation_Workspace workspace;
	void ** ptrs;                                   /* seven arrays of E pointers */
} Block_State;

static int fill(Block_State * s, const Ref_Block_Args * a) {
	const int E = a->num_routed_experts;
	memset(s, 0, sizeof(*s));
	s->ptrs = (void **) calloc((size_t) E * 8, sizeof(void *));
	if (!s->ptrs) {
		return -1;
	}
	void ** w_1 = s->ptrs, ** w_3 = s->ptrs + E, ** w_2 = s->ptrs + 2 * E, ** dw_2 = s->ptrs + 3 * E;
	void ** x_1 = s->ptrs + 4 * E, ** x_3 = s->ptrs + 5 * E, ** g_x_1 = s->ptrs + 6 * E, ** g_x_3 = s->ptrs + 7 * E;
	for (int e = 0; e < E; e++) {
		w_1[e] = (char *) a->w1_base + (uint64_t) e * a->expert_stride_bytes;
		w_3[e] = (char *) a->w3_base + (uint64_t) e * a->expert_stride_bytes;
		w_2[e] = (char *) a->w2_base + (uint64_t) e * a->expert_stride_bytes;
		dw_2[e] = a->dw2_base ? (char *) a->dw2_base + (uint64_t) e * a->expert_stride_bytes : NULL;
	}
	Transformer_Block * blocks[2] = {&s->block, &s->grad_weights};
	for (int b = 0; b < 2; b++) {
		Transformer_Block_Config * c = &blocks[b]->config;
		c->block_dt = (DataflowDatatype) a->block_dt;
		c->compute_dt = (DataflowDatatype) a->compute_dt;
		c->eps = a->eps;
		c->theta = 10000;
		c->model_dim = a->model_dim;
		c->num_q_heads = a->num_q_heads;
		c->num_kv_heads = a->num_kv_heads;
		c->head_dim = a->head_dim;
		c->attn_dim = a->attn_dim;
		c->kv_dim = a->kv_dim;
		c->ffn_dim = a->ffn_dim;
		c->moe_config.top_k_experts = a->top_k_experts;
		c->moe_config.num_shared_experts = 0;
		c->moe_config.num_global_routed_experts = E;
		c->moe_config.num_local_experts = E;
		blocks[b]->layer_id = 0;
	}
	s->block.w_attn_norm = a->w_attn_norm;
	s->block.w_q = a->w_q;
	s->block.w_k = a->w_k;
	s->block.w_v = a->w_v;
	s->block.w_o = a->w_o;
	s->block.w_ffn_norm = a->w_ffn_norm;
	s->block.w_router = a->w_router;
	s->block.w_1 = w_1;
	s->block.w_3 = w_3;
	s->block.w_2 = w_2;
	s->grad_weights.w_2 = dw_2;
	s->grad_weights.w_ffn_norm = a->dw_ffn_norm;
	s->grad_weights.w_attn_norm = a->dw_attn_norm;

	s->fwd_context.total_context_tokens = a->total_q;
	s->fwd_context.x_k = a->ctx_k;
	s->fwd_context.x_v = a->ctx_v;
	s->bwd_context.total_context_tokens = a->total_q;
	s->bwd_context.x_k = a->g_ctx_k;
	s->bwd_context.x_v = a->g_ctx_v;

	s->seq_batch.attention_config.num_seqs = 1;
	s->seq_batch.attention_config.total_q = a->total_q;
	s->seq_batch.attention_config.total_k = a->total_q;
	s->seq_batch.attention_config.max_seqlen_q = a->total_q;
	s->seq_batch.attention_config.max_seqlen_k = a->total_q;
	s->seq_batch.moe_config.host_expert_counts = a->host_expert_counts;    /* layer 0: offset 0 */

	s->fwd.seq_batch = &s->seq_batch;
	s->fwd.x_inp = a->x_inp;
	s->fwd.attn_norm_rms_vals = a->attn_norm_rms_vals;
	s->fwd.ffn_norm_rms_vals = a->ffn_norm_rms_vals;
	s->fwd.x_q = a->x_q;
	s->fwd.x_k_local = a->x_k_local;
	s->fwd.x_v_local = a->x_v_local;
	s->fwd.x_attn_out = a->x_attn_out;
	s->fwd.softmax_lse = a->softmax_lse;
	s->fwd.x_o = a->x_o;
	s->fwd.x_routed = a->x_routed;
	s->fwd.token_expert_weights = a->token_expert_weights;
	s->fwd.chosen_experts = a->chosen_experts;
	s->fwd.expert_counts = a->expert_counts;
	s->fwd.expert_counts_cumsum = a->expert_counts_cumsum;
	s->fwd.expert_mapping = a->expert_mapping;
	s->fwd.token_mapping = a->token_mapping;
	s->fwd.x_1 = x_1;
	s->fwd.x_3 = x_3;
	x_1[0] = a->x1_base;                             /* the reference's set_moe_working_activations_offsets carves the rest */
	x_3[0] = a->x3_base;

	s->recomputed.recomputed_ffn_norm = a->recomputed_ffn_norm;
	s->recomputed.recomputed_attn_norm = a->recomputed_attn_norm;
	s->bwd.seq_batch = &s->seq_batch;
	s->bwd.recomputed_activations = &s->recomputed;
	s->bwd.x_routed = a->g_x_routed;
	s->bwd.x_q = a->g_x_q;
	s->bwd.x_k_local = a->g_x_k_local;
	s->bwd.x_v_local = a->g_x_v_local;
	s->bwd.x_o = a->g_x_o;
	s->bwd.x_1 = g_x_1;
	s->bwd.x_3 = g_x_3;
	g_x_1[0] = a->g_x1_base;
	g_x_3[0] = a->g_x3_base;

	s->workspace.x_temp = a->x_temp;
	s->workspace.x_temp_mlp = a->x_temp_mlp;
	s->workspace.x_expert_zones = a->expert_zones;
	s->workspace.kernelWorkspace = a->kernel_workspace;
	s->workspace.kernelWorkspaceBytes = a->kernel_workspace_bytes;
	return 0;
}

int ref_moe_block_forward(Dataflow_Handle * handle, int compute_stream_id, int secondary_compute_stream_id, const Ref_Block_Args * a) {
	Block_State s;
	if (fill(&s, a)) {
		return -1;
	}
	s.seq_batch.context = &s.fwd_context;
	Transformer_Block_Transition in, out;
	memset(&in, 0, sizeof(in));
	memset(&out, 0, sizeof(out));
	in.seq_batch = &s.seq_batch;
	in.X = a->X_in;
	out.seq_batch = &s.seq_batch;
	out.X = a->X_out;
	Transformer_Block_Activations activations;
	memset(&activations, 0, sizeof(activations));
	activations.working_activations = &s.fwd;
	activations.activation_workspace = &s.workspace;
	int ret = dataflow_submit_transformer_moe_block(handle, compute_stream_id, secondary_compute_stream_id, &in, &s.block, &activations, &out);
	free(s.ptrs);
	return ret;
}

int ref_moe_block_bwd_x(Dataflow_Handle * handle, int compute_stream_id, int secondary_compute_stream_id, const Ref_Block_Args * a) {
	Block_State s;
	if (fill(&s, a)) {
		return -1;
	}
	s.seq_batch.context = &s.bwd_context;            /* bwd_x accumulates the context gradients through the batch's context */
	Transformer_Block_Transition in, out;
	memset(&in, 0, sizeof(in));
	memset(&out, 0, sizeof(out));
	in.seq_batch = &s.seq_batch;
	in.X = a->X_in;
	out.seq_batch = &s.seq_batch;
	out.X = a->X_out;
	Transformer_Block_Activations grad_activations;
	memset(&grad_activations, 0, sizeof(grad_activations));
	grad_activations.working_activations = &s.bwd;
	grad_activations.activation_workspace = &s.workspace;
	int ret = dataflow_submit_transformer_moe_block_bwd_x(handle, compute_stream_id, secondary_compute_stream_id, &s.block, &in, &s.fwd, &s.fwd_context,
														  &grad_activations, &s.grad_weights, &out);
	free(s.ptrs);
	return ret;
}
