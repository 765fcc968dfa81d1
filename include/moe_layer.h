/*
 * moe_layer.h -- host-side driver of one mixture-of-experts layer on top of a Dataflow_Handle.
 *
 * It submits the same operator sequence as the MoE part of the reference's transformer block:
 *   forward   libdataflowmodels/src/transformer/src/dataflow_transformer.c:2700-2986
 *   bwd_x     dataflow_transformer.c:3386-3719
 *   bwd_w     dataflow_transformer.c:4013-4185
 * with the same buffer roles (libdataflowmodels/include/transformer/seq_batch_structs.h:256-281, 369-395:
 * x_routed, token_expert_weights, chosen_experts, expert_counts, expert_counts_cumsum, expert_mapping,
 * token_mapping, x_1, x_3, x_expert_zones, kernelWorkspace) and the same per-expert weight layout
 * (prep_transformer.c:152-160: w1, w3, w2 of expert e stored back to back, experts at a fixed stride).
 *
 * Three schedules; the first two produce the same results bit for bit:
 *   AMD_MOE_PER_EXPERT  the reference's: sync after routing, read host_expert_counts, then a host loop over
 *                       experts alternating two streams (one matmul / swiglu launch per expert);
 *   AMD_MOE_GROUPED     this backend's: no host round trip; every per-expert loop is one grouped launch
 *                       that reads the device-side prefix sum (independent launches go out in pairs on the two
 *                       streams);
 *   AMD_MOE_FUSED       the grouped schedule with a shorter backward: the reference recomputes the expert outputs
 *                       y = h W2^T to form the router gradient <y_r, dY_t> (dataflow_transformer.c:3494-3535); this
 *                       schedule takes it from the hidden gradient it computes anyway, <y_r, dY_t> = <h_r, dh_r> / w
 *                       (one GEMM, one SwiGLU pass and the read of the expert outputs less per step).  Where w1 and w3
 *                       of an expert lie back to back (H*D*2 bytes a multiple of 256) the two up-projections run as
 *                       one GEMM over the stacked [2H][D] matrix and x1 | x3 are saved side by side per row; backward
 *                       then forms dx1 W1 + dx3 W3 in one GEMM with K = 2H and dW1 | dW3 in one with N = 2H.  The
 *                       forward values, dx1, dx3, dW1, dW3 and dW2 are bit-identical to AMD_MOE_GROUPED; the router
 *                       gradient and dX (one rounding less between the two products) equal within rounding.  Forward
 *                       and backward must both use this schedule or neither.  The stacked up-projection fetches the
 *                       rows of X through expert_mapping itself while X is below 4 GiB (no dispatch copy); with
 *                       AMD_MOE_NO_GATHER set in the environment it takes the copy + packed form that otherwise
 *                       only runs beyond that size.  The stacked dW1 | dW3 GEMM runs on a re-dispatched copy of X (the
 *                       faster form for a reduction over scattered rows); with AMD_MOE_BWD_GATHER set in the
 *                       environment it gathers the rows too.  Test hooks: every form gives the same bits.
 * All functions return 0 on success and -1 on error with a message on stderr.
 */
#ifndef MOE_LAYER_H
#define MOE_LAYER_H

#include "dataflow_amd.h"
#include "dataflow_amd_ops.h"

#ifdef __cplusplus
extern "C" {
#endif

#define AMD_MOE_PER_EXPERT 0
#define AMD_MOE_GROUPED 1
#define AMD_MOE_FUSED 2
/* Added to the schedule of amd_moe_layer_backward (schedule | AMD_MOE_FIRST_MICRO_BATCH): the weight gradients dW1, dW3, dW2
 * and dWr are written instead of accumulated (every weight-gradient GEMM runs with beta = 0 and no C operand; experts without
 * tokens get zeros), so the first micro-batch of an accumulation needs no cleared gradient buffers and reads none.  The
 * reference always accumulates (beta = 1, dataflow_transformer.c:3548-3555, 4101-4148) into buffers its driver clears per
 * step; the result here equals clearing the buffers and accumulating, bit for bit. */
#define AMD_MOE_FIRST_MICRO_BATCH 0x100

typedef struct amd_moe_layer {
	/* shape */
	int max_tokens;                  /* capacity T the buffers were sized for */
	int model_dim;                   /* D */
	int num_experts;                 /* E */
	int top_k;                       /* K */
	int expert_dim;                  /* H */
	DataflowDatatype dt;             /* DATAFLOW_BF16 */

	/* one device slab owns everything below (NULL if the caller bound its own buffers) */
	void * slab;
	uint64_t slab_bytes;

	/* parameters: router [E][D]; expert e has w1 [H][D], w3 [H][D], w2 [D][H] at base + e * expert_stride_bytes */
	void * w_router;
	void * w1;
	void * w3;
	void * w2;
	uint64_t expert_stride_bytes;
	/* gradients, same layout, accumulated into */
	void * dw_router;
	void * dw1;
	void * dw3;
	void * dw2;

	/* saved forward activations */
	void * x_routed;                 /* [T][E] bf16 router logits */
	float * token_expert_weights;    /* [T][K] */
	uint16_t * chosen_experts;       /* [T][K] */
	int * expert_counts;             /* [E+1], last entry is the select_experts launch ticket */
	int * expert_counts_cumsum;      /* [E], inclusive after forward */
	int * expert_mapping;            /* [T*K] routed row -> token */
	int * token_mapping;             /* [T][K] (token, slot) -> routed row */
	void * x1;                       /* [T*K][H]; x3 follows it directly, and the fused schedule uses the pair as one */
	void * x3;                       /* [T*K][H]   [T*K][2H] array with x1 | x3 side by side per row */
	int * host_expert_counts;        /* [E] device-visible host memory */

	/* backward activations */
	void * d_routed;                 /* [T][E] gradient of the router logits */
	void * dx1;                      /* [T*K][H]; dx3 follows it directly (the same two uses as x1 / x3) */
	void * dx3;                      /* [T*K][H] */

	/* workspaces */
	void * expert_zones;             /* [T*K][D] */
	void * kernel_workspace;         /* >= T*K*H elements (+256) : swiglu output / hidden gradient */
	uint64_t kernel_workspace_bytes;

	/* state of the last forward call, checked by backward */
	int last_forward_tokens;         /* its num_tokens: the saved activations are those of that many tokens */
	int saved_side_by_side;          /* non-zero: x1 / x3 were saved as one [T*K][2H] array, x1 | x3 side by side per row (the
	                                  * fused schedule with stacked up-projection weights); backward must read them that way */
	int host_counts_synced;          /* non-zero once the compute stream has been waited for since that forward, i.e.
	                                  * host_expert_counts is complete; the per-expert backward waits if it is not */
} Amd_Moe_Layer;

/* bytes of the slab amd_moe_layer_alloc would allocate */
uint64_t amd_moe_layer_bytes(int max_tokens, int model_dim, int num_experts, int top_k, int expert_dim);

/* allocates one device slab with handle->alloc_mem, carves every buffer at 256-byte alignment, allocates
 * host_expert_counts as device-visible host memory and zeroes the gradient buffers */
int amd_moe_layer_alloc(Dataflow_Handle * handle, Amd_Moe_Layer * layer,
						int max_tokens, int model_dim, int num_experts, int top_k, int expert_dim);
void amd_moe_layer_free(Dataflow_Handle * handle, Amd_Moe_Layer * layer);

/* X [T][D]: the normalised layer input.  out [T][D]: holds the residual on entry, residual + MoE(X) on return.
 * logit_bias: NULL, or a [T][E] bf16 matrix added to the router product as the matmul's beta*C term (a
 * workload-construction hook for skewed routing; the reference's router has no bias).
 * Work is submitted on compute_stream_id; secondary_stream_id carries every other expert in the per-expert
 * schedule and the second of each pair of independent GEMM launches in the grouped one, and is joined back into
 * compute_stream_id before the call returns.  The call itself returns without waiting for the device except for the
 * reference schedule's own sync after routing. */
int amd_moe_layer_forward(Dataflow_Handle * handle, int compute_stream_id, int secondary_stream_id,
						  Amd_Moe_Layer * layer, int num_tokens, void * X, void * logit_bias, void * out, int schedule);

/* dY [T][D]: upstream gradient.  dX [T][D]: receives the gradient w.r.t. X.  Weight gradients are accumulated
 * into dw_*.  Needs the saved activations of the last forward call, which must have had the same num_tokens (-1
 * otherwise).  The per-expert and the grouped schedule may follow each other's forward (the per-expert one waits for the
 * compute stream first if the forward did not, because it reads host_expert_counts); the fused schedule only its own. */
int amd_moe_layer_backward(Dataflow_Handle * handle, int compute_stream_id, int secondary_stream_id,
						   Amd_Moe_Layer * layer, int num_tokens, void * X, void * dY, void * dX, int schedule);

/* ---- the reference's files, as far as this layer meets them ---- */

/* Byte offsets of a transformer block's arrays inside its weight buffer / `combined_layer.weight` file, restating
 * set_transformer_block_weight_offsets (libdataflowmodels/src/transformer/src/prep_transformer.c:24-165) for an
 * exact-attention, RMS-norm, MoE block: attn norm, w_q, w_k, w_v, w_o, ffn norm, router, then for every expert w_1,
 * w_3, w_2; each array starts at the running size rounded up to pointer_alignment.  w_1 / w_3 / w_2 are expert 0's;
 * expert e adds e * expert_stride. */
typedef struct amd_moe_block_offsets {
	uint64_t w_attn_norm, w_q, w_k, w_v, w_o, w_ffn_norm, w_router;
	uint64_t w_1, w_3, w_2;
	uint64_t expert_stride;
	uint64_t raw_size;
	uint64_t aligned_size;
} Amd_Moe_Block_Offsets;

int amd_moe_block_weight_offsets(int model_dim, int attn_dim, int kv_dim, int num_experts, int expert_dim,
								 DataflowDatatype dt, int pointer_alignment, Amd_Moe_Block_Offsets * out);

/* Loads the router and expert weights of one block file (`<model>/layers/<i>/combined_layer.weight`, written by
 * models/init_model.py:205-318; the reference reads it whole, prep_transformer.c:366-388) into an allocated layer.
 * attn_dim / kv_dim size the attention weights that precede the MoE part in the file; pointer_alignment is the one
 * the file's block was laid out with (the reference's drivers use 256).  ffn_norm_weight: NULL, or a device buffer
 * of model_dim elements that receives the norm weight in front of the router.  Synchronous on stream_id. */
int amd_moe_layer_load_block_file(Dataflow_Handle * handle, int stream_id, Amd_Moe_Layer * layer, const char * filename,
								  int attn_dim, int kv_dim, int pointer_alignment, void * ffn_norm_weight);

/* Path of a saved array in the reference's scheme (save_file, dataflow_transformer.c:46-160; its DATA_SAVE_DIR is the
 * save_dir argument here): activations go to <dir>/layers_fwd|layers_bwd/<layer>/seq_<s>_chunk_<c>_<name>.dat,
 * weights (seq_id == -1) to <dir>/model|model_grads/layers/<layer>/<name>.dat; layer -2 / -1 are embedding / head. */
int amd_moe_saved_array_path(char * path, size_t path_bytes, const char * save_dir, int layer_id, int seq_id, int chunk_id,
							 int is_bwd, const char * name);

/* Copies an M x N device array to the host and writes it raw to that path (the directory must exist). */
int amd_moe_save_array(Dataflow_Handle * handle, int stream_id, const char * save_dir, int layer_id, int seq_id, int chunk_id,
					   int is_bwd, const char * name, void * dev_ptr, int M, int N, DataflowDatatype dt);

#ifdef __cplusplus
}
#endif

#endif
