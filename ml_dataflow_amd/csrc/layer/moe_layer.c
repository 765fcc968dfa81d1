/*
 * moe_layer.c -- submits the MoE layer's operator sequence to a Dataflow_Handle (see include/moe_layer.h).
 *
 * The per-expert schedule restates, op for op, the MoE part of
 * libdataflowmodels/src/transformer/src/dataflow_transformer.c (forward :2700-2986, bwd_x :3386-3719,
 * bwd_w :4013-4185) including its stream fork/join and workspace halving; the grouped schedule replaces
 * each host loop over experts by one grouped launch and never waits for the device; the fused schedule is the
 * grouped one without the backward recompute of the expert outputs.
 */
#include "moe_layer.h"

#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define ALIGN256(x) (((uint64_t) (x) + 255UL) & ~255UL)
#define CHECK(call, msg) do { if ((call)) { fprintf(stderr, "Error: %s...\n", msg); return -1; } } while (0)

typedef struct slab_cursor {
	uint8_t * base;
	uint64_t off;
} Slab_Cursor;

static void * carve(Slab_Cursor * c, uint64_t bytes) {
	c->off = ALIGN256(c->off);
	void * p = c->base ? (void *) (c->base + c->off) : NULL;
	c->off += bytes;
	return p;
}

/* lays the buffers out in one slab; with base == NULL only measures */
static uint64_t layout(Amd_Moe_Layer * L, uint8_t * base, int T, int D, int E, int K, int H) {
	Slab_Cursor c = {base, 0};
	uint64_t el = 2;
	uint64_t R = (uint64_t) T * (uint64_t) K;
	uint64_t w_up = ALIGN256((uint64_t) H * D * el);
	uint64_t w_down = ALIGN256((uint64_t) D * H * el);
	uint64_t stride = 2 * w_up + w_down;

	void * w_router = carve(&c, (uint64_t) E * D * el);
	void * experts = carve(&c, stride * (uint64_t) E);
	void * dw_router = carve(&c, (uint64_t) E * D * el);
	void * dexperts = carve(&c, stride * (uint64_t) E);
	void * x_routed = carve(&c, (uint64_t) T * E * el);
	void * weights = carve(&c, R * sizeof(float));
	void * chosen = carve(&c, R * sizeof(uint16_t));
	void * counts = carve(&c, (uint64_t) (E + 1) * sizeof(int));
	void * cumsum = carve(&c, (uint64_t) E * sizeof(int));
	void * expert_mapping = carve(&c, R * sizeof(int));
	void * token_mapping = carve(&c, R * sizeof(int));
	/* x1 and x3 (and their gradients) back to back: two [R][H] arrays for the reference's op sequence, or one [R][2H]
	 * array whose rows hold x1 | x3 side by side for the fused schedule */
	void * x1 = carve(&c, 2 * R * H * el);
	void * x3 = x1 ? (void *) ((uint8_t *) x1 + R * H * el) : NULL;
	void * d_routed = carve(&c, (uint64_t) T * E * el);
	void * dx1 = carve(&c, 2 * R * H * el);
	void * dx3 = dx1 ? (void *) ((uint8_t *) dx1 + R * H * el) : NULL;
	void * zones = carve(&c, R * D * el);
	/* two halves, one per stream in the per-expert schedule; each can hold an expert with up to T*K rows */
	uint64_t ws_bytes = 2 * ALIGN256(R * H * el) + 512;
	void * ws = carve(&c, ws_bytes);
	uint64_t total = ALIGN256(c.off);

	if (L) {
		L->w_router = w_router;
		L->w1 = experts;
		L->w3 = experts ? (uint8_t *) experts + w_up : NULL;
		L->w2 = experts ? (uint8_t *) experts + 2 * w_up : NULL;
		L->expert_stride_bytes = stride;
		L->dw_router = dw_router;
		L->dw1 = dexperts;
		L->dw3 = dexperts ? (uint8_t *) dexperts + w_up : NULL;
		L->dw2 = dexperts ? (uint8_t *) dexperts + 2 * w_up : NULL;
		L->x_routed = x_routed;
		L->token_expert_weights = (float *) weights;
		L->chosen_experts = (uint16_t *) chosen;
		L->expert_counts = (int *) counts;
		L->expert_counts_cumsum = (int *) cumsum;
		L->expert_mapping = (int *) expert_mapping;
		L->token_mapping = (int *) token_mapping;
		L->x1 = x1;
		L->x3 = x3;
		L->d_routed = d_routed;
		L->dx1 = dx1;
		L->dx3 = dx3;
		L->expert_zones = zones;
		L->kernel_workspace = ws;
		L->kernel_workspace_bytes = ws_bytes;
	}
	return total;
}

uint64_t amd_moe_layer_bytes(int max_tokens, int model_dim, int num_experts, int top_k, int expert_dim) {
	return layout(NULL, NULL, max_tokens, model_dim, num_experts, top_k, expert_dim);
}

int amd_moe_layer_alloc(Dataflow_Handle * handle, Amd_Moe_Layer * layer,
						int max_tokens, int model_dim, int num_experts, int top_k, int expert_dim) {
	if (!handle || !layer) {
		fprintf(stderr, "Error: amd_moe_layer_alloc needs a handle and a layer...\n");
		return -1;
	}
	if (max_tokens < 1 || num_experts < 1 || top_k < 1 || top_k > num_experts || (model_dim & 7) || (expert_dim & 7) || model_dim < 8 || expert_dim < 8) {
		fprintf(stderr, "Error: bad MoE layer shape T=%d D=%d E=%d K=%d H=%d (D and H must be multiples of 8, 1 <= K <= E)...\n",
				max_tokens, model_dim, num_experts, top_k, expert_dim);
		return -1;
	}
	memset(layer, 0, sizeof(*layer));
	layer->max_tokens = max_tokens;
	layer->model_dim = model_dim;
	layer->num_experts = num_experts;
	layer->top_k = top_k;
	layer->expert_dim = expert_dim;
	layer->dt = DATAFLOW_BF16;
	uint64_t bytes = layout(NULL, NULL, max_tokens, model_dim, num_experts, top_k, expert_dim);
	void * slab = (handle->alloc_mem)(handle, bytes);
	if (!slab) {
		fprintf(stderr, "Error: could not allocate %lu bytes for the MoE layer...\n", (unsigned long) bytes);
		return -1;
	}
	layer->slab = slab;
	layer->slab_bytes = bytes;
	layout(layer, (uint8_t *) slab, max_tokens, model_dim, num_experts, top_k, expert_dim);
	layer->host_expert_counts = (int *) dataflow_amd_alloc_host_mem(handle, (uint64_t) num_experts * sizeof(int));
	if (!layer->host_expert_counts) {
		(handle->free_mem)(handle, slab);
		memset(layer, 0, sizeof(*layer));
		return -1;
	}
	memset(layer->host_expert_counts, 0, (size_t) num_experts * sizeof(int));
	/* gradients accumulate, so they start at zero */
	CHECK((handle->set_mem)(handle, -1, layer->dw_router, 0, (uint64_t) num_experts * model_dim * 2), "failed to clear router gradient");
	CHECK((handle->set_mem)(handle, -1, layer->dw1, 0, layer->expert_stride_bytes * (uint64_t) num_experts), "failed to clear expert gradients");
	return 0;
}

void amd_moe_layer_free(Dataflow_Handle * handle, Amd_Moe_Layer * layer) {
	if (!handle || !layer) {
		return;
	}
	if (layer->host_expert_counts) {
		dataflow_amd_free_host_mem(handle, layer->host_expert_counts);
	}
	if (layer->slab) {
		(handle->free_mem)(handle, layer->slab);
	}
	memset(layer, 0, sizeof(*layer));
}

static int check_call(const Amd_Moe_Layer * L, int T, int schedule) {
	if (!L || T < 0 || T > L->max_tokens) {
		fprintf(stderr, "Error: MoE layer call with %d tokens, capacity %d...\n", T, L ? L->max_tokens : 0);
		return -1;
	}
	if (schedule != AMD_MOE_PER_EXPERT && schedule != AMD_MOE_GROUPED && schedule != AMD_MOE_FUSED) {
		fprintf(stderr, "Error: unknown MoE schedule %d...\n", schedule);
		return -1;
	}
	return 0;
}

/* w1 and w3 of an expert (and dw1 / dw3) lie back to back with no padding between them: together a [2H][D] matrix */
static int up_weights_stacked(const Amd_Moe_Layer * L) {
	return (uint8_t *) L->w3 == (uint8_t *) L->w1 + (uint64_t) L->expert_dim * L->model_dim * 2
		&& (uint8_t *) L->dw3 == (uint8_t *) L->dw1 + (uint64_t) L->expert_dim * L->model_dim * 2;
}

/* May the GEMM loaders fetch the rows of X through expert_mapping themselves (no dispatch copy)?  Their offsets are 32 bits,
 * so X has to stay below 4 GiB.  AMD_MOE_NO_GATHER in the environment (any value) forces the copy + packed form, which
 * otherwise only runs beyond that size: the tests compare the two forms bit for bit that way. */
static int gather_allowed(int T, int D) {
	return (uint64_t) T * (uint64_t) D * 2u <= 0xFFFFFFFFull && getenv("AMD_MOE_NO_GATHER") == NULL;
}

static void * expert_ptr(void * base, uint64_t stride, int e) {
	return (void *) ((uint8_t *) base + stride * (uint64_t) e);
}

/* the two streams meet: `waiter` will not run past this point before `signaller` reaches it
 * (dataflow_transformer.c:2814-2826) */
static int stream_wait(Dataflow_Handle * h, int waiter, int signaller) {
	void * state = (h->get_stream_state)(h, signaller);
	if (!state) {
		fprintf(stderr, "Error: failed to get stream state for stream #%d...\n", signaller);
		return -1;
	}
	if ((h->submit_dependency)(h, waiter, state)) {
		fprintf(stderr, "Error: failed to submit dependency for stream #%d to wait for stream #%d...\n", waiter, signaller);
		return -1;
	}
	return 0;
}

/* ------------------------------------------------------------------ forward */

int amd_moe_layer_forward(Dataflow_Handle * h, int cs, int ss, Amd_Moe_Layer * L, int T, void * X, void * logit_bias, void * out, int schedule) {
	if (check_call(L, T, schedule)) {
		return -1;
	}
	if (T == 0) {
		return 0;
	}
	const DataflowDatatype dt = L->dt;
	const DataflowDatatype cdt = DATAFLOW_FP32;
	const int D = L->model_dim, E = L->num_experts, K = L->top_k, H = L->expert_dim;
	const uint64_t el = 2;

	/* 1. router logits (bf16 out), dataflow_transformer.c:2710-2717 */
	CHECK(dataflow_submit_matmul(h, cs, dt, dt, logit_bias ? dt : DATAFLOW_NONE, dt, cdt, 1, 0, E, D, T,
								 1.0f, logit_bias ? 1.0f : 0.0f, L->w_router, X, logit_bias, L->x_routed,
								 L->kernel_workspace_bytes, L->kernel_workspace), "failed to submit router matmul");

	/* 2. select experts, :2737-2757 */
	/* counts and their prefix sum start at zero (dataflow_transformer.c:2737-2747); one fill where the two arrays follow
	 * each other in memory, as they do in a layer that amd_moe_layer_alloc carved (256-byte aligned, counts first) */
	const uint64_t counts_bytes = (uint64_t) (E + 1) * sizeof(int), cumsum_bytes = (uint64_t) E * sizeof(int);
	const uint64_t apart = (uint64_t) ((uint8_t *) L->expert_counts_cumsum - (uint8_t *) L->expert_counts);
	if ((uint8_t *) L->expert_counts_cumsum > (uint8_t *) L->expert_counts && apart < counts_bytes + 256) {
		CHECK((h->set_mem)(h, cs, L->expert_counts, 0, apart + cumsum_bytes), "failed to set expert counts and their prefix sum to 0");
	} else {
		CHECK((h->set_mem)(h, cs, L->expert_counts, 0, counts_bytes), "failed to set expert counts to 0");
		CHECK((h->set_mem)(h, cs, L->expert_counts_cumsum, 0, cumsum_bytes), "failed to set expert counts cumsum to 0");
	}
	CHECK(dataflow_submit_default_select_experts(h, cs, dt, T, E, K, L->x_routed, L->token_expert_weights, L->chosen_experts,
												 L->expert_counts, L->expert_counts_cumsum, L->host_expert_counts), "failed to submit select experts");
	/* 3. mapping, :2781-2784 */
	CHECK(dataflow_submit_default_build_expert_mapping(h, cs, T, E, K, L->chosen_experts, L->expert_counts_cumsum,
													   L->expert_mapping, L->token_mapping), "failed to submit build expert mapping");

	L->last_forward_tokens = T;
	L->host_counts_synced = 0;
	L->saved_side_by_side = 0;
	if (schedule == AMD_MOE_FUSED && up_weights_stacked(L)) {
		/* One GEMM over the stacked [2H][D] up-projection weights: row r of the result holds x1[r,:] | x3[r,:] side by
		 * side.  Twice the tiles per launch (the last, partial round of tiles over the compute units weighs half as
		 * much) and the token rows are fetched once for both products. */
		L->saved_side_by_side = 1;
		void * x13 = L->x1;
		if (gather_allowed(T, D)) {
			/* no dispatch copy: the GEMM's loaders fetch row expert_mapping[r] of X for routed row r themselves (the
			 * same values reach the same multiplies, so the result is that of the copy + GEMM below, bit for bit) */
			CHECK(dataflow_submit_amd_grouped_matmul_gathered(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, AMD_GROUPED_RAGGED_N, 2 * H, D, T * K,
															  E, L->expert_counts_cumsum, 1.0f, 0.0f, L->w1, L->expert_stride_bytes, X, NULL, x13, 0,
															  L->expert_mapping, T),
				  "failed to submit gathered grouped w1|w3 matmul");
		} else {
			CHECK(dataflow_submit_default_prepare_experts(h, cs, dt, dt, T, D, K, X, L->token_mapping, L->expert_zones), "failed to submit prepare experts");
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, AMD_GROUPED_RAGGED_N, 2 * H, D, T * K,
													 E, L->expert_counts_cumsum, 1.0f, 0.0f, L->w1, L->expert_stride_bytes, L->expert_zones, NULL, x13, 0),
				  "failed to submit grouped w1|w3 matmul");
		}
		CHECK(dataflow_submit_amd_swiglu_strided(h, cs, dt, T * K, H, 2 * H, x13, (uint8_t *) x13 + (uint64_t) H * el, L->kernel_workspace),
			  "failed to submit strided swiglu");
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, AMD_GROUPED_RAGGED_N, D, H, T * K,
												 E, L->expert_counts_cumsum, 1.0f, 0.0f, L->w2, L->expert_stride_bytes, L->kernel_workspace, NULL, L->expert_zones, 0),
			  "failed to submit grouped w2 matmul");
		CHECK(dataflow_submit_default_merge_experts(h, cs, dt, dt, T, D, K, L->expert_zones, L->token_mapping, L->token_expert_weights, out),
			  "failed to submit merge experts");
		return 0;
	}
	if (schedule != AMD_MOE_PER_EXPERT) {
		CHECK(dataflow_submit_default_prepare_experts(h, cs, dt, dt, T, D, K, X, L->token_mapping, L->expert_zones), "failed to submit prepare experts");
		/* The two up-projections are independent: the second goes to the secondary stream, so its work-groups move
		 * into the compute units that the first one's last, partial round of tiles leaves idle. */
		CHECK(stream_wait(h, ss, cs), "secondary stream could not wait for the compute stream");
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, AMD_GROUPED_RAGGED_N, H, D, T * K,
												 E, L->expert_counts_cumsum, 1.0f, 0.0f, L->w1, L->expert_stride_bytes, L->expert_zones, NULL, L->x1, 0),
			  "failed to submit grouped w1 matmul");
		CHECK(dataflow_submit_amd_grouped_matmul(h, ss, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, AMD_GROUPED_RAGGED_N, H, D, T * K,
												 E, L->expert_counts_cumsum, 1.0f, 0.0f, L->w3, L->expert_stride_bytes, L->expert_zones, NULL, L->x3, 0),
			  "failed to submit grouped w3 matmul");
		CHECK(stream_wait(h, cs, ss), "compute stream could not wait for the secondary stream");
		CHECK(dataflow_submit_default_swiglu(h, cs, dt, T * K, H, L->x1, L->x3, L->kernel_workspace), "failed to submit swiglu");
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, AMD_GROUPED_RAGGED_N, D, H, T * K,
												 E, L->expert_counts_cumsum, 1.0f, 0.0f, L->w2, L->expert_stride_bytes, L->kernel_workspace, NULL, L->expert_zones, 0),
			  "failed to submit grouped w2 matmul");
		CHECK(dataflow_submit_default_merge_experts(h, cs, dt, dt, T, D, K, L->expert_zones, L->token_mapping, L->token_expert_weights, out),
			  "failed to submit merge experts");
		return 0;
	}

	/* reference schedule: the host needs the counts, :2789-2800 */
	CHECK((h->sync_stream)(h, cs), "failed to sync with compute stream after building expert mapping");
	L->host_counts_synced = 1;
	long routed = 0;
	for (int e = 0; e < E; e++) {
		routed += L->host_expert_counts[e];
	}
	if (routed != (long) T * K) {
		fprintf(stderr, "Error: total routed tokens does not match expected number of tokens. Chunk size: %d, top_k_active: %d => expected %ld, got %ld\n",
				T, K, (long) T * K, routed);
		return -1;
	}
	CHECK(dataflow_submit_default_prepare_experts(h, cs, dt, dt, T, D, K, X, L->token_mapping, L->expert_zones), "failed to submit prepare experts");
	CHECK(stream_wait(h, ss, cs), "secondary stream could not wait for the compute stream");

	uint64_t half = L->kernel_workspace_bytes / 2;                          /* :2840-2842 */
	uint8_t * ws[2] = {(uint8_t *) L->kernel_workspace, (uint8_t *) L->kernel_workspace + half};
	int streams[2] = {cs, ss};
	int which = 0;
	uint64_t row = 0;
	for (int e = 0; e < E; e++) {                                           /* :2848-2940 */
		int n = L->host_expert_counts[e];
		if (n == 0) {
			continue;
		}
		uint8_t * zone = (uint8_t *) L->expert_zones + row * D * el;
		uint8_t * x1 = (uint8_t *) L->x1 + row * H * el;
		uint8_t * x3 = (uint8_t *) L->x3 + row * H * el;
		uint64_t temp_bytes = (uint64_t) n * H * el;
		if (temp_bytes > half) {                                            /* :2889-2892 */
			fprintf(stderr, "Error: expert #%d has too many tokens for current kernel workspace. (# tokens: %d, streamKernelWorkspaceBytes: %lu)\n", e, n, (unsigned long) half);
			return -1;
		}
		uint8_t * temp = ws[which];
		/* the expert GEMMs get no workspace (the reference hands cuBLASLt the rest of this half, :2894-2897): with one,
		 * a small expert would be split along K and round differently from the same expert inside the grouped launch */
		int s = streams[which];
		CHECK(dataflow_submit_matmul(h, s, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, H, D, n, 1.0f, 0.0f,
									 expert_ptr(L->w1, L->expert_stride_bytes, e), zone, NULL, x1, 0, NULL), "failed to submit w1 matmul");
		CHECK(dataflow_submit_matmul(h, s, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, H, D, n, 1.0f, 0.0f,
									 expert_ptr(L->w3, L->expert_stride_bytes, e), zone, NULL, x3, 0, NULL), "failed to submit w3 matmul");
		CHECK(dataflow_submit_default_swiglu(h, s, dt, n, H, x1, x3, temp), "failed to submit swiglu");
		CHECK(dataflow_submit_matmul(h, s, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, D, H, n, 1.0f, 0.0f,
									 expert_ptr(L->w2, L->expert_stride_bytes, e), temp, NULL, zone, 0, NULL), "failed to submit w2 matmul");
		row += (uint64_t) n;
		which ^= 1;
	}
	CHECK(stream_wait(h, cs, ss), "compute stream could not wait for the secondary stream");   /* :2951-2961 */
	CHECK(dataflow_submit_default_merge_experts(h, cs, dt, dt, T, D, K, L->expert_zones, L->token_mapping, L->token_expert_weights, out),
		  "failed to submit merge experts");                                                 /* :2964-2970 */
	return 0;
}

/* ------------------------------------------------------------------ backward */

int amd_moe_layer_backward(Dataflow_Handle * h, int cs, int ss, Amd_Moe_Layer * L, int T, void * X, void * dY, void * dX, int schedule) {
	/* first micro-batch of an accumulation: the weight gradients are written (beta = 0, no C operand), not added to */
	const int first_micro_batch = (schedule & AMD_MOE_FIRST_MICRO_BATCH) != 0;
	schedule &= ~AMD_MOE_FIRST_MICRO_BATCH;
	if (check_call(L, T, schedule)) {
		return -1;
	}
	if (T == 0) {
		return 0;
	}
	const DataflowDatatype dt = L->dt;
	const DataflowDatatype cdt = DATAFLOW_FP32;
	const int D = L->model_dim, E = L->num_experts, K = L->top_k, H = L->expert_dim;
	const uint64_t el = 2;
	const float wbeta = first_micro_batch ? 0.0f : 1.0f;                 /* of every weight-gradient GEMM */
	const DataflowDatatype wc_dt = first_micro_batch ? DATAFLOW_NONE : dt;
#define WGRAD_C(ptr) (first_micro_batch ? NULL : (ptr))
	const uint64_t S = L->expert_stride_bytes;

	if (T != L->last_forward_tokens) {
		fprintf(stderr, "Error: MoE backward over %d tokens, but the saved activations are those of a forward over %d...\n", T, L->last_forward_tokens);
		return -1;
	}
	const int side_by_side = schedule == AMD_MOE_FUSED && up_weights_stacked(L);
	if (side_by_side != L->saved_side_by_side) {
		fprintf(stderr, "Error: MoE backward schedule %d cannot read the activations the last forward saved (%s): run both passes with the fused schedule or neither...\n",
				schedule, L->saved_side_by_side ? "x1 | x3 side by side per row" : "x1 and x3 as separate arrays");
		return -1;
	}
	if (schedule == AMD_MOE_PER_EXPERT && !L->host_counts_synced) {
		/* the forward ran a schedule that never waits for the device: host_expert_counts is written by select_experts
		 * on the compute stream and is only known to be complete once that stream has been waited for */
		CHECK((h->sync_stream)(h, cs), "failed to sync with compute stream before reading the expert counts");
		L->host_counts_synced = 1;
	}

	/* router-logit gradients start at zero, dataflow_transformer.c:3399 */
	CHECK((h->set_mem)(h, cs, L->d_routed, 0, (uint64_t) T * E * el), "failed to set router derivs to 0");

	if (schedule == AMD_MOE_FUSED) {
		void * temp = L->kernel_workspace;
		int * cum = L->expert_counts_cumsum;
		/* No recompute of the expert outputs: <y_r, dY_t> = <h_r, dh_r> / w with dh_r = (w dY_t) W2 the hidden gradient.
		 * w-scaled dY rows straight from dY -> dh -> (router gradient, dx1, dx3, h) in one pass -> dW2. */
		CHECK(dataflow_submit_amd_prepare_experts_scaled(h, cs, dt, dt, T, D, K, dY, L->token_mapping, L->token_expert_weights, L->expert_zones),
			  "failed to submit scaled prepare experts (dY)");
		if (side_by_side) {
			/* x1 | x3 and dx1 | dx3 side by side per row: one GEMM with K = 2H gives dx1 W1 + dx3 W3 (no rounding of the
			 * first product in between, no read of it back), one with N = 2H gives dW1 and dW3 */
			void * dh = (uint8_t *) L->kernel_workspace + L->kernel_workspace_bytes / 2;
			void * x13 = L->x1, * dx13 = L->dx1;
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, H, D, T * K, E, cum,
													 1.0f, 0.0f, L->w2, S, L->expert_zones, NULL, dh, 0), "failed to submit grouped dh matmul");
			CHECK(dataflow_submit_amd_swiglu_bwd_x_routed(h, cs, dt, dt, T * K, H, E, K, 2 * H, 2 * H, L->expert_mapping, L->token_mapping,
														  L->chosen_experts, L->token_expert_weights, x13, (uint8_t *) x13 + (uint64_t) H * el, dh,
														  L->d_routed, dx13, (uint8_t *) dx13 + (uint64_t) H * el, temp),
				  "failed to submit routed swiglu bwd x");
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, wc_dt, dt, cdt, 0, 1, AMD_GROUPED_RAGGED_K, H, 0, D, E, cum,
													 1.0f, wbeta, temp, 0, L->expert_zones, WGRAD_C(L->dw2), L->dw2, S), "failed to submit grouped dW2 matmul");
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, D, 2 * H, T * K, E, cum,
													 1.0f, 0.0f, L->w1, S, dx13, NULL, L->expert_zones, 0), "failed to submit grouped dX matmul");
		} else {
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, H, D, T * K, E, cum,
													 1.0f, 0.0f, L->w2, S, L->expert_zones, NULL, L->dx1, 0), "failed to submit grouped dh matmul");
			CHECK(dataflow_submit_amd_swiglu_bwd_x_routed(h, cs, dt, dt, T * K, H, E, K, H, H, L->expert_mapping, L->token_mapping, L->chosen_experts,
														  L->token_expert_weights, L->x1, L->x3, L->dx1, L->d_routed, L->dx1, L->dx3, temp),
				  "failed to submit routed swiglu bwd x");
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, wc_dt, dt, cdt, 0, 1, AMD_GROUPED_RAGGED_K, H, 0, D, E, cum,
													 1.0f, wbeta, temp, 0, L->expert_zones, WGRAD_C(L->dw2), L->dw2, S), "failed to submit grouped dW2 matmul");
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, D, H, T * K, E, cum,
													 1.0f, 0.0f, L->w1, S, L->dx1, NULL, L->expert_zones, 0), "failed to submit grouped dX(w1) matmul");
			CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, dt, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, D, H, T * K, E, cum,
													 1.0f, 1.0f, L->w3, S, L->dx3, L->expert_zones, L->expert_zones, 0), "failed to submit grouped dX(w3) matmul");
		}
	} else if (schedule == AMD_MOE_GROUPED) {
		void * temp = L->kernel_workspace;
		int * cum = L->expert_counts_cumsum;
		/* recompute the expert outputs (:3494-3511) for all experts at once */
		CHECK(dataflow_submit_default_swiglu(h, cs, dt, T * K, H, L->x1, L->x3, temp), "failed to submit swiglu recompute");
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, AMD_GROUPED_RAGGED_N, D, H, T * K, E, cum,
												 1.0f, 0.0f, L->w2, S, temp, NULL, L->expert_zones, 0), "failed to submit grouped w2 recompute");
		/* router gradient + scaled upstream rows (:3525-3535) */
		CHECK(dataflow_submit_amd_router_bwd_x_all(h, cs, dt, dt, T, D, E, K, L->token_mapping, L->chosen_experts, L->token_expert_weights,
												   L->expert_zones, dY, L->d_routed, L->expert_zones), "failed to submit router bwd x");
		/* dW2 += g^T h (:3548-3555) and dh = g W2 (:3568-3575).  The reference writes dh over h, which orders the two;
		 * here dh goes to the dx1 buffer (swiglu_bwd_x then works in place: it reads an element of dh before it writes
		 * that element of dx1), so the two GEMMs are independent and the second runs on the secondary stream, filling
		 * the compute units that the first one's last round of tiles leaves idle. */
		CHECK(stream_wait(h, ss, cs), "secondary stream could not wait for the compute stream");
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, wc_dt, dt, cdt, 0, 1, AMD_GROUPED_RAGGED_K, H, 0, D, E, cum,
												 1.0f, wbeta, temp, 0, L->expert_zones, WGRAD_C(L->dw2), L->dw2, S), "failed to submit grouped dW2 matmul");
		CHECK(dataflow_submit_amd_grouped_matmul(h, ss, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, H, D, T * K, E, cum,
												 1.0f, 0.0f, L->w2, S, L->expert_zones, NULL, L->dx1, 0), "failed to submit grouped dh matmul");
		CHECK(stream_wait(h, cs, ss), "compute stream could not wait for the secondary stream");
		CHECK(dataflow_submit_default_swiglu_bwd_x(h, cs, dt, dt, T * K, H, L->x1, L->x3, L->dx1, L->dx1, L->dx3), "failed to submit swiglu bwd x");
		/* zone = dx1 W1, zone += dx3 W3 (:3601-3621) */
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, D, H, T * K, E, cum,
												 1.0f, 0.0f, L->w1, S, L->dx1, NULL, L->expert_zones, 0), "failed to submit grouped dX(w1) matmul");
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, dt, dt, cdt, 0, 0, AMD_GROUPED_RAGGED_N, D, H, T * K, E, cum,
												 1.0f, 1.0f, L->w3, S, L->dx3, L->expert_zones, L->expert_zones, 0), "failed to submit grouped dX(w3) matmul");
	} else {
		long routed = 0;
		for (int e = 0; e < E; e++) {
			routed += L->host_expert_counts[e];
		}
		if (routed != (long) T * K) {                                        /* :3407-3411 */
			fprintf(stderr, "Error: seen tokens (%ld) != total q (%d) * top k (%d) in bwd_x...\n", routed, T, K);
			return -1;
		}
		CHECK(stream_wait(h, ss, cs), "secondary stream could not wait for the compute stream");
		uint64_t half = L->kernel_workspace_bytes / 2;
		uint8_t * ws[2] = {(uint8_t *) L->kernel_workspace, (uint8_t *) L->kernel_workspace + half};
		int streams[2] = {cs, ss};
		int which = 0;
		uint64_t row = 0;
		for (int e = 0; e < E; e++) {                                        /* :3460-3641 */
			int n = L->host_expert_counts[e];
			if (n == 0) {
				if (first_micro_batch) {                                         /* no launch writes this expert's gradients */
					void * unwritten[3] = {expert_ptr(L->dw1, S, e), expert_ptr(L->dw3, S, e), expert_ptr(L->dw2, S, e)};
					for (int g = 0; g < 3; g++) {
						CHECK((h->set_mem)(h, cs, unwritten[g], 0, (uint64_t) H * D * el), "failed to clear the gradients of an expert without tokens");
					}
				}
				continue;
			}
			uint8_t * zone = (uint8_t *) L->expert_zones + row * D * el;
			uint8_t * x1 = (uint8_t *) L->x1 + row * H * el;
			uint8_t * x3 = (uint8_t *) L->x3 + row * H * el;
			uint8_t * dx1 = (uint8_t *) L->dx1 + row * H * el;
			uint8_t * dx3 = (uint8_t *) L->dx3 + row * H * el;
			uint64_t temp_bytes = (uint64_t) n * H * el;
			if (temp_bytes > half) {
				fprintf(stderr, "Error: expert #%d has too many tokens for current kernel workspace. (# tokens: %d, streamKernelWorkspaceBytes: %lu)\n", e, n, (unsigned long) half);
				return -1;
			}
			uint8_t * temp = ws[which];
			int s = streams[which];
			void * w1 = expert_ptr(L->w1, S, e), * w3 = expert_ptr(L->w3, S, e), * w2 = expert_ptr(L->w2, S, e);
			void * dw2 = expert_ptr(L->dw2, S, e);
			CHECK(dataflow_submit_default_swiglu(h, s, dt, n, H, x1, x3, temp), "failed to submit swiglu recompute");
			CHECK(dataflow_submit_matmul(h, s, dt, dt, DATAFLOW_NONE, dt, cdt, 1, 0, D, H, n, 1.0f, 0.0f, w2, temp, NULL, zone, 0, NULL),
				  "failed to submit w2 recompute matmul");
			CHECK(dataflow_submit_router_bwd_x(h, s, dt, dt, n, D, E, K, e, L->expert_counts_cumsum, L->expert_mapping, L->chosen_experts,
											   L->token_expert_weights, zone, dY, L->d_routed, zone), "failed to submit router bwd x");
			CHECK(dataflow_submit_matmul(h, s, dt, dt, wc_dt, dt, cdt, 0, 1, H, n, D, 1.0f, wbeta, temp, zone, WGRAD_C(dw2), dw2, 0, NULL),
				  "failed to submit dW2 matmul");
			CHECK(dataflow_submit_matmul(h, s, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, H, D, n, 1.0f, 0.0f, w2, zone, NULL, temp, 0, NULL),
				  "failed to submit dh matmul");
			CHECK(dataflow_submit_default_swiglu_bwd_x(h, s, dt, dt, n, H, x1, x3, temp, dx1, dx3), "failed to submit swiglu bwd x");
			CHECK(dataflow_submit_matmul(h, s, dt, dt, DATAFLOW_NONE, dt, cdt, 0, 0, D, H, n, 1.0f, 0.0f, w1, dx1, NULL, zone, 0, NULL),
				  "failed to submit dX(w1) matmul");
			CHECK(dataflow_submit_matmul(h, s, dt, dt, dt, dt, cdt, 0, 0, D, H, n, 1.0f, 1.0f, w3, dx3, zone, zone, 0, NULL),
				  "failed to submit dX(w3) matmul");
			row += (uint64_t) n;
			which ^= 1;
		}
		CHECK(stream_wait(h, cs, ss), "compute stream could not wait for the secondary stream");
	}

	/* gather the expert-side gradients back per token (:3666-3678), softmax-gate backward (:3695-3700) and the
	 * router's contribution to dX (:3707-3714) */
	if (schedule == AMD_MOE_FUSED) {
		/* the same sum without clearing dX first and reading the zeros back */
		CHECK(dataflow_submit_amd_merge_experts_fresh(h, cs, dt, dt, T, D, K, L->expert_zones, L->token_mapping, NULL, dX), "failed to submit merge experts (bwd)");
	} else {
		CHECK((h->set_mem)(h, cs, dX, 0, (uint64_t) T * D * el), "failed to clear dX");
		CHECK(dataflow_submit_default_merge_experts(h, cs, dt, dt, T, D, K, L->expert_zones, L->token_mapping, NULL, dX), "failed to submit merge experts (bwd)");
	}
	CHECK(dataflow_submit_router_gate_bwd_x(h, cs, dt, dt, T, E, K, L->chosen_experts, L->token_expert_weights, L->d_routed), "failed to submit router gate bwd x");
	CHECK(dataflow_submit_matmul(h, cs, dt, dt, dt, dt, cdt, 0, 0, D, E, T, 1.0f, 1.0f, L->w_router, L->d_routed, dX, dX,
								 L->kernel_workspace_bytes, L->kernel_workspace), "failed to submit router dX matmul");

	/* bwd_w: re-dispatch the inputs (:4062-4066), dW1 / dW3 (:4101-4148), dWr (:4174-4181) */
	/* The stacked dW1 | dW3 GEMM can take the k-rows of X through expert_mapping (no re-dispatch), as the up-projection
	 * does in the forward; here that form loses: a k-row of a tile is a 512-byte piece of a scattered row of X, and the
	 * launch takes longer by more than the copy costs (config 4: 5.47 against 5.39 ms per step, config 5: 38.6 against
	 * 38.0).  The copy + packed form is the default; AMD_MOE_BWD_GATHER in the environment selects the gathered one,
	 * which gives the same bits. */
	const int gathered = side_by_side && gather_allowed(T, D) && getenv("AMD_MOE_BWD_GATHER") != NULL;
	if (!gathered) {
		CHECK(dataflow_submit_default_prepare_experts(h, cs, dt, dt, T, D, K, X, L->token_mapping, L->expert_zones), "failed to submit prepare experts (bwd_w)");
	}
	if (gathered) {
		/* no re-dispatch: the GEMM takes the rows of X through expert_mapping (same values, same result) */
		CHECK(dataflow_submit_amd_grouped_matmul_gathered(h, cs, dt, dt, wc_dt, dt, cdt, 0, 1, AMD_GROUPED_RAGGED_K, D, 0, 2 * H, E, L->expert_counts_cumsum,
														  1.0f, wbeta, X, 0, L->dx1, WGRAD_C(L->dw1), L->dw1, S, L->expert_mapping, T),
			  "failed to submit gathered grouped dW1|dW3 matmul");
	} else if (side_by_side) {
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, wc_dt, dt, cdt, 0, 1, AMD_GROUPED_RAGGED_K, D, 0, 2 * H, E, L->expert_counts_cumsum,
												 1.0f, wbeta, L->expert_zones, 0, L->dx1, WGRAD_C(L->dw1), L->dw1, S), "failed to submit grouped dW1|dW3 matmul");
	} else if (schedule != AMD_MOE_PER_EXPERT) {
		/* independent of each other: the second on the secondary stream, as for the up-projections */
		CHECK(stream_wait(h, ss, cs), "secondary stream could not wait for the compute stream");
		CHECK(dataflow_submit_amd_grouped_matmul(h, cs, dt, dt, wc_dt, dt, cdt, 0, 1, AMD_GROUPED_RAGGED_K, D, 0, H, E, L->expert_counts_cumsum,
												 1.0f, wbeta, L->expert_zones, 0, L->dx1, WGRAD_C(L->dw1), L->dw1, S), "failed to submit grouped dW1 matmul");
		CHECK(dataflow_submit_amd_grouped_matmul(h, ss, dt, dt, wc_dt, dt, cdt, 0, 1, AMD_GROUPED_RAGGED_K, D, 0, H, E, L->expert_counts_cumsum,
												 1.0f, wbeta, L->expert_zones, 0, L->dx3, WGRAD_C(L->dw3), L->dw3, S), "failed to submit grouped dW3 matmul");
		CHECK(stream_wait(h, cs, ss), "compute stream could not wait for the secondary stream");
	} else {
		CHECK(stream_wait(h, ss, cs), "secondary stream could not wait for the compute stream");
		int streams[2] = {cs, ss};
		int which = 0;
		uint64_t row = 0;
		for (int e = 0; e < E; e++) {
			int n = L->host_expert_counts[e];
			if (n == 0) {
				continue;
			}
			uint8_t * zone = (uint8_t *) L->expert_zones + row * D * el;
			uint8_t * dx1 = (uint8_t *) L->dx1 + row * H * el;
			uint8_t * dx3 = (uint8_t *) L->dx3 + row * H * el;
			void * dw1 = expert_ptr(L->dw1, S, e), * dw3 = expert_ptr(L->dw3, S, e);
			int s = streams[which];
			CHECK(dataflow_submit_matmul(h, s, dt, dt, wc_dt, dt, cdt, 0, 1, D, n, H, 1.0f, wbeta, zone, dx1, WGRAD_C(dw1), dw1, 0, NULL), "failed to submit dW1 matmul");
			CHECK(dataflow_submit_matmul(h, s, dt, dt, wc_dt, dt, cdt, 0, 1, D, n, H, 1.0f, wbeta, zone, dx3, WGRAD_C(dw3), dw3, 0, NULL), "failed to submit dW3 matmul");
			row += (uint64_t) n;
			which ^= 1;
		}
		CHECK(stream_wait(h, cs, ss), "compute stream could not wait for the secondary stream");
	}
	CHECK(dataflow_submit_matmul(h, cs, dt, dt, wc_dt, dt, cdt, 0, 1, D, T, E, 1.0f, wbeta, X, L->d_routed, WGRAD_C(L->dw_router), L->dw_router,
								 L->kernel_workspace_bytes, L->kernel_workspace), "failed to submit router dW matmul");
#undef WGRAD_C
	return 0;
}
