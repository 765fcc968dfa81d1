/*
 * launch_config.c -- grid / block / LDS sizes for the native gfx950 kernels, looked up by symbol
 * ("<op>_set_launch_config") when the handle registers the code object.
 *
 * Same role as backends/nvidia/src/ops/src/native/src/moe/moe_config.c and
 * .../activations/swiglu_config.c; the shapes are chosen for CDNA4 (64-lane waves, 256 compute units,
 * launches of thousands of 256-thread work-groups) rather than derived from the SM count.
 * A grid of 0 tells the handle there is nothing to launch.
 */
#include "dataflow_amd.h"

#include <stdint.h>
#include <stdio.h>
#include <string.h>

#define ARG_INT(op, i) (*((int *) ((op)->op_args[(i)])))

static void set_1d(Hip_Launch_Config * cfg, unsigned int grid, unsigned int block, unsigned int lds) {
	cfg->gridDimX = grid;
	cfg->gridDimY = 1;
	cfg->gridDimZ = 1;
	cfg->blockDimX = block;
	cfg->blockDimY = 1;
	cfg->blockDimZ = 1;
	cfg->sharedMemBytes = lds;
}

static int check_row_len(const char * op, int len) {
	if (len <= 0 || (len & 7)) {
		fprintf(stderr, "Error: %s needs a row length that is a positive multiple of 8, got %d...\n", op, len);
		return -1;
	}
	return 0;
}

/* a group of 2^ceil(log2 top_k) lanes per token (one slot per lane), 32 tokens per work-group; the expert
 * histogram of the work-group in dynamic LDS */
int default_select_experts_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int total_tokens = ARG_INT(op, 0);
	int n_experts = ARG_INT(op, 1);
	int top_k = ARG_INT(op, 2);
	if (total_tokens < 0 || n_experts < 1 || n_experts > 4096 || top_k < 1 || top_k > n_experts) {
		fprintf(stderr, "Error: select_experts needs 1 <= top_k <= n_experts <= 4096, got tokens=%d experts=%d top_k=%d...\n", total_tokens, n_experts, top_k);
		return -1;
	}
	if (top_k > 32) {
		fprintf(stderr, "Error: select_experts supports top_k up to 32, got %d...\n", top_k);
		return -1;
	}
	unsigned int lds = (unsigned int) n_experts * 4u;
	/* one slot per lane: a group of `lanes` lanes (the power of two >= top_k) per token, 32 tokens per work-group */
	unsigned int lanes = 1;
	while ((int) lanes < top_k) {
		lanes <<= 1;
	}
	/* an empty batch still has to draw the ticket and write zero counts: launch one work-group */
	unsigned int grid = total_tokens > 0 ? (unsigned int) ((total_tokens + 31) / 32) : 1u;
	set_1d(cfg, grid, 32u * lanes, lds);
	return 0;
}

/* at most 256 work-groups, each owning a 256-aligned slice of the T*K entries */
int default_build_expert_mapping_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int num_tokens = ARG_INT(op, 0);
	int n_experts = ARG_INT(op, 1);
	int top_k = ARG_INT(op, 2);
	unsigned int lds = 6u * (unsigned int) n_experts * 4u;
	/* private histograms of the four waves (routing.hip, build_private_copies): up to 32 counters per expert and wave */
	unsigned int copies = 32;
	while (copies > 1 && (unsigned int) n_experts * copies > 2048u) {
		copies >>= 1;
	}
	if (copies > 1) {
		lds += 4u * (unsigned int) n_experts * copies * 4u;
	}
	if (num_tokens < 0 || n_experts < 1 || top_k < 1 || lds > 65536u) {
		fprintf(stderr, "Error: build_expert_mapping needs n_experts in [1, 2730], got tokens=%d experts=%d top_k=%d...\n", num_tokens, n_experts, top_k);
		return -1;
	}
	long entries = (long) num_tokens * (long) top_k;
	long groups = (entries + 255) / 256;
	if (groups > 256) {
		groups = 256;
	}
	if (groups < 1) {
		groups = 1;
	}
	set_1d(cfg, (unsigned int) groups, 256, lds);
	return 0;
}

int default_prepare_experts_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int total_tokens = ARG_INT(op, 0);
	if (check_row_len("prepare_experts", ARG_INT(op, 1))) {
		return -1;
	}
	set_1d(cfg, total_tokens > 0 ? (unsigned int) total_tokens : 0u, 256, 0);
	return 0;
}

int amd_prepare_experts_scaled_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int total_tokens = ARG_INT(op, 0);
	if (check_row_len("prepare_experts_scaled", ARG_INT(op, 1))) {
		return -1;
	}
	set_1d(cfg, total_tokens > 0 ? (unsigned int) total_tokens : 0u, 256, 0);
	return 0;
}

/* the row count of the expert is only known on the device: a fixed grid strides over the rows */
int default_prepare_expert_zone_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) fn;
	if (check_row_len("prepare_expert_zone", ARG_INT(op, 0))) {
		return -1;
	}
	set_1d(cfg, (unsigned int) (handle->get_num_procs)(handle) * 8u, 256, 0);
	return 0;
}

int default_merge_experts_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int total_tokens = ARG_INT(op, 0);
	if (check_row_len("merge_experts", ARG_INT(op, 1))) {
		return -1;
	}
	set_1d(cfg, total_tokens > 0 ? (unsigned int) total_tokens : 0u, 256, 0);
	return 0;
}

int default_merge_expert_result_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int rows = ARG_INT(op, 0);
	if (check_row_len("merge_expert_result", ARG_INT(op, 1))) {
		return -1;
	}
	set_1d(cfg, rows > 0 ? (unsigned int) rows : 0u, 256, 0);
	return 0;
}

int default_router_bwd_x_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int rows = ARG_INT(op, 0);
	if (check_row_len("router_bwd_x", ARG_INT(op, 1))) {
		return -1;
	}
	set_1d(cfg, rows > 0 ? (unsigned int) rows : 0u, 256, 0);
	return 0;
}

int amd_router_bwd_x_all_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int tokens = ARG_INT(op, 0);
	if (check_row_len("router_bwd_x_all", ARG_INT(op, 1))) {
		return -1;
	}
	set_1d(cfg, tokens > 0 ? (unsigned int) tokens : 0u, 256, 0);
	return 0;
}

static int check_row_stride(const char * op, int cols, int stride) {
	if (stride < cols || (stride & 7)) {
		fprintf(stderr, "Error: %s needs a row stride that is a multiple of 8 and at least the row length %d, got %d...\n", op, cols, stride);
		return -1;
	}
	return 0;
}

int amd_swiglu_strided_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int rows = ARG_INT(op, 0);
	int cols = ARG_INT(op, 1);
	if (rows < 0 || check_row_len("swiglu_strided", cols) || check_row_stride("swiglu_strided", cols, ARG_INT(op, 2))) {
		return -1;
	}
	unsigned long vecs = ((unsigned long) rows * (unsigned long) cols) >> 3;
	unsigned long groups = (vecs + 255) / 256;
	if (groups > 0x7fffffffUL) {
		fprintf(stderr, "Error: swiglu_strided over %d x %d elements needs too many work-groups...\n", rows, cols);
		return -1;
	}
	set_1d(cfg, (unsigned int) groups, 256, 0);
	return 0;
}

/* one wave per routed row, 4 rows per work-group */
int amd_swiglu_bwd_x_routed_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int rows = ARG_INT(op, 0);
	int top_k = ARG_INT(op, 3);
	if (rows < 0 || check_row_len("swiglu_bwd_x_routed", ARG_INT(op, 1))) {
		return -1;
	}
	if (top_k < 1 || top_k > 64) {
		fprintf(stderr, "Error: swiglu_bwd_x_routed needs 1 <= top_k <= 64 (one lane per slot), got %d...\n", top_k);
		return -1;
	}
	if (check_row_stride("swiglu_bwd_x_routed", ARG_INT(op, 1), ARG_INT(op, 4)) || check_row_stride("swiglu_bwd_x_routed", ARG_INT(op, 1), ARG_INT(op, 5))) {
		return -1;
	}
	set_1d(cfg, (unsigned int) ((rows + 3) / 4), 256, 0);
	return 0;
}

int default_router_gate_bwd_x_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int tokens = ARG_INT(op, 0);
	set_1d(cfg, tokens > 0 ? (unsigned int) ((tokens + 255) / 256) : 0u, 256, 0);
	return 0;
}

static int elementwise_config(Hip_Launch_Config * cfg, Op * op, const char * name) {
	int rows = ARG_INT(op, 0);
	int cols = ARG_INT(op, 1);
	if (rows < 0 || check_row_len(name, cols)) {
		return -1;
	}
	unsigned long vecs = ((unsigned long) rows * (unsigned long) cols) >> 3;
	unsigned long groups = (vecs + 255) / 256;
	if (groups > 0x7fffffffUL) {
		fprintf(stderr, "Error: %s launch of %lu work-groups is too large...\n", name, groups);
		return -1;
	}
	set_1d(cfg, (unsigned int) groups, 256, 0);
	return 0;
}

int default_swiglu_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	return elementwise_config(cfg, op, "swiglu");
}

int default_swiglu_bwd_x_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	return elementwise_config(cfg, op, "swiglu_bwd_x");
}

/* ---- RMS norm (backends/nvidia/src/ops/src/native/src/norm/rms_norm_config.c) ---- */

static int row_kernel_config(Hip_Launch_Config * cfg, Op * op, const char * name) {
	int rows = ARG_INT(op, 0);
	int cols = ARG_INT(op, 1);
	if (rows < 0 || check_row_len(name, cols)) {
		return -1;
	}
	set_1d(cfg, (unsigned int) rows, 256, 0);
	return 0;
}

int default_rms_norm_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	return row_kernel_config(cfg, op, "rms_norm");
}

int default_rms_norm_recompute_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	return row_kernel_config(cfg, op, "rms_norm_recompute");
}

int default_rms_norm_bwd_x_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	return row_kernel_config(cfg, op, "rms_norm_bwd_x");
}

/* As many work-groups as the workspace has room for partial rows, at most 512 and at most one per row.
 * The caller's workspace starts with a 256-byte header (the work-group count), then the fp32 partial rows:
 * op_args[8] is its total size (libdataflowops/src/submit_ops/norm_ops.c:92-108). */
int default_rms_norm_bwd_w_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int rows = ARG_INT(op, 0);
	int cols = ARG_INT(op, 1);
	uint64_t workspace_bytes = *((uint64_t *) op->op_args[8]);
	if (rows < 0 || check_row_len("rms_norm_bwd_w", cols)) {
		return -1;
	}
	uint64_t per_group = (uint64_t) cols * 4u;
	uint64_t room = workspace_bytes > 256 ? (workspace_bytes - 256) / per_group : 0;
	if (room < 1) {
		fprintf(stderr, "Error: rms_norm_bwd_w needs a workspace of at least %lu bytes, got %lu...\n",
				(unsigned long) (256 + per_group), (unsigned long) workspace_bytes);
		return -1;
	}
	uint64_t groups = 512;
	if (groups > room) {
		groups = room;
	}
	if (groups > (uint64_t) rows) {
		groups = (uint64_t) rows;
	}
	if (groups == 0) {
		groups = 1;                                    /* no rows: still record the count and write one zero row */
	}
	set_1d(cfg, (unsigned int) groups, 256, 0);
	cfg->gridDimY = (unsigned int) ((cols / 8 + 255) / 256);
	return 0;
}

int default_rms_norm_bwd_w_combine_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int model_dim = ARG_INT(op, 1);
	if (model_dim < 1) {
		fprintf(stderr, "Error: rms_norm_bwd_w_combine needs a positive model dim, got %d...\n", model_dim);
		return -1;
	}
	set_1d(cfg, (unsigned int) ((model_dim + 63) / 64), 1024, 0);
	return 0;
}

/* ---- AdamW (backends/nvidia/src/ops/src/native/src/optimizer/adamw_step_config.c) ---- */

int default_adamw_step_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	uint64_t num_els = *((uint64_t *) op->op_args[0]);
	int step_num = ARG_INT(op, 1);
	if (step_num < 1) {
		fprintf(stderr, "Error: adamw step needs a step number of at least 1 (bias correction divides by 1 - beta^step), got %d...\n", step_num);
		return -1;
	}
	uint64_t groups = (num_els + 2047) / 2048;               /* 8 elements per lane */
	if (groups > 8192) {
		groups = 8192;
	}
	set_1d(cfg, (unsigned int) groups, 256, 0);
	return 0;
}

/* ---- casts (backends/nvidia/src/ops/src/native/src/cast/cast_config.c:3-54) ---- */

static void set_elementwise_8(Hip_Launch_Config * cfg, uint64_t num_els) {
	uint64_t groups = (num_els + 2047) / 2048;               /* 8 elements per lane */
	if (groups > 8192) {
		groups = 8192;
	}
	set_1d(cfg, (unsigned int) groups, 256, 0);              /* no elements: an empty grid, nothing is launched */
}

int default_cast_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	set_elementwise_8(cfg, *((uint64_t *) op->op_args[0]));
	return 0;
}

int default_cast_and_add_set_launch_config(Hip_Launch_Config * cfg, Dataflow_Handle * handle, Hip_Function * fn, Op * op) {
	(void) handle; (void) fn;
	int64_t num_els = *((int64_t *) op->op_args[0]);
	if (num_els < 0) {
		fprintf(stderr, "Error: cast_and_add with a negative element count %ld...\n", (long) num_els);
		return -1;
	}
	set_elementwise_8(cfg, (uint64_t) num_els);
	return 0;
}
