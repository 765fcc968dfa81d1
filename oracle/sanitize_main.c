/*
 * sanitize_main.c -- TEST INFRASTRUCTURE: a driver that runs the CPU-side C of this repository under AddressSanitizer
 * and UndefinedBehaviorSanitizer (oracle/Makefile, target `asan`; tests/test_sanitizers.py builds and runs it).
 *
 * Covered: the oracle (moe_oracle.c: every kernel restatement through the layer's forward and backward, plus the
 * norm / AdamW / cast functions, on small and ragged shapes), and the host-side C of the product that needs no GPU:
 * the table, fingerprint and datatype utilities (csrc/core/dataflow_core.c), every op skeleton setter
 * (csrc/ops/dataflow_ops.c) and the block weight file layout and saved-array naming (csrc/layer/moe_files.c).
 * Exit status 0 and no sanitizer report = clean.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "moe_oracle.h"
#include "dataflow_amd.h"
#include "dataflow_amd_ops.h"
#include "moe_layer.h"

static uint32_t rng_state = 12345u;
static float rnd(void) {
	rng_state = rng_state * 1664525u + 1013904223u;
	return (float) ((rng_state >> 8) & 0xffff) / 32768.0f - 1.0f;
}
static uint16_t bf(float f) {
	uint32_t b;
	memcpy(&b, &f, 4);
	b += 0x7fffu + ((b >> 16) & 1u);
	return (uint16_t) (b >> 16);
}
static uint16_t * rand_bf16(size_t n, float scale) {
	uint16_t * p = (uint16_t *) malloc(n * 2 + 2);
	for (size_t i = 0; i < n; i++) {
		p[i] = bf(rnd() * scale);
	}
	return p;
}

static int run_layer(int T, int D, int E, int K, int H) {
	const size_t R = (size_t) T * K;
	Oracle_Moe_Layer L;
	memset(&L, 0, sizeof(L));
	L.T = T; L.D = D; L.E = E; L.K = K; L.H = H;
	uint16_t * Wr = rand_bf16((size_t) E * D, 0.2f), * W1 = rand_bf16((size_t) E * H * D, 0.1f), * W3 = rand_bf16((size_t) E * H * D, 0.1f),
			 * W2 = rand_bf16((size_t) E * D * H, 0.1f), * X = rand_bf16((size_t) T * D, 1.0f), * dY = rand_bf16((size_t) T * D, 1.0f),
			 * out = rand_bf16((size_t) T * D, 1.0f);
	L.Wr = Wr; L.W1 = W1; L.W3 = W3; L.W2 = W2; L.w_stride = (size_t) H * D;
	L.logits = (uint16_t *) calloc((size_t) T * E, 2);
	L.weights = (float *) calloc((size_t) T * K, 4);
	L.chosen = (uint16_t *) calloc((size_t) T * K, 2);
	L.counts = (int *) calloc((size_t) E + 1, 4);
	L.cumsum = (int *) calloc((size_t) E, 4);
	L.expert_mapping = (int *) calloc(R, 4);
	L.token_mapping = (int *) calloc(R, 4);
	L.x1 = (uint16_t *) calloc(R * H, 2); L.x3 = (uint16_t *) calloc(R * H, 2);
	L.zones = (uint16_t *) calloc(R * D, 2); L.temp = (uint16_t *) calloc(R * H, 2);
	L.dx1 = (uint16_t *) calloc(R * H, 2); L.dx3 = (uint16_t *) calloc(R * H, 2);
	L.dlogits = (uint16_t *) calloc((size_t) T * E, 2);
	L.dWr = (uint16_t *) calloc((size_t) E * D, 2);
	L.dW1 = (uint16_t *) calloc((size_t) E * H * D, 2); L.dW3 = (uint16_t *) calloc((size_t) E * H * D, 2); L.dW2 = (uint16_t *) calloc((size_t) E * D * H, 2);
	uint16_t * dX = (uint16_t *) calloc((size_t) T * D, 2);
	int ret = oracle_moe_forward(&L, X, NULL, out);
	if (!ret) {
		ret = oracle_moe_backward(&L, X, dY, dX);
	}
	/* the functions around the layer */
	float * rms = (float *) calloc((size_t) T, 4);
	uint16_t * w = rand_bf16((size_t) D, 1.0f), * normed = (uint16_t *) calloc((size_t) T * D, 2), * dw = (uint16_t *) calloc((size_t) D, 2);
	oracle_rms_norm(T, D, 1e-5f, w, X, normed, rms);
	oracle_rms_norm_recompute(T, D, w, rms, X, normed);
	oracle_rms_norm_bwd_x(T, D, 1e-5f, rms, w, X, dY, dX, normed);
	oracle_rms_norm_bwd_w(T, D, 1e-5f, rms, X, dY, dw);
	uint16_t * mean = (uint16_t *) calloc((size_t) E * D, 2), * var = (uint16_t *) calloc((size_t) E * D, 2);
	uint16_t * param = rand_bf16((size_t) E * D, 0.1f);
	oracle_adamw_step((uint64_t) E * D, 1, 1e-3f, 0.9f, 0.999f, 0.01f, 1e-8f, param, L.dWr, mean, var);
	float * wide = (float *) calloc((size_t) T * D, 4);
	oracle_cast_bf16_fp32((uint64_t) T * D, X, wide);
	oracle_cast_and_add((uint64_t) T * D, 0.5f, wide, 2.0f, dY, dX);
	/* the other element types: fp32 logits through the selection, fp32 and fp16 rows through SwiGLU and its backward */
	{
		float * flog = (float *) calloc((size_t) T * E, 4), * fw = (float *) calloc((size_t) T * K, 4);
		uint16_t * fch = (uint16_t *) calloc((size_t) T * K, 2);
		int * fcounts = (int *) calloc((size_t) E + 1, 4), * fcum = (int *) calloc((size_t) E, 4);
		for (size_t i = 0; i < (size_t) T * E; i++) {
			flog[i] = rnd();
		}
		oracle_select_experts_fp32(T, E, K, flog, fw, fch, fcounts, fcum, NULL);
		float * f1 = (float *) calloc((size_t) T * D, 4), * f3 = (float *) calloc((size_t) T * D, 4), * fo = (float *) calloc((size_t) T * D, 4);
		uint16_t * h1 = (uint16_t *) calloc((size_t) T * D, 2), * h3 = (uint16_t *) calloc((size_t) T * D, 2), * ho = (uint16_t *) calloc((size_t) T * D, 2);
		for (size_t i = 0; i < (size_t) T * D; i++) {
			f1[i] = rnd() * 4.0f; f3[i] = rnd();
			h1[i] = oracle_f32_to_fp16(f1[i] * 1e4f); h3[i] = oracle_f32_to_fp16(f3[i] * 1e-6f);      /* overflow and subnormals on purpose */
		}
		oracle_swiglu_typed(0, T, D, f1, f3, fo);
		oracle_swiglu_bwd_x_typed(0, T, D, f1, f3, fo, f1, f3);
		oracle_swiglu_typed(1, T, D, h1, h3, ho);
		oracle_swiglu_bwd_x_typed(1, T, D, h1, h3, ho, h1, h3);
		/* typed matmul on the arrays above: [T][D] x [T][D]^T -> [T][T], every kind, both layouts of each operand */
		float * fd = (float *) calloc((size_t) T * T, 4);
		uint16_t * hd = (uint16_t *) calloc((size_t) T * T, 2);
		for (int tr = 0; tr < 4; tr++) {
			/* read as [D][T] instead where an operand is taken k-major: same bytes, K = D or T swapped accordingly */
			int ta = tr & 1, tb = tr >> 1;
			if (oracle_matmul_typed(ORACLE_ELEM_FP32, ORACLE_ELEM_FP32, ta, tb, T, D, T, 1.0f, 0.0f, f1, f3, NULL, fd) ||
				oracle_matmul_typed(ORACLE_ELEM_FP16, ORACLE_ELEM_FP16, ta, tb, T, D, T, 0.5f, 1.0f, h1, h3, hd, hd) ||
				oracle_matmul_typed(ORACLE_ELEM_FP16, ORACLE_ELEM_FP32, ta, tb, T, D, T, 1.0f, 1.0f, h1, h3, fd, fd) ||
				oracle_matmul_typed(ORACLE_ELEM_BF16, ORACLE_ELEM_FP32, ta, tb, T, D, T, 1.0f, 0.0f, h1, h3, NULL, fd)) {
				fprintf(stderr, "typed matmul oracle refused a valid kind\n");
				return 1;
			}
		}
		if (oracle_matmul_typed(9, 0, 1, 0, 1, 1, 1, 1.0f, 0.0f, f1, f3, NULL, fd) != -1) {
			fprintf(stderr, "typed matmul oracle accepted an unknown kind\n");
			return 1;
		}
		void * more[] = {flog, fw, fch, fcounts, fcum, f1, f3, fo, h1, h3, ho, fd, hd};
		for (size_t i = 0; i < sizeof(more) / sizeof(more[0]); i++) {
			free(more[i]);
		}
	}
	void * all[] = {Wr, W1, W3, W2, X, dY, out, L.logits, L.weights, L.chosen, L.counts, L.cumsum, L.expert_mapping, L.token_mapping, L.x1, L.x3,
					L.zones, L.temp, L.dx1, L.dx3, L.dlogits, L.dWr, L.dW1, L.dW3, L.dW2, dX, rms, w, normed, dw, mean, var, param, wide};
	for (size_t i = 0; i < sizeof(all) / sizeof(all[0]); i++) {
		free(all[i]);
	}
	return ret;
}

static uint64_t fingerprint_hash(void * key, uint64_t table_size) {
	uint64_t v;
	memcpy(&v, (uint8_t *) key + DATAFLOW_OP_IDENTIFIER_FINGERPRINT_NUM_BYTES - 8, 8);
	return v % table_size;
}

static int run_host_side(void) {
	const DataflowDatatype BF = DATAFLOW_BF16;
	Op_Skeleton sk[26];
	int n = 0;
	dataflow_set_matmul_skeleton(&sk[n++]);
	dataflow_set_default_swiglu_skeleton(&sk[n++], BF);
	dataflow_set_default_swiglu_bwd_x_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_select_experts_skeleton(&sk[n++], BF);
	dataflow_set_default_build_expert_mapping_skeleton(&sk[n++]);
	dataflow_set_default_prepare_expert_zone_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_prepare_experts_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_merge_expert_result_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_merge_experts_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_router_bwd_x_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_router_gate_bwd_x_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_rms_norm_skeleton(&sk[n++], BF);
	dataflow_set_default_rms_norm_recompute_skeleton(&sk[n++], BF);
	dataflow_set_default_rms_norm_bwd_x_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_rms_norm_bwd_w_skeleton(&sk[n++], BF, BF);
	dataflow_set_default_rms_norm_bwd_w_combine_skeleton(&sk[n++], BF);
	dataflow_set_default_adamw_step_skeleton(&sk[n++], BF, BF, BF, BF);
	dataflow_set_default_cast_skeleton(&sk[n++], BF, DATAFLOW_FP32, DATAFLOW_NONE);
	dataflow_set_default_cast_and_add_skeleton(&sk[n++], DATAFLOW_FP32, BF, BF);
	dataflow_set_amd_grouped_matmul_skeleton(&sk[n++]);
	dataflow_set_amd_router_bwd_x_all_skeleton(&sk[n++], BF, BF);
	dataflow_set_amd_grouped_matmul_gathered_skeleton(&sk[n++]);
	dataflow_set_amd_merge_experts_fresh_skeleton(&sk[n++], BF, BF);
	dataflow_set_amd_swiglu_strided_skeleton(&sk[n++], BF);
	dataflow_set_amd_prepare_experts_scaled_skeleton(&sk[n++], BF, BF);
	dataflow_set_amd_swiglu_bwd_x_routed_skeleton(&sk[n++], BF, BF);
	/* a small table that has to grow: insert, find, remove every fingerprint */
	Dataflow_Table table;
	if (dataflow_init_table(&table, fingerprint_hash, DATAFLOW_OP_IDENTIFIER_FINGERPRINT_NUM_BYTES, sizeof(int), 4, 1 << 16, 0.5f, 0.1f)) {
		return -1;
	}
	for (int i = 0; i < n; i++) {
		int value = i;
		if (dataflow_insert_table(&table, sk[i].identifier.fingerprint, &value)) {
			return -1;
		}
	}
	for (int i = 0; i < n; i++) {
		int value = -1;
		void * ret = &value;
		if (dataflow_find_table(&table, sk[i].identifier.fingerprint, true, &ret) < 0 || value != i) {
			fprintf(stderr, "table lookup of skeleton %d failed\n", i);
			return -1;
		}
	}
	for (int i = 0; i < n; i++) {
		int value = -1;
		if (dataflow_remove_table(&table, sk[i].identifier.fingerprint, &value) || value != i) {
			return -1;
		}
	}
	dataflow_destroy_table(&table);
	for (int dt = 0; dt < 16; dt++) {
		(void) dataflow_sizeof_element((DataflowDatatype) dt);
		(void) dataflow_datatype_as_string((DataflowDatatype) dt);
	}
	Amd_Moe_Block_Offsets off;
	if (amd_moe_block_weight_offsets(4096, 4096, 1024, 64, 1024, BF, 256, &off) || amd_moe_block_weight_offsets(72, 64, 32, 4, 24, BF, 256, &off)) {
		return -1;
	}
	char path[64];
	(void) amd_moe_saved_array_path(path, sizeof(path), "/tmp/some/rather/long/directory/name/for/the/saved/arrays", 3, 7, 11, 1, "x_router_logits");   /* too long: an error, no overflow */
	char longer[512];
	if (amd_moe_saved_array_path(longer, sizeof(longer), "/tmp/saved", 3, 7, 11, 0, "x_router_logits")) {
		return -1;
	}
	return 0;
}

int main(void) {
	if (run_layer(64, 32, 8, 2, 64) || run_layer(1, 16, 4, 2, 8) || run_layer(37, 24, 12, 4, 40) || run_layer(20, 16, 64, 8, 8)) {
		fprintf(stderr, "oracle layer failed\n");
		return 1;
	}
	if (run_host_side()) {
		fprintf(stderr, "host-side checks failed\n");
		return 1;
	}
	printf("sanitizer run clean\n");
	return 0;
}
