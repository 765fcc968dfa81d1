/*
 * moe_oracle.c -- scalar CPU restatement of the reference's MoE-layer kernels (see moe_oracle.h).
 * TEST INFRASTRUCTURE ONLY: never linked into or loaded by the product library.
 */
#include "moe_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#include <stdio.h>

/* ---------------------------------------------------------------- bf16 */

static inline float bf_to_f(uint16_t v) {
	uint32_t bits = ((uint32_t) v) << 16;
	float f;
	memcpy(&f, &bits, sizeof(f));
	return f;
}

/* Round to nearest even, as __float2bfloat16 / __float22bfloat162_rn do on the device
 * (swiglu.cu:134-137, merge_expert_result.cu:240-243). */
static inline uint16_t f_to_bf(float f) {
	uint32_t bits;
	memcpy(&bits, &f, sizeof(bits));
	if ((bits & 0x7fffffffu) > 0x7f800000u) {
		return (uint16_t) ((bits >> 16) | 0x0040u);
	}
	uint32_t lsb = (bits >> 16) & 1u;
	bits += 0x7fffu + lsb;
	return (uint16_t) (bits >> 16);
}

float oracle_bf16_to_f32(uint16_t v) { return bf_to_f(v); }
uint16_t oracle_f32_to_bf16(float f) { return f_to_bf(f); }

#define BF(v) bf_to_f(v)
#define TOBF(f) f_to_bf(f)

/* ---------------------------------------------------------------- matmul */

/* fp64 dot of two strided bf16 vectors, eight partial sums so the compiler can vectorise */
static double dot_bf16(const uint16_t * a, size_t sa, const uint16_t * b, size_t sb, int n) {
	double acc[8] = {0, 0, 0, 0, 0, 0, 0, 0};
	int k = 0;
	if (sa == 1 && sb == 1) {
		for (; k + 8 <= n; k += 8) {
			for (int j = 0; j < 8; j++) {
				acc[j] += (double) BF(a[k + j]) * (double) BF(b[k + j]);
			}
		}
	}
	for (; k < n; k++) {
		acc[k & 7] += (double) BF(a[(size_t) k * sa]) * (double) BF(b[(size_t) k * sb]);
	}
	return ((acc[0] + acc[1]) + (acc[2] + acc[3])) + ((acc[4] + acc[5]) + (acc[6] + acc[7]));
}

void oracle_matmul(int transa, int transb, int M, int K, int N, float alpha, float beta,
				   const uint16_t * A, const uint16_t * B, const uint16_t * C, uint16_t * D) {
	/* op(A)[m][k]: transa -> A[m*K + k], else A[k*M + m].  op(B)[k][n]: transb -> B[k*N + n], else B[n*K + k].
	 * Output element (m, n) lives at D[n*M + m]  (matmul_helper.c:345-425: column-major, ld = M). */
	int use_c = (C != NULL) && (beta != 0.0f);

	/* when an operand is strided along k, make a k-contiguous copy once so the inner loop streams */
	uint16_t * At = NULL;
	uint16_t * Bt = NULL;
	if (!transa) {
		At = malloc((size_t) M * (size_t) K * sizeof(uint16_t) + 16);
		#pragma omp parallel for schedule(static)
		for (int m = 0; m < M; m++) {
			for (int k = 0; k < K; k++) {
				At[(size_t) m * K + k] = A[(size_t) k * M + m];
			}
		}
	}
	if (transb) {
		Bt = malloc((size_t) N * (size_t) K * sizeof(uint16_t) + 16);
		#pragma omp parallel for schedule(static)
		for (int n = 0; n < N; n++) {
			for (int k = 0; k < K; k++) {
				Bt[(size_t) n * K + k] = B[(size_t) k * N + n];
			}
		}
	}
	const uint16_t * Ak = transa ? A : At;
	const uint16_t * Bk = transb ? Bt : B;

	#pragma omp parallel for schedule(static)
	for (int n = 0; n < N; n++) {
		for (int m = 0; m < M; m++) {
			double acc = dot_bf16(Ak + (size_t) m * K, 1, Bk + (size_t) n * K, 1, K);
			double r = (double) alpha * acc;
			if (use_c) {
				r += (double) beta * (double) BF(C[(size_t) n * M + m]);
			}
			D[(size_t) n * M + m] = TOBF((float) r);
		}
	}
	free(At);
	free(Bt);
}

/* ---------------------------------------------------------------- select_experts */

/* logits_bf16 or logits_f32 is given; the two kernels differ in the element type and in the softmax's difference, which
 * the bf16 kernel rounds to bf16 (:480, :488) and the fp32 kernel (select_experts.cu:3-295, :181, :189) does not */
static void select_experts_any(int total_tokens, int n_experts, int top_k, const uint16_t * logits_bf16, const float * logits_f32,
							   float * token_expert_weights, uint16_t * chosen_experts,
							   int * expert_counts, int * expert_counts_cumsum, int * host_expert_counts) {

	float * val = malloc(sizeof(float) * (size_t) top_k);
	uint16_t * idx = malloc(sizeof(uint16_t) * (size_t) top_k);

	for (int t = 0; t < total_tokens; t++) {
		const size_t row = (size_t) t * n_experts;

		/* select_experts.cu:399-411: slots start at -inf / 0xFFFF, running minimum at slot 0 */
		for (int k = 0; k < top_k; k++) {
			val[k] = -INFINITY;
			idx[k] = 0xFFFF;
		}
		float min_val = -INFINITY;
		int min_slot = 0;
		float max_val = -INFINITY;

		for (int e = 0; e < n_experts; e++) {
			float v = logits_bf16 ? BF(logits_bf16[row + e]) : logits_f32[row + e];
			/* :440 strict greater-than against the running minimum (bf16 values compare like their floats) */
			if (v > min_val) {
				if (v > max_val) {
					max_val = v;
				}
				val[min_slot] = v;
				idx[min_slot] = (uint16_t) e;
				/* :449-462 rescan: smallest value; among equal values the slot holding the larger expert id */
				min_val = INFINITY;
				min_slot = 0;
				uint16_t min_exp = 0xFFFF;
				for (int k = 0; k < top_k; k++) {
					if ((val[k] < min_val) || (val[k] == min_val && idx[k] > min_exp)) {
						min_val = val[k];
						min_slot = k;
						min_exp = idx[k];
					}
				}
			}
		}

		/* :476-497 softmax over the K slots; the difference is formed in bf16 before expf */
		float sum = 0.0f;
		for (int k = 0; k < top_k; k++) {
			float d = logits_bf16 ? BF(TOBF(val[k] - max_val)) : val[k] - max_val;
			sum += expf(d);
		}
		for (int k = 0; k < top_k; k++) {
			float d = logits_bf16 ? BF(TOBF(val[k] - max_val)) : val[k] - max_val;
			token_expert_weights[(size_t) t * top_k + k] = expf(d) / sum;
			chosen_experts[(size_t) t * top_k + k] = idx[k];
			if (idx[k] < n_experts) {
				expert_counts[idx[k]] += 1;
			}
		}
	}
	free(val);
	free(idx);

	/* :509-515 completion ticket (one "block" here) */
	expert_counts[n_experts] += 1;

	/* :535-580 exclusive scan */
	int running = 0;
	for (int e = 0; e < n_experts; e++) {
		expert_counts_cumsum[e] = running;
		running += expert_counts[e];
	}
	/* :585-593 copy to the host-visible array */
	if (host_expert_counts) {
		for (int e = 0; e < n_experts; e++) {
			host_expert_counts[e] = expert_counts[e];
		}
	}
}

void oracle_select_experts(int total_tokens, int n_experts, int top_k,
						   const uint16_t * X_routed, float * token_expert_weights, uint16_t * chosen_experts,
						   int * expert_counts, int * expert_counts_cumsum, int * host_expert_counts) {
	select_experts_any(total_tokens, n_experts, top_k, X_routed, NULL, token_expert_weights, chosen_experts,
					   expert_counts, expert_counts_cumsum, host_expert_counts);
}

void oracle_select_experts_fp32(int total_tokens, int n_experts, int top_k,
								const float * X_routed, float * token_expert_weights, uint16_t * chosen_experts,
								int * expert_counts, int * expert_counts_cumsum, int * host_expert_counts) {
	select_experts_any(total_tokens, n_experts, top_k, NULL, X_routed, token_expert_weights, chosen_experts,
					   expert_counts, expert_counts_cumsum, host_expert_counts);
}

/* ---------------------------------------------------------------- build_expert_mapping */

void oracle_build_expert_mapping(int num_tokens, int num_routed_experts, int num_selected_experts,
								 const uint16_t * chosen_experts, int * expert_counts_cumsum,
								 int * expert_mapping, int * token_mapping) {
	/* build_expert_mapping.cu:63-67 takes write positions with atomicAdd on the running offsets; walking
	 * (token, slot) in ascending order makes that a stable counting sort and leaves the inclusive sum behind. */
	(void) num_routed_experts;
	for (int t = 0; t < num_tokens; t++) {
		for (int k = 0; k < num_selected_experts; k++) {
			uint16_t e = chosen_experts[(size_t) t * num_selected_experts + k];
			int pos = expert_counts_cumsum[e]++;
			expert_mapping[pos] = t;
			token_mapping[(size_t) t * num_selected_experts + k] = pos;
		}
	}
}

/* ---------------------------------------------------------------- dispatch */

void oracle_prepare_experts(int total_tokens, int model_dim, int num_selected_experts,
							const uint16_t * X, const int * token_mapping, uint16_t * expert_zones) {
	#pragma omp parallel for schedule(static)
	for (int t = 0; t < total_tokens; t++) {
		for (int k = 0; k < num_selected_experts; k++) {
			int row = token_mapping[(size_t) t * num_selected_experts + k];
			memcpy(expert_zones + (size_t) row * model_dim, X + (size_t) t * model_dim, (size_t) model_dim * sizeof(uint16_t));
		}
	}
}

void oracle_prepare_expert_zone(int model_dim, const uint16_t * X, int expert_id, const int * expert_counts,
								const int * expert_counts_cumsum, const int * expert_mapping, uint16_t * expert_zone) {
	int n = expert_counts[expert_id];
	int base = expert_counts_cumsum[expert_id] - n;      /* prepare_expert_zone.cu:46 */
	for (int r = 0; r < n; r++) {
		int t = expert_mapping[base + r];
		memcpy(expert_zone + (size_t) r * model_dim, X + (size_t) t * model_dim, (size_t) model_dim * sizeof(uint16_t));
	}
}

/* ---------------------------------------------------------------- swiglu */

void oracle_swiglu(int num_rows, int num_cols, const uint16_t * x_w1, const uint16_t * x_w3, uint16_t * out) {
	size_t n = (size_t) num_rows * (size_t) num_cols;
	#pragma omp parallel for schedule(static)
	for (size_t i = 0; i < n; i++) {
		float a = BF(x_w1[i]);
		float b = BF(x_w3[i]);
		float silu = a / (1.0f + expf(-a));          /* swiglu.cu:117 */
		out[i] = TOBF(silu * b);                     /* :126, :134 */
	}
}

void oracle_swiglu_bwd_x(int num_rows, int num_cols, const uint16_t * x_w1, const uint16_t * x_w3,
						 const uint16_t * upstream_dX, uint16_t * dX_w1, uint16_t * dX_w3) {
	size_t n = (size_t) num_rows * (size_t) num_cols;
	#pragma omp parallel for schedule(static)
	for (size_t i = 0; i < n; i++) {
		float a = BF(x_w1[i]);
		float b = BF(x_w3[i]);
		float g = BF(upstream_dX[i]);
		float s = 1.0f / (1.0f + expf(-a));          /* swiglu_bwd_x.cu:167-176 */
		float silu = a * s;                          /* :185 */
		float d3 = g * silu;                         /* :195 */
		float ds = s * (1.0f - s);                   /* :205 */
		float dsilu = s + a * ds;                    /* :214 */
		float d1 = g * b * dsilu;                    /* :223 */
		dX_w1[i] = TOBF(d1);
		dX_w3[i] = TOBF(d3);
	}
}

/* ---- fp32 and fp16 elements (swiglu.cu:4-64, swiglu_bwd_x.cu:4-109): the same expressions, one rounding to the element type ---- */

float oracle_fp16_to_f32(uint16_t h) {
	uint32_t sign = ((uint32_t) h & 0x8000u) << 16, exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
	if (exp == 0) {
		if (man == 0) {
			bits = sign;
		} else {                                     /* subnormal: man * 2^-24 */
			float f = (float) man * 5.9604644775390625e-08f;
			memcpy(&bits, &f, 4);
			bits |= sign;
		}
	} else if (exp == 31) {
		bits = sign | 0x7F800000u | (man << 13);
	} else {
		bits = sign | ((exp + 112u) << 23) | (man << 13);
	}
	float out;
	memcpy(&out, &bits, 4);
	return out;
}

/* round to nearest even, as __float2half */
uint16_t oracle_f32_to_fp16(float f) {
	uint32_t bits;
	memcpy(&bits, &f, 4);
	uint16_t sign = (uint16_t) ((bits >> 16) & 0x8000u);
	uint32_t mag = bits & 0x7FFFFFFFu;
	if (mag > 0x7F800000u) {
		return (uint16_t) (sign | 0x7E00u);          /* NaN */
	}
	if (mag >= 0x47800000u) {                        /* >= 65536: overflows (65520 and up round to inf below) */
		return (uint16_t) (sign | 0x7C00u);
	}
	if (mag < 0x33000000u) {                         /* < 2^-25: rounds to zero */
		return sign;
	}
	int exp = (int) (mag >> 23) - 127;
	uint32_t man = (mag & 0x7FFFFFu) | 0x800000u;    /* 24 bits */
	int shift = exp >= -14 ? 13 : 13 + (-14 - exp);  /* bits dropped: normal / subnormal result */
	uint32_t kept = man >> shift, rest = man & ((1u << shift) - 1u), half = 1u << (shift - 1);
	if (rest > half || (rest == half && (kept & 1u))) {
		kept++;
	}
	uint32_t out = exp >= -14 ? (((uint32_t) (exp + 15) << 10) + (kept - 0x400u)) : kept;   /* a carry runs into the exponent */
	return (uint16_t) (sign | out);
}

static inline float elem_get(int fp16, const void * p, size_t i) {
	return fp16 ? oracle_fp16_to_f32(((const uint16_t *) p)[i]) : ((const float *) p)[i];
}
static inline void elem_put(int fp16, void * p, size_t i, float v) {
	if (fp16) {
		((uint16_t *) p)[i] = oracle_f32_to_fp16(v);
	} else {
		((float *) p)[i] = v;
	}
}

void oracle_swiglu_typed(int fp16, int num_rows, int num_cols, const void * x_w1, const void * x_w3, void * out) {
	size_t n = (size_t) num_rows * (size_t) num_cols;
	for (size_t i = 0; i < n; i++) {
		float a = elem_get(fp16, x_w1, i), b = elem_get(fp16, x_w3, i);
		float silu = a / (1 + expf(-1 * a));         /* swiglu.cu:18 / :40 */
		elem_put(fp16, out, i, silu * b);            /* :21 / :43 */
	}
}

void oracle_swiglu_bwd_x_typed(int fp16, int num_rows, int num_cols, const void * x_w1, const void * x_w3,
							   const void * upstream_dX, void * dX_w1, void * dX_w3) {
	size_t n = (size_t) num_rows * (size_t) num_cols;
	for (size_t i = 0; i < n; i++) {
		float a = elem_get(fp16, x_w1, i), b = elem_get(fp16, x_w3, i), g = elem_get(fp16, upstream_dX, i);
		float s = 1.0f / (1.0f + expf(-a));          /* swiglu_bwd_x.cu:25-26 / :69-70 */
		float silu = a * s;                          /* :27 */
		float d3 = g * silu;                         /* :31 */
		float ds = s * (1.0f - s);                   /* :39 */
		float dsilu = s + a * ds;                    /* :40 */
		float d1 = g * b * dsilu;                    /* :43 */
		elem_put(fp16, dX_w1, i, d1);
		elem_put(fp16, dX_w3, i, d3);
	}
}

/* element kinds of oracle_matmul_typed */
static inline double kind_get(int kind, const void * p, size_t i) {
	switch (kind) {
		case ORACLE_ELEM_FP32: return (double) ((const float *) p)[i];
		case ORACLE_ELEM_FP16: return (double) oracle_fp16_to_f32(((const uint16_t *) p)[i]);
		default: return (double) bf_to_f(((const uint16_t *) p)[i]);
	}
}

int oracle_matmul_typed(int ab_kind, int cd_kind, int transa, int transb, int M, int K, int N, float alpha, float beta,
						const void * A, const void * B, const void * C, void * D) {
	if (ab_kind < ORACLE_ELEM_FP32 || ab_kind > ORACLE_ELEM_BF16 || cd_kind < ORACLE_ELEM_FP32 || cd_kind > ORACLE_ELEM_BF16) {
		return -1;
	}
	int use_c = (C != NULL) && (beta != 0.0f);
	/* same layouts as oracle_matmul (matmul_helper.c:345-425) */
	#pragma omp parallel for schedule(static)
	for (int n = 0; n < N; n++) {
		for (int m = 0; m < M; m++) {
			double acc = 0.0;
			for (int k = 0; k < K; k++) {
				double a = kind_get(ab_kind, A, transa ? (size_t) m * K + k : (size_t) k * M + m);
				double b = kind_get(ab_kind, B, transb ? (size_t) k * N + n : (size_t) n * K + k);
				acc += a * b;
			}
			size_t off = (size_t) n * M + m;
			double r = (double) alpha * acc;
			if (use_c) {
				r += (double) beta * kind_get(cd_kind, C, off);
			}
			switch (cd_kind) {
				case ORACLE_ELEM_FP32: ((float *) D)[off] = (float) r; break;
				case ORACLE_ELEM_FP16: ((uint16_t *) D)[off] = oracle_f32_to_fp16((float) r); break;
				default: ((uint16_t *) D)[off] = f_to_bf((float) r); break;
			}
		}
	}
	return 0;
}

/* ---------------------------------------------------------------- combine */

void oracle_merge_experts(int total_tokens, int model_dim, int num_selected_experts,
						  const uint16_t * expert_zones, const int * token_mapping,
						  const float * token_expert_weights, uint16_t * X_combined) {
	#pragma omp parallel for schedule(static)
	for (int t = 0; t < total_tokens; t++) {
		uint16_t * home = X_combined + (size_t) t * model_dim;
		for (int i = 0; i < model_dim; i++) {
			float acc = BF(home[i]);                                                 /* merge_expert_result.cu:140-163 */
			for (int k = 0; k < num_selected_experts; k++) {                         /* :178 slot order */
				int row = token_mapping[(size_t) t * num_selected_experts + k];
				float w = token_expert_weights ? token_expert_weights[(size_t) t * num_selected_experts + k] : 1.0f;
				float v = BF(expert_zones[(size_t) row * model_dim + i]);
				if (w != 1.0f) {
					acc = fmaf(w, v, acc);                                           /* :197-205 (a += w*v contracts to one fma) */
				} else {
					acc += v;                                                        /* :207-215 */
				}
			}
			home[i] = TOBF(acc);                                                     /* :240-243 */
		}
	}
}

void oracle_merge_expert_result(int num_tokens, int model_dim, int top_k_experts, const uint16_t * expert_zone,
								int expert_id, const int * expert_counts_cumsum, const int * expert_mapping,
								const float * token_expert_weights, const uint16_t * chosen_experts,
								uint16_t * X_combined) {
	int base = expert_counts_cumsum[expert_id] - num_tokens;                          /* merge_expert_result.cu:11 */
	for (int r = 0; r < num_tokens; r++) {
		int t = expert_mapping[base + r];
		float w = 1.0f;
		if (token_expert_weights) {
			w = 0.0f;
			for (int k = 0; k < top_k_experts; k++) {
				if (chosen_experts[(size_t) t * top_k_experts + k] == (uint16_t) expert_id) {
					w = token_expert_weights[(size_t) t * top_k_experts + k];
					break;
				}
			}
		}
		if (w == 0.0f) {
			continue;                                                                 /* :49-54 */
		}
		for (int i = 0; i < model_dim; i++) {
			float home = BF(X_combined[(size_t) t * model_dim + i]);
			float v = BF(expert_zone[(size_t) r * model_dim + i]);
			X_combined[(size_t) t * model_dim + i] = TOBF(fmaf(w, v, home));          /* :89-96, :99-102 */
		}
	}
}

/* ---------------------------------------------------------------- router backward */

void oracle_router_bwd_x(int num_expert_tokens, int model_dim, int num_routed_experts, int top_k_active,
						 int expert_id, const int * expert_counts_cumsum, const int * expert_mapping,
						 const uint16_t * chosen_experts, const float * token_expert_weights,
						 const uint16_t * expert_out, const uint16_t * upstream_dX,
						 uint16_t * dX_routed, uint16_t * dX_expert_out) {
	int base = expert_counts_cumsum[expert_id] - num_expert_tokens;                   /* router_bwd_x.cu:24 */
	#pragma omp parallel for schedule(static)
	for (int r = 0; r < num_expert_tokens; r++) {
		int t = expert_mapping[base + r];
		const uint16_t * y = expert_out + (size_t) r * model_dim;
		const uint16_t * g = upstream_dX + (size_t) t * model_dim;
		double acc = dot_bf16(y, 1, g, 1, model_dim);                                 /* :43-47 */
		dX_routed[(size_t) t * num_routed_experts + expert_id] = TOBF((float) acc);   /* :64 */
		float w = 0.0f;
		for (int k = 0; k < top_k_active; k++) {                                      /* :69-74 */
			if (chosen_experts[(size_t) t * top_k_active + k] == (uint16_t) expert_id) {
				w = token_expert_weights[(size_t) t * top_k_active + k];
				break;
			}
		}
		if (w != 0.0f) {
			float wb = BF(TOBF(w));                                                   /* :82 weight rounded to bf16 */
			uint16_t * o = dX_expert_out + (size_t) r * model_dim;
			for (int i = 0; i < model_dim; i++) {
				o[i] = TOBF(BF(g[i]) * wb);                                           /* :85 bf16 product, one rounding */
			}
		}
	}
}

void oracle_router_gate_bwd_x(int num_tokens, int num_routed_experts, int top_k_active,
							  const uint16_t * chosen_experts, const float * token_expert_weights,
							  uint16_t * dX_routed) {
	for (int t = 0; t < num_tokens; t++) {
		uint16_t * d = dX_routed + (size_t) t * num_routed_experts;
		const uint16_t * c = chosen_experts + (size_t) t * top_k_active;
		const float * p = token_expert_weights + (size_t) t * top_k_active;
		float m = 0.0f;
		for (int k = 0; k < top_k_active; k++) {                                      /* router_gate_bwd_x.cu:30-33 */
			m += BF(d[c[k]]) * p[k];
		}
		for (int k = 0; k < top_k_active; k++) {                                      /* :49-52 */
			d[c[k]] = TOBF(p[k] * (BF(d[c[k]]) - m));
		}
	}
}

/* ---------------------------------------------------------------- the layer */

int oracle_moe_forward(Oracle_Moe_Layer * L, const uint16_t * X, const uint16_t * logit_bias, uint16_t * out) {
	int T = L->T, D = L->D, E = L->E, K = L->K, H = L->H;

	/* dataflow_transformer.c:2710-2717 router logits, bf16 out */
	if (!L->logits_given) {
		oracle_matmul(1, 0, E, D, T, 1.0f, logit_bias ? 1.0f : 0.0f, L->Wr, X, logit_bias, L->logits);
	}

	/* :2737-2747 */
	memset(L->counts, 0, sizeof(int) * (size_t) (E + 1));
	memset(L->cumsum, 0, sizeof(int) * (size_t) E);
	/* :2751-2757, :2781-2784 */
	oracle_select_experts(T, E, K, L->logits, L->weights, L->chosen, L->counts, L->cumsum, NULL);
	oracle_build_expert_mapping(T, E, K, L->chosen, L->cumsum, L->expert_mapping, L->token_mapping);

	long total = 0;
	for (int e = 0; e < E; e++) {
		total += L->counts[e];
	}
	if (total != (long) T * K) {                                                      /* :2797-2800 */
		fprintf(stderr, "oracle: routed rows %ld != %ld\n", total, (long) T * K);
		return -1;
	}

	/* :2804-2808 */
	oracle_prepare_experts(T, D, K, X, L->token_mapping, L->zones);

	/* :2848-2940 */
	size_t row = 0;
	for (int e = 0; e < E; e++) {
		int n = L->counts[e];
		if (n == 0) {
			continue;
		}
		uint16_t * zone = L->zones + row * D;
		uint16_t * x1 = L->x1 + row * H;
		uint16_t * x3 = L->x3 + row * H;
		oracle_matmul(1, 0, H, D, n, 1.0f, 0.0f, L->W1 + (size_t) e * L->w_stride, zone, NULL, x1);
		oracle_matmul(1, 0, H, D, n, 1.0f, 0.0f, L->W3 + (size_t) e * L->w_stride, zone, NULL, x3);
		oracle_swiglu(n, H, x1, x3, L->temp);
		oracle_matmul(1, 0, D, H, n, 1.0f, 0.0f, L->W2 + (size_t) e * L->w_stride, L->temp, NULL, zone);
		row += (size_t) n;
	}

	/* :2964-2970 */
	oracle_merge_experts(T, D, K, L->zones, L->token_mapping, L->weights, out);
	return 0;
}

int oracle_moe_backward(Oracle_Moe_Layer * L, const uint16_t * X, const uint16_t * dY, uint16_t * dX) {
	int T = L->T, D = L->D, E = L->E, K = L->K, H = L->H;

	/* bwd_x: dataflow_transformer.c:3399 */
	memset(L->dlogits, 0, sizeof(uint16_t) * (size_t) T * E);

	size_t row = 0;
	for (int e = 0; e < E; e++) {                                                     /* :3460-3641 */
		int n = L->counts[e];
		if (n == 0) {
			continue;
		}
		uint16_t * zone = L->zones + row * D;
		const uint16_t * x1 = L->x1 + row * H;
		const uint16_t * x3 = L->x3 + row * H;
		uint16_t * dx1 = L->dx1 + row * H;
		uint16_t * dx3 = L->dx3 + row * H;
		const uint16_t * W1 = L->W1 + (size_t) e * L->w_stride;
		const uint16_t * W3 = L->W3 + (size_t) e * L->w_stride;
		const uint16_t * W2 = L->W2 + (size_t) e * L->w_stride;
		uint16_t * dW2 = L->dW2 + (size_t) e * L->w_stride;

		oracle_swiglu(n, H, x1, x3, L->temp);                                         /* :3494-3497 */
		oracle_matmul(1, 0, D, H, n, 1.0f, 0.0f, W2, L->temp, NULL, zone);            /* :3504-3511 */
		oracle_router_bwd_x(n, D, E, K, e, L->cumsum, L->expert_mapping, L->chosen, L->weights,
							zone, dY, L->dlogits, zone);                              /* :3525-3535 */
		oracle_matmul(0, 1, H, n, D, 1.0f, 1.0f, L->temp, zone, dW2, dW2);            /* :3548-3555 */
		oracle_matmul(0, 0, H, D, n, 1.0f, 0.0f, W2, zone, NULL, L->temp);            /* :3568-3575 */
		oracle_swiglu_bwd_x(n, H, x1, x3, L->temp, dx1, dx3);                         /* :3583-3588 */
		oracle_matmul(0, 0, D, H, n, 1.0f, 0.0f, W1, dx1, NULL, zone);                /* :3601-3608 */
		oracle_matmul(0, 0, D, H, n, 1.0f, 1.0f, W3, dx3, zone, zone);                /* :3614-3621 */
		row += (size_t) n;
	}

	memset(dX, 0, sizeof(uint16_t) * (size_t) T * D);                                 /* :3666 */
	oracle_merge_experts(T, D, K, L->zones, L->token_mapping, NULL, dX);              /* :3672-3678 */
	oracle_router_gate_bwd_x(T, E, K, L->chosen, L->weights, L->dlogits);             /* :3695-3700 */
	oracle_matmul(0, 0, D, E, T, 1.0f, 1.0f, L->Wr, L->dlogits, dX, dX);              /* :3707-3714 */

	/* bwd_w: :4062-4066 */
	oracle_prepare_experts(T, D, K, X, L->token_mapping, L->zones);
	row = 0;
	for (int e = 0; e < E; e++) {                                                     /* :4101-4148 */
		int n = L->counts[e];
		if (n == 0) {
			continue;
		}
		uint16_t * zone = L->zones + row * D;
		uint16_t * dW1 = L->dW1 + (size_t) e * L->w_stride;
		uint16_t * dW3 = L->dW3 + (size_t) e * L->w_stride;
		oracle_matmul(0, 1, D, n, H, 1.0f, 1.0f, zone, L->dx1 + row * H, dW1, dW1);
		oracle_matmul(0, 1, D, n, H, 1.0f, 1.0f, zone, L->dx3 + row * H, dW3, dW3);
		row += (size_t) n;
	}
	oracle_matmul(0, 1, D, T, E, 1.0f, 1.0f, X, L->dlogits, L->dWr, L->dWr);          /* :4174-4181 */
	return 0;
}

/* ---------------------------------------------------------------- RMS norm */

void oracle_rms_norm(int n_rows, int n_cols, float eps, const uint16_t * rms_weight, const uint16_t * X,
					 uint16_t * out, float * rms_vals) {
	#pragma omp parallel for
	for (int row = 0; row < n_rows; row++) {
		const uint16_t * x = X + (size_t) row * n_cols;
		double sq = 0.0;
		for (int i = 0; i < n_cols; i++) {
			float f = BF(x[i]);
			sq += (double) (f * f);                 /* a product of two bf16 values is exact in fp32 */
		}
		const float mean = (float) sq * (1.0f / (float) n_cols);   /* rms_norm.cu:298-299 */
		const float r = 1.0f / sqrtf(mean + eps);
		if (rms_vals) {
			rms_vals[row] = r;
		}
		for (int i = 0; i < n_cols; i++) {
			out[(size_t) row * n_cols + i] = TOBF((BF(x[i]) * r) * BF(rms_weight[i]));   /* :326-331 */
		}
	}
}

void oracle_rms_norm_recompute(int n_rows, int n_cols, const uint16_t * rms_weight, const float * rms_vals,
							   const uint16_t * X, uint16_t * out) {
	#pragma omp parallel for
	for (int row = 0; row < n_rows; row++) {
		const float r = rms_vals[row];
		for (int i = 0; i < n_cols; i++) {
			const size_t at = (size_t) row * n_cols + i;
			out[at] = TOBF((BF(X[at]) * r) * BF(rms_weight[i]));     /* rms_norm_recompute.cu:112-114 */
		}
	}
}

void oracle_rms_norm_bwd_x(int n_rows, int n_cols, float eps, const float * fwd_rms_vals, const uint16_t * rms_weight,
						   const uint16_t * X_inp, const uint16_t * upstream_dX, uint16_t * dX, uint16_t * X_out) {
	(void) eps;
	#pragma omp parallel for
	for (int row = 0; row < n_rows; row++) {
		const size_t base = (size_t) row * n_cols;
		const float r = fwd_rms_vals[row];
		double c = 0.0;
		for (int i = 0; i < n_cols; i++) {
			const float y = BF(X_inp[base + i]) * r * BF(rms_weight[i]);          /* rms_norm_bwd_x.cu:311-312 */
			if (X_out) {
				X_out[base + i] = TOBF(y);
			}
			c += (double) (y * BF(upstream_dX[base + i]));                        /* :315, the unrounded y */
		}
		const float c_div_n = (float) c / (float) n_cols;                         /* :344-345 */
		for (int i = 0; i < n_cols; i++) {
			const float x = BF(X_inp[base + i]);
			const float deriv = r * (BF(upstream_dX[base + i]) * BF(rms_weight[i]) - c_div_n * (x * r));   /* :369 */
			dX[base + i] = TOBF(BF(dX[base + i]) + deriv);                        /* :373-377 */
		}
	}
}

void oracle_rms_norm_bwd_w(int n_rows, int n_cols, float eps, const float * fwd_rms_vals, const uint16_t * X_inp,
						   const uint16_t * upstream_dX, uint16_t * dW) {
	(void) eps;
	#pragma omp parallel for
	for (int i = 0; i < n_cols; i++) {
		double s = 0.0;
		for (int row = 0; row < n_rows; row++) {
			const size_t at = (size_t) row * n_cols + i;
			s += (double) (BF(upstream_dX[at]) * BF(X_inp[at]) * fwd_rms_vals[row]);   /* rms_norm_bwd_w.cu:303-306 */
		}
		dW[i] = TOBF(BF(dW[i]) + (float) s);                                       /* rms_norm_bwd_w_combine.cu:213,288 */
	}
}

/* ---------------------------------------------------------------- AdamW */

void oracle_adamw_step(uint64_t num_els, int step_num, float lr, float beta1, float beta2, float weight_decay, float epsilon,
					   uint16_t * param, const uint16_t * grad, uint16_t * mean, uint16_t * var) {
	const float corr1 = 1.0f - powf(beta1, (float) step_num);                    /* adamw_step.cu:52-53 */
	const float corr2 = 1.0f - powf(beta2, (float) step_num);
	#pragma omp parallel for
	for (uint64_t i = 0; i < num_els; i++) {
		const float p = BF(param[i]), g = BF(grad[i]), m = BF(mean[i]), v = BF(var[i]);
		const float m_t = beta1 * m + (1.0f - beta1) * g;                        /* :45-46 */
		const float v_t = beta2 * v + (1.0f - beta2) * g * g;
		const float m_hat = m_t / corr1;
		const float v_hat = v_t / corr2;
		param[i] = TOBF(p - lr * (m_hat / (sqrtf(v_hat) + epsilon) + weight_decay * p));   /* :59-61 */
		mean[i] = TOBF(m_t);
		var[i] = TOBF(v_t);
	}
}

/* ---------------------------------------------------------------- casts */

void oracle_cast_bf16_fp32(uint64_t num_elements, const uint16_t * src, float * dst) {
	for (uint64_t i = 0; i < num_elements; i++) {
		dst[i] = BF(src[i]);                                                     /* cast.cu:31-45: exact */
	}
}

void oracle_cast_and_add(uint64_t num_elements, float alpha, const float * A, float beta, const uint16_t * B, uint16_t * C) {
	const float beta_bf16 = BF(TOBF(beta));                                      /* cast.cu:78-79 */
	for (uint64_t i = 0; i < num_elements; i++) {
		const float t1 = BF(TOBF(alpha * A[i]));                                 /* :90-92: fp32 product, __float22bfloat162_rn */
		const float t2 = BF(TOBF(beta_bf16 * BF(B[i])));                         /* :93 __hmul2: bf16 product, rounded */
		C[i] = TOBF(t1 + t2);                                                    /* :94 __hadd2: bf16 sum, rounded */
	}
}

