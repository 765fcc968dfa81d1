/*
 * moe_oracle.h -- CPU restatement of ml_dataflow's MoE-layer kernels.  TEST INFRASTRUCTURE ONLY.
 *
 * Nothing in the product (ml_dataflow_amd/, include/) may link, load or call this library; it is the
 * checker used by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py.
 *
 * Each function follows the CUDA kernel (or cuBLASLt call site) cited above it, one routed row / token
 * at a time, in plain scalar C.  All tensors are dense row-major; bf16 tensors are passed as uint16_t.
 *
 * Pinning status (what independent evidence each function is checked against in tests/test_oracle_*.py):
 *   select_experts        ids/slot order: closed-form cases (all-equal, increasing, decreasing, straddling ties)
 *                         and an independent (value desc, index asc) sort for the selected SET; weights: fp64
 *                         softmax over the selected logits; counts: numpy bincount; cumsum: numpy cumsum.
 *   build_expert_mapping  numpy stable argsort of the flattened ids (a library routine) + bijection invariants.
 *   prepare_experts / prepare_expert_zone   byte equality with numpy fancy indexing.
 *   matmul                numpy fp64 matmul of the bf16 inputs, one rounding; identity / one-hot special cases.
 *                         The reference computes this in closed-source cuBLASLt and holds no vectors for it:
 *                         PARITY UNPINNED against the reference itself, pinned against the mathematics only.
 *   matmul_typed          (fp32 / fp16 / bf16 operands, fp32 / fp16 results) the same: numpy's fp64 matmul and numpy's own
 *                         fp64 -> fp32 -> fp16 conversions must give the same bits, all four layouts, alpha / beta / C, identity.
 *   swiglu, swiglu_bwd_x  fp64 closed form; backward also by central differences.
 *   select_experts_fp32   brute-force (value desc, index asc) top-k for the set, an independent replay of the slot walk
 *                         for the order, numpy bincount / cumsum, fp64 softmax to fp32 accuracy, and a case whose
 *                         difference bf16 would round.
 *   fp16 <-> f32          numpy float16: all 65536 patterns one way; random values, every tie between neighbouring
 *                         halves, the overflow threshold and the subnormals the other way.
 *   swiglu_typed, swiglu_bwd_x_typed (fp32, fp16)   fp64 closed form and central differences; the fp16 result equals
 *                         numpy's rounding of the fp32 result.
 *   merge_experts / merge_expert_result     dense one-hot matmul in fp64; w=NULL equals numpy add.at.
 *   router_bwd_x, router_gate_bwd_x, layer backward   central finite differences of <dY, MoE(X)> in an
 *                         independent fp64 numpy model with routing held fixed, plus analytic identities.
 *   rms_norm, rms_norm_recompute   fp64 closed form x / sqrt(mean(x^2) + eps) * w, one rounding; saved statistic against
 *                         numpy.  rms_norm_bwd_x: central finite differences of <g, norm(x)> in fp64 and the identity
 *                         <dX, x> = 0 for unit scale.  rms_norm_bwd_w: numpy fp64 column sums.
 *   adamw_step            fp64 closed form of the AdamW update (Loshchilov & Hutter) element by element; fixed points
 *                         (zero gradient and zero moments leave only the weight decay).
 *   cast, cast_and_add    numpy: the widening cast is exact; cast_and_add against numpy's own bf16 rounding of the three
 *                         steps computed in fp64, plus the cases alpha = 0, beta = 0 and beta = 1 with B = 0.
 * No golden vectors for this path exist in the reference (its MoE checks print diffs against a CUDA-only
 * PyTorch model), so every pin above is mathematical, not a reference-held fixture.
 */
#ifndef MOE_ORACLE_H
#define MOE_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

float oracle_bf16_to_f32(uint16_t v);
uint16_t oracle_f32_to_bf16(float f);   /* round to nearest even, NaN kept quiet */

/* D = alpha*op(A)*op(B) + beta*C in the column-major BLAS convention of the reference's matmul op
 * (backends/nvidia/src/ops/src/external/matmul_helper/src/matmul_helper.c:345-425 for the layouts,
 * :686-750 for argument decoding; libdataflowops/src/submit_ops/matmul_op.c:11-66 for the wrapper).
 * Row-major reading: A is [M][K] if transa else [K][M]; B is [K][N] if transb else [N][K]; C, D are [N][M].
 * bf16 in, fp64 accumulate, one rounding to bf16.  C may be NULL (or beta 0) and may alias D. */
void oracle_matmul(int transa, int transb, int M, int K, int N, float alpha, float beta,
				   const uint16_t * A, const uint16_t * B, const uint16_t * C, uint16_t * D);

/* backends/nvidia/src/ops/src/native/src/moe/select_experts.cu:302-594.
 * expert_counts has n_experts+1 entries and expert_counts_cumsum n_experts; both are ADDED INTO / written the
 * way the kernel does, so the caller zeroes them first (dataflow_transformer.c:2737-2747).
 * expert_counts[n_experts] is the kernel's block ticket; here it is incremented by one.
 * host_expert_counts may be NULL. */
void oracle_select_experts(int total_tokens, int n_experts, int top_k,
						   const uint16_t * X_routed, float * token_expert_weights, uint16_t * chosen_experts,
						   int * expert_counts, int * expert_counts_cumsum, int * host_expert_counts);
/* the same op on fp32 logits (select_experts.cu:3-295): same walk, the softmax's difference is not rounded */
void oracle_select_experts_fp32(int total_tokens, int n_experts, int top_k,
								const float * X_routed, float * token_expert_weights, uint16_t * chosen_experts,
								int * expert_counts, int * expert_counts_cumsum, int * host_expert_counts);

/* IEEE half <-> float, round to nearest even (what __half2float / __float2half do) */
float oracle_fp16_to_f32(uint16_t h);
uint16_t oracle_f32_to_fp16(float f);
/* swiglu / swiglu_bwd_x on fp32 (fp16 == 0) or fp16 (fp16 != 0: uint16_t bit patterns) elements
 * (swiglu.cu:4-64, swiglu_bwd_x.cu:4-109) */
void oracle_swiglu_typed(int fp16, int num_rows, int num_cols, const void * x_w1, const void * x_w3, void * out);
void oracle_swiglu_bwd_x_typed(int fp16, int num_rows, int num_cols, const void * x_w1, const void * x_w3,
							   const void * upstream_dX, void * dX_w1, void * dX_w3);

/* The matmul on the element types its reference accepts beside all-bf16 (matmul_helper.c:168-296, fp32 compute type):
 * A and B of kind ab_kind, C and D of kind cd_kind, layouts as oracle_matmul.  fp64 accumulate; the result goes through
 * fp32 once and is then rounded to the output kind (exact for fp32).  Returns -1 for an unknown kind. */
enum { ORACLE_ELEM_FP32 = 0, ORACLE_ELEM_FP16 = 1, ORACLE_ELEM_BF16 = 2 };
int oracle_matmul_typed(int ab_kind, int cd_kind, int transa, int transb, int M, int K, int N, float alpha, float beta,
						const void * A, const void * B, const void * C, void * D);

/* build_expert_mapping.cu:18-103, with the order inside an expert fixed to ascending token id (the kernel's
 * atomics leave it unspecified).  expert_counts_cumsum: exclusive on entry, inclusive on return. */
void oracle_build_expert_mapping(int num_tokens, int num_routed_experts, int num_selected_experts,
								 const uint16_t * chosen_experts, int * expert_counts_cumsum,
								 int * expert_mapping, int * token_mapping);

/* prepare_expert_zone.cu:69-117 */
void oracle_prepare_experts(int total_tokens, int model_dim, int num_selected_experts,
							const uint16_t * X, const int * token_mapping, uint16_t * expert_zones);

/* prepare_expert_zone.cu:28-67 (expert_counts_cumsum inclusive) */
void oracle_prepare_expert_zone(int model_dim, const uint16_t * X, int expert_id, const int * expert_counts,
								const int * expert_counts_cumsum, const int * expert_mapping, uint16_t * expert_zone);

/* backends/nvidia/src/ops/src/native/src/activations/swiglu.cu:66-151.  out may alias x_w1 or x_w3. */
void oracle_swiglu(int num_rows, int num_cols, const uint16_t * x_w1, const uint16_t * x_w3, uint16_t * out);

/* swiglu_bwd_x.cu:111-256 */
void oracle_swiglu_bwd_x(int num_rows, int num_cols, const uint16_t * x_w1, const uint16_t * x_w3,
						 const uint16_t * upstream_dX, uint16_t * dX_w1, uint16_t * dX_w3);

/* merge_expert_result.cu:118-247.  token_expert_weights may be NULL (weight 1). */
void oracle_merge_experts(int total_tokens, int model_dim, int num_selected_experts,
						  const uint16_t * expert_zones, const int * token_mapping,
						  const float * token_expert_weights, uint16_t * X_combined);

/* merge_expert_result.cu:3-115.  num_tokens = rows of this expert; cumsum inclusive. */
void oracle_merge_expert_result(int num_tokens, int model_dim, int top_k_experts, const uint16_t * expert_zone,
								int expert_id, const int * expert_counts_cumsum, const int * expert_mapping,
								const float * token_expert_weights, const uint16_t * chosen_experts,
								uint16_t * X_combined);

/* router_bwd_x.cu:4-92.  num_expert_tokens = rows of this expert; dX_expert_out may alias expert_out. */
void oracle_router_bwd_x(int num_expert_tokens, int model_dim, int num_routed_experts, int top_k_active,
						 int expert_id, const int * expert_counts_cumsum, const int * expert_mapping,
						 const uint16_t * chosen_experts, const float * token_expert_weights,
						 const uint16_t * expert_out, const uint16_t * upstream_dX,
						 uint16_t * dX_routed, uint16_t * dX_expert_out);

/* router_gate_bwd_x.cu:7-57 */
void oracle_router_gate_bwd_x(int num_tokens, int num_routed_experts, int top_k_active,
							  const uint16_t * chosen_experts, const float * token_expert_weights,
							  uint16_t * dX_routed);

/* ---- the layer: the op sequence of libdataflowmodels/src/transformer/src/dataflow_transformer.c ---- */

/* ---- RMS norm around the layer (backends/nvidia/src/ops/src/native/src/norm) ---- */

/* rms_norm.cu:226-340: rms_vals[row] = 1/sqrt(mean(x^2) + eps) (nullable), out = bf16((x * r) * w) */
void oracle_rms_norm(int n_rows, int n_cols, float eps, const uint16_t * rms_weight, const uint16_t * X,
					 uint16_t * out, float * rms_vals);
/* rms_norm_recompute.cu:63-135 */
void oracle_rms_norm_recompute(int n_rows, int n_cols, const uint16_t * rms_weight, const float * rms_vals,
							   const uint16_t * X, uint16_t * out);
/* rms_norm_bwd_x.cu:241-393: dX += r * (g * w - (C / n) * (x * r)), C = sum (x * r * w) * g; X_out nullable */
void oracle_rms_norm_bwd_x(int n_rows, int n_cols, float eps, const float * fwd_rms_vals, const uint16_t * rms_weight,
						   const uint16_t * X_inp, const uint16_t * upstream_dX, uint16_t * dX, uint16_t * X_out);
/* rms_norm_bwd_w.cu:225-324 + rms_norm_bwd_w_combine.cu:200-294: dW = bf16(float(dW) + sum_rows g * x * r) */
void oracle_rms_norm_bwd_w(int n_rows, int n_cols, float eps, const float * fwd_rms_vals, const uint16_t * X_inp,
						   const uint16_t * upstream_dX, uint16_t * dW);

/* adamw_step.cu:6-65, in place on param, mean, var (bf16), fp32 arithmetic, step_num >= 1 */
void oracle_adamw_step(uint64_t num_els, int step_num, float lr, float beta1, float beta2, float weight_decay, float epsilon,
					   uint16_t * param, const uint16_t * grad, uint16_t * mean, uint16_t * var);

/* cast.cu:11-47 and :61-113 (C may alias B) */
void oracle_cast_bf16_fp32(uint64_t num_elements, const uint16_t * src, float * dst);
void oracle_cast_and_add(uint64_t num_elements, float alpha, const float * A, float beta, const uint16_t * B, uint16_t * C);

typedef struct oracle_moe_layer {
	int T, D, E, K, H;
	/* non-zero: forward takes `logits` as given instead of computing the router product (lets a test replay the
	 * routing of another implementation's logits, which may differ from the fp64-accumulated ones by a rounding) */
	int logits_given;
	/* parameters (bf16). Expert e: W1 at W1 + e*w_stride elements ([H][D]), W3 likewise, W2 ([D][H]). */
	const uint16_t * Wr;              /* [E][D] */
	const uint16_t * W1;
	const uint16_t * W3;
	const uint16_t * W2;
	size_t w_stride;                  /* elements between consecutive experts of one matrix */
	/* saved forward activations */
	uint16_t * logits;                /* [T][E]; reused as the router-logit gradient in backward */
	float * weights;                  /* [T][K] */
	uint16_t * chosen;                /* [T][K] */
	int * counts;                     /* [E+1] */
	int * cumsum;                     /* [E] inclusive after forward */
	int * expert_mapping;             /* [T*K] */
	int * token_mapping;              /* [T][K] */
	uint16_t * x1;                    /* [T*K][H] */
	uint16_t * x3;                    /* [T*K][H] */
	/* workspaces */
	uint16_t * zones;                 /* [T*K][D] */
	uint16_t * temp;                  /* [max n_e][H] */
	/* backward outputs */
	uint16_t * dx1;                   /* [T*K][H] */
	uint16_t * dx3;                   /* [T*K][H] */
	uint16_t * dlogits;               /* [T][E] */
	uint16_t * dWr;                   /* [E][D], accumulated into */
	uint16_t * dW1;                   /* same layout/stride as W1, accumulated into */
	uint16_t * dW3;
	uint16_t * dW2;
} Oracle_Moe_Layer;

/* dataflow_transformer.c:2700-2986.  X is the (already normalised) layer input [T][D]; out [T][D] holds the
 * residual on entry and residual + MoE(X) on return.  logit_bias ([T][E] bf16, or NULL) is added to the
 * router product as the matmul's beta*C term (used only to build skewed-routing test workloads).
 * Returns 0, or -1 if the routed-row total is not T*K. */
int oracle_moe_forward(Oracle_Moe_Layer * L, const uint16_t * X, const uint16_t * logit_bias, uint16_t * out);

/* dataflow_transformer.c:3386-3719 (bwd_x) then :4013-4185 (bwd_w).  dY [T][D] is the upstream gradient,
 * X the same layer input as in forward; dX [T][D] receives the gradient w.r.t. X. */
int oracle_moe_backward(Oracle_Moe_Layer * L, const uint16_t * X, const uint16_t * dY, uint16_t * dX);

#ifdef __cplusplus
}
#endif

#endif
