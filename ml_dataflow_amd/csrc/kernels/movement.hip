/*
 * movement.hip -- the bandwidth-bound kernels of the MoE layer for gfx950: dispatch gather, weighted
 * combine, SwiGLU forward/backward and the router backward row kernels.
 *
 * Every kernel moves whole bf16 rows with 16-byte accesses (8 bf16 per lane per access, 1 KB per wave
 * instruction), keeps fp32 only in registers, and touches each HBM byte once.  Row lengths must be
 * multiples of 8 elements and row bases 16-byte aligned, as in the reference
 * (prepare_expert_zone.cu:82-83, swiglu.cu:68-70).
 */
#include "moe_common.h"

#define ROW_THREADS 256
#define ROW_WAVES (ROW_THREADS / WAVE)
#define MAX_VEC_PER_THREAD 4          /* rows up to 256*4*8 = 8192 elements stay in registers */

/* ------------------------------------------------------------------ dispatch */

/* expert_zones[token_mapping[t,k], :] = X[t, :]  (prepare_expert_zone.cu:69-117).
 * One work-group per token: the row is read once into registers and stored K times.
 * Algorithmic HBM bytes: 2*T*D read + 4*T*K read + 2*T*K*D written.
 * Launch: grid = T, block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_prepare_experts_bf16_bf16_kernel(int total_tokens, int model_dim, int num_selected_experts,
										 const bf16_t * __restrict__ X, const int * __restrict__ token_mapping,
										 bf16_t * __restrict__ expert_zones) {
	const int t = blockIdx.x;
	if (t >= total_tokens) {
		return;
	}
	const int nvec = model_dim >> 3;
	const u32x4 * src = (const u32x4 *) (X + (size_t) t * model_dim);
	const int * rows = token_mapping + (size_t) t * num_selected_experts;

	for (int v0 = 0; v0 < nvec; v0 += ROW_THREADS * MAX_VEC_PER_THREAD) {
		u32x4 r[MAX_VEC_PER_THREAD];
		#pragma unroll
		for (int j = 0; j < MAX_VEC_PER_THREAD; j++) {
			int v = v0 + j * ROW_THREADS + threadIdx.x;
			if (v < nvec) {
				r[j] = src[v];
			}
		}
		for (int k = 0; k < num_selected_experts; k++) {
			u32x4 * dst = (u32x4 *) (expert_zones + (size_t) rows[k] * model_dim);
			#pragma unroll
			for (int j = 0; j < MAX_VEC_PER_THREAD; j++) {
				int v = v0 + j * ROW_THREADS + threadIdx.x;
				if (v < nvec) {
					dst[v] = r[j];
				}
			}
		}
	}
}

/* Per-expert gather through expert_mapping (prepare_expert_zone.cu:28-67); expert_counts_cumsum inclusive.
 * Launch: grid = min(n_e, 65535) (the config reads nothing from the device: grid = a fixed number of
 * work-groups that stride over the rows), block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_prepare_expert_zone_bf16_bf16_kernel(int model_dim, const bf16_t * __restrict__ X, int expert_id,
											 const int * __restrict__ expert_counts, const int * __restrict__ expert_counts_cumsum,
											 const int * __restrict__ expert_mapping, bf16_t * __restrict__ expert_zone) {
	const int n = expert_counts[expert_id];
	const int base = expert_counts_cumsum[expert_id] - n;
	const int nvec = model_dim >> 3;
	for (int r = blockIdx.x; r < n; r += gridDim.x) {
		const int t = expert_mapping[base + r];
		const u32x4 * src = (const u32x4 *) (X + (size_t) t * model_dim);
		u32x4 * dst = (u32x4 *) (expert_zone + (size_t) r * model_dim);
		for (int v = threadIdx.x; v < nvec; v += ROW_THREADS) {
			dst[v] = src[v];
		}
	}
}

/* ------------------------------------------------------------------ combine */

#define MERGE_K 8

/* acc += w * row (fp32); a weight of exactly 1.0f adds without the multiply, as the reference does */
__device__ __forceinline__ void merge_add(float (&acc)[8], const u32x4 & row, float w) {
	float f[8];
	unpack8(row, f);
	if (w != 1.0f) {
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			acc[i] = __builtin_fmaf(w, f[i], acc[i]);
		}
	} else {
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			acc[i] += f[i];
		}
	}
}

/* One token's row of the combine: acc = FRESH ? 0 : float(X_combined[t,:]); acc += w[t,k] * float(expert_zones[
 * token_mapping[t,k],:]) for k ascending in fp32; one rounding. */
template <bool FRESH>
__device__ __forceinline__ void merge_experts_row(int t, int model_dim, int num_selected_experts,
												  const bf16_t * __restrict__ expert_zones, const int * __restrict__ token_mapping,
												  const float * __restrict__ token_expert_weights, bf16_t * X_combined) {
	const int nvec = model_dim >> 3;
	const int K = num_selected_experts;
	const int * rows = token_mapping + (size_t) t * K;
	const float * wts = token_expert_weights ? token_expert_weights + (size_t) t * K : nullptr;
	u32x4 * home = (u32x4 *) (X_combined + (size_t) t * model_dim);

	/* Two vectors of the row per lane and pass, and up to eight expert rows of each requested before the first of them
	 * is used: sixteen 16-byte gathers in flight per lane.  The additions stay in slot order. */
	for (int v0 = threadIdx.x; v0 < nvec; v0 += 2 * ROW_THREADS) {
		const int v1 = v0 + ROW_THREADS;
		const bool two = v1 < nvec;
		float acc0[8], acc1[8];
		if (FRESH) {
			#pragma unroll
			for (int i = 0; i < 8; i++) {
				acc0[i] = 0.0f;
				acc1[i] = 0.0f;
			}
		} else {
			unpack8(home[v0], acc0);
			if (two) {
				unpack8(home[v1], acc1);
			}
		}
		for (int k0 = 0; k0 < K; k0 += MERGE_K) {
			u32x4 q0[MERGE_K], q1[MERGE_K];
			float w[MERGE_K];
			#pragma unroll
			for (int j = 0; j < MERGE_K; j++) {
				if (k0 + j < K) {
					const u32x4 * src = (const u32x4 *) (expert_zones + (size_t) rows[k0 + j] * model_dim);
					q0[j] = __builtin_nontemporal_load(src + v0);
					if (two) {
						q1[j] = __builtin_nontemporal_load(src + v1);
					}
					w[j] = wts ? wts[k0 + j] : 1.0f;
				}
			}
			#pragma unroll
			for (int j = 0; j < MERGE_K; j++) {
				if (k0 + j < K) {
					merge_add(acc0, q0[j], w[j]);
					if (two) {
						merge_add(acc1, q1[j], w[j]);
					}
				}
			}
		}
		home[v0] = pack8(acc0);
		if (two) {
			home[v1] = pack8(acc1);
		}
	}
}

/* X_combined[t,:] = bf16( float(X_combined[t,:]) + sum_k w[t,k] * float(expert_zones[token_mapping[t,k],:]) ),
 * k ascending, fp32, one rounding (merge_expert_result.cu:118-247).  w == NULL, or a weight equal to 1.0f,
 * adds without the multiply exactly as the reference does.  Gather formulation: no atomics.
 * Algorithmic HBM bytes: 2*T*K*D + 2*T*D read, 8*T*K read, 2*T*D written.
 * Launch: grid = T, block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_merge_experts_bf16_bf16_kernel(int total_tokens, int model_dim, int num_selected_experts,
									   const bf16_t * __restrict__ expert_zones, const int * __restrict__ token_mapping,
									   const float * __restrict__ token_expert_weights, bf16_t * X_combined) {
	if ((int) blockIdx.x < total_tokens) {
		merge_experts_row<false>((int) blockIdx.x, model_dim, num_selected_experts, expert_zones, token_mapping, token_expert_weights, X_combined);
	}
}

/* The same sum into a row that counts as zero: what the reference gets by clearing X_combined before the combine
 * (dataflow_transformer.c:3666-3678), without the fill and without reading the zeros back.  The sum starts from
 * +0.0f like the cleared row's, so the result is that of fill + default_merge_experts bit for bit.
 * Algorithmic HBM bytes: 2*T*K*D + 8*T*K read, 2*T*D written.  Launch: grid = T, block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
amd_merge_experts_fresh_bf16_bf16_kernel(int total_tokens, int model_dim, int num_selected_experts,
										 const bf16_t * __restrict__ expert_zones, const int * __restrict__ token_mapping,
										 const float * __restrict__ token_expert_weights, bf16_t * X_combined) {
	if ((int) blockIdx.x < total_tokens) {
		merge_experts_row<true>((int) blockIdx.x, model_dim, num_selected_experts, expert_zones, token_mapping, token_expert_weights, X_combined);
	}
}

/* Per-expert read-modify-write combine (merge_expert_result.cu:3-115).  num_tokens = this expert's rows.
 * Launch: grid = num_tokens, block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_merge_expert_result_bf16_bf16_kernel(int num_tokens, int model_dim, int top_k_experts, const bf16_t * __restrict__ expert_zone,
											 int expert_id, const int * __restrict__ expert_counts_cumsum,
											 const int * __restrict__ expert_mapping, const float * __restrict__ token_expert_weights,
											 const uint16_t * __restrict__ chosen_experts, bf16_t * X_combined) {
	const int r = blockIdx.x;
	if (r >= num_tokens) {
		return;
	}
	const int base = expert_counts_cumsum[expert_id] - num_tokens;
	const int t = expert_mapping[base + r];
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
		return;
	}
	const int nvec = model_dim >> 3;
	const u32x4 * src = (const u32x4 *) (expert_zone + (size_t) r * model_dim);
	u32x4 * home = (u32x4 *) (X_combined + (size_t) t * model_dim);
	for (int v = threadIdx.x; v < nvec; v += ROW_THREADS) {
		float a[8], f[8];
		unpack8(home[v], a);
		unpack8(src[v], f);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			a[i] = __builtin_fmaf(w, f[i], a[i]);
		}
		home[v] = pack8(a);
	}
}

/* ------------------------------------------------------------------ SwiGLU */

__device__ __forceinline__ float sigmoid_f32(float x) {
	return 1.0f / (1.0f + __expf(-x));
}

/* out = bf16( x1 / (1 + exp(-x1)) * x3 ), fp32 math (swiglu.cu:66-151).  Flat over rows*cols; out may alias
 * an input because every lane reads its 8 elements before it writes them.
 * Algorithmic HBM bytes: 6 * rows * cols.   Launch: grid = ceil(rows*cols/8 / 256), block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_swiglu_bf16_kernel(int num_rows, int num_cols, const bf16_t * x_w1, const bf16_t * x_w3, bf16_t * out) {
	const size_t nvec = ((size_t) num_rows * (size_t) num_cols) >> 3;
	const size_t v = (size_t) blockIdx.x * ROW_THREADS + threadIdx.x;
	if (v >= nvec) {
		return;
	}
	float a[8], b[8], o[8];
	unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w1) + v), a);
	unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w3) + v), b);
	#pragma unroll
	for (int i = 0; i < 8; i++) {
		float silu = a[i] / (1.0f + __expf(-a[i]));
		o[i] = silu * b[i];
	}
	((u32x4 *) out)[v] = pack8(o);
}

/* dX3 = dOut * silu(x1);  dX1 = dOut * x3 * (s + x1 * s * (1 - s)),  s = sigmoid(x1)  (swiglu_bwd_x.cu:111-256).
 * Algorithmic HBM bytes: 10 * rows * cols.   Launch as above. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_swiglu_bwd_x_bf16_bf16_kernel(int num_rows, int num_cols, const bf16_t * x_w1, const bf16_t * x_w3,
									  const bf16_t * upstream_dX, bf16_t * dX_w1, bf16_t * dX_w3) {
	const size_t nvec = ((size_t) num_rows * (size_t) num_cols) >> 3;
	const size_t v = (size_t) blockIdx.x * ROW_THREADS + threadIdx.x;
	if (v >= nvec) {
		return;
	}
	float a[8], b[8], g[8], d1[8], d3[8];
	unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w1) + v), a);
	unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w3) + v), b);
	unpack8(__builtin_nontemporal_load(((const u32x4 *) upstream_dX) + v), g);
	#pragma unroll
	for (int i = 0; i < 8; i++) {
		float s = sigmoid_f32(a[i]);
		float silu = a[i] * s;
		d3[i] = g[i] * silu;
		float ds = s * (1.0f - s);
		float dsilu = s + a[i] * ds;
		d1[i] = g[i] * b[i] * dsilu;
	}
	((u32x4 *) dX_w1)[v] = pack8(d1);
	((u32x4 *) dX_w3)[v] = pack8(d3);
}

/* ---- SwiGLU for fp32 and fp16 elements (swiglu.cu:4-64, swiglu_bwd_x.cu:4-109): the reference's expressions in fp32,
 * one rounding to the element type at the end; same launch as the bf16 kernels (8 elements per lane, flat over
 * rows * cols, a multiple of 8). ---- */

typedef float f32x4_t __attribute__((ext_vector_type(4)));
template <typename T> struct Elem8;
template <> struct Elem8<float> {
	static __device__ __forceinline__ void load(const float * p, size_t v, float f[8]) {
		const f32x4_t lo = __builtin_nontemporal_load(((const f32x4_t *) p) + 2 * v), hi = __builtin_nontemporal_load(((const f32x4_t *) p) + 2 * v + 1);
		f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w; f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
	}
	static __device__ __forceinline__ void store(float * p, size_t v, const float f[8]) {
		((f32x4_t *) p)[2 * v] = f32x4_t{f[0], f[1], f[2], f[3]};
		((f32x4_t *) p)[2 * v + 1] = f32x4_t{f[4], f[5], f[6], f[7]};
	}
};
template <> struct Elem8<_Float16> {
	typedef _Float16 h8 __attribute__((ext_vector_type(8)));
	static __device__ __forceinline__ void load(const _Float16 * p, size_t v, float f[8]) {
		const h8 q = __builtin_nontemporal_load(((const h8 *) p) + v);
		#pragma unroll
		for (int i = 0; i < 8; i++) { f[i] = (float) q[i]; }
	}
	static __device__ __forceinline__ void store(_Float16 * p, size_t v, const float f[8]) {
		h8 q;
		#pragma unroll
		for (int i = 0; i < 8; i++) { q[i] = (_Float16) f[i]; }      /* round to nearest even, as __float2half */
		((h8 *) p)[v] = q;
	}
};

template <typename T>
__device__ __forceinline__ void swiglu_elems(int num_rows, int num_cols, const T * x_w1, const T * x_w3, T * out) {
	const size_t nvec = ((size_t) num_rows * (size_t) num_cols) >> 3;
	const size_t v = (size_t) blockIdx.x * ROW_THREADS + threadIdx.x;
	if (v >= nvec) {
		return;
	}
	float a[8], b[8], o[8];
	Elem8<T>::load(x_w1, v, a);
	Elem8<T>::load(x_w3, v, b);
	#pragma unroll
	for (int i = 0; i < 8; i++) {
		const float silu = a[i] / (1.0f + expf(-1.0f * a[i]));       /* swiglu.cu:18, :40 */
		o[i] = silu * b[i];
	}
	Elem8<T>::store(out, v, o);
}

template <typename T>
__device__ __forceinline__ void swiglu_bwd_x_elems(int num_rows, int num_cols, const T * x_w1, const T * x_w3, const T * upstream_dX, T * dX_w1, T * dX_w3) {
	const size_t nvec = ((size_t) num_rows * (size_t) num_cols) >> 3;
	const size_t v = (size_t) blockIdx.x * ROW_THREADS + threadIdx.x;
	if (v >= nvec) {
		return;
	}
	float a[8], b[8], g[8], d1[8], d3[8];
	Elem8<T>::load(x_w1, v, a);
	Elem8<T>::load(x_w3, v, b);
	Elem8<T>::load(upstream_dX, v, g);
	#pragma unroll
	for (int i = 0; i < 8; i++) {
		const float s = 1.0f / (1.0f + expf(-a[i]));                 /* swiglu_bwd_x.cu:25-26 */
		const float silu = a[i] * s;
		d3[i] = g[i] * silu;                                           /* :31 */
		const float ds = s * (1.0f - s);
		const float dsilu = s + a[i] * ds;                             /* :39-40 */
		d1[i] = g[i] * b[i] * dsilu;                                   /* :43 */
	}
	Elem8<T>::store(dX_w1, v, d1);
	Elem8<T>::store(dX_w3, v, d3);
}

extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_swiglu_fp32_kernel(int num_rows, int num_cols, const float * x_w1, const float * x_w3, float * out) {
	swiglu_elems<float>(num_rows, num_cols, x_w1, x_w3, out);
}
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_swiglu_fp16_kernel(int num_rows, int num_cols, const _Float16 * x_w1, const _Float16 * x_w3, _Float16 * out) {
	swiglu_elems<_Float16>(num_rows, num_cols, x_w1, x_w3, out);
}
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_swiglu_bwd_x_fp32_fp32_kernel(int num_rows, int num_cols, const float * x_w1, const float * x_w3, const float * upstream_dX, float * dX_w1, float * dX_w3) {
	swiglu_bwd_x_elems<float>(num_rows, num_cols, x_w1, x_w3, upstream_dX, dX_w1, dX_w3);
}
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_swiglu_bwd_x_fp16_fp16_kernel(int num_rows, int num_cols, const _Float16 * x_w1, const _Float16 * x_w3, const _Float16 * upstream_dX, _Float16 * dX_w1, _Float16 * dX_w3) {
	swiglu_bwd_x_elems<_Float16>(num_rows, num_cols, x_w1, x_w3, upstream_dX, dX_w1, dX_w3);
}

/* ------------------------------------------------------------------ router backward rows */

/* sum over a 256-thread work-group of `n` values per thread (n <= 8); result valid in every thread */
template <int N>
__device__ __forceinline__ void block_sum(float (&vals)[N], float * scratch /* [ROW_WAVES * N] */) {
	const int lane = threadIdx.x & (WAVE - 1);
	const int wave = threadIdx.x / WAVE;
	#pragma unroll
	for (int i = 0; i < N; i++) {
		vals[i] = wave_sum(vals[i]);
	}
	__syncthreads();
	if (lane == 0) {
		#pragma unroll
		for (int i = 0; i < N; i++) {
			scratch[wave * N + i] = vals[i];
		}
	}
	__syncthreads();
	#pragma unroll
	for (int i = 0; i < N; i++) {
		float s = 0.0f;
		#pragma unroll
		for (int w = 0; w < ROW_WAVES; w++) {
			s += scratch[w * N + i];
		}
		vals[i] = s;
	}
}

/* scale a packed pair of bf16 by a bf16 weight with one rounding per element: the fp32 product of two bf16
 * values is exact, so rounding it once equals the reference's __hmul2 (router_bwd_x.cu:83-86) */
__device__ __forceinline__ u32x4 scale8(const u32x4 & g, float wb) {
	float f[8];
	unpack8(g, f);
	#pragma unroll
	for (int i = 0; i < 8; i++) {
		f[i] *= wb;
	}
	return pack8(f);
}

/* One expert's rows (router_bwd_x.cu:4-92): for row r of expert e, t = expert_mapping[cumsum[e] - n_e + r]:
 *   dX_routed[t, e] = bf16( <expert_out[r,:], upstream_dX[t,:]> )         fp32 accumulation
 *   dX_expert_out[r,:] = upstream_dX[t,:] * bf16(w[t, slot of e])         bf16 product
 * dX_expert_out may alias expert_out: each lane overwrites only elements it has already read.
 * Launch: grid = n_e, block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_router_bwd_x_bf16_bf16_kernel(int num_expert_tokens, int model_dim, int num_routed_experts, int top_k_active,
									  int expert_id, const int * expert_counts_cumsum, const int * expert_mapping,
									  const uint16_t * chosen_experts, const float * token_expert_weights,
									  const bf16_t * expert_out, const bf16_t * upstream_dX,
									  bf16_t * dX_routed, bf16_t * dX_expert_out) {
	__shared__ float scratch[ROW_WAVES];
	const int r = blockIdx.x;
	if (r >= num_expert_tokens) {
		return;
	}
	const int base = expert_counts_cumsum[expert_id] - num_expert_tokens;
	const int t = expert_mapping[base + r];
	const int nvec = model_dim >> 3;
	const u32x4 * y = (const u32x4 *) (expert_out + (size_t) r * model_dim);
	const u32x4 * g = (const u32x4 *) (upstream_dX + (size_t) t * model_dim);

	float part[1] = {0.0f};
	for (int v = threadIdx.x; v < nvec; v += ROW_THREADS) {
		float a[8], b[8];
		unpack8(y[v], a);
		unpack8(g[v], b);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			part[0] = __builtin_fmaf(a[i], b[i], part[0]);
		}
	}
	block_sum<1>(part, scratch);
	if (threadIdx.x == 0) {
		dX_routed[(size_t) t * num_routed_experts + expert_id] = f32_to_bf16(part[0]);
	}
	float w = 0.0f;
	for (int k = 0; k < top_k_active; k++) {
		if (chosen_experts[(size_t) t * top_k_active + k] == (uint16_t) expert_id) {
			w = token_expert_weights[(size_t) t * top_k_active + k];
			break;
		}
	}
	if (w != 0.0f) {
		const float wb = bf16_to_f32(f32_to_bf16(w));
		u32x4 * o = (u32x4 *) (dX_expert_out + (size_t) r * model_dim);
		for (int v = threadIdx.x; v < nvec; v += ROW_THREADS) {
			o[v] = scale8(g[v], wb);
		}
	}
}

/* All experts in one launch, token-major (an addition; the reference launches the kernel above once per
 * expert).  For token t the gradient row dY[t,:] is read once and used for all K routed copies:
 *   r = token_mapping[t,k], e = chosen_experts[t,k]:
 *   dX_routed[t,e] = bf16(<expert_out[r,:], dY[t,:]>),  dX_expert_out[r,:] = dY[t,:] * bf16(w[t,k]).
 * Algorithmic HBM bytes: 2*T*D (dY) + 2*T*K*D (expert_out) + 2*T*K*D (written) + 10*T*K.
 * Launch: grid = T, block = 256, requires K <= 8 per pass (larger K loops). */
#define RBX_K 8
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
amd_router_bwd_x_all_bf16_bf16_kernel(int num_tokens, int model_dim, int num_routed_experts, int top_k_active,
									  const int * token_mapping, const uint16_t * chosen_experts,
									  const float * token_expert_weights,
									  const bf16_t * expert_out, const bf16_t * upstream_dX,
									  bf16_t * dX_routed, bf16_t * dX_expert_out) {
	__shared__ float scratch[ROW_WAVES * RBX_K];
	const int t = blockIdx.x;
	if (t >= num_tokens) {
		return;
	}
	const int nvec = model_dim >> 3;
	const u32x4 * g = (const u32x4 *) (upstream_dX + (size_t) t * model_dim);
	const int * rows = token_mapping + (size_t) t * top_k_active;
	const uint16_t * ids = chosen_experts + (size_t) t * top_k_active;
	const float * wts = token_expert_weights + (size_t) t * top_k_active;

	for (int k0 = 0; k0 < top_k_active; k0 += RBX_K) {
		const int kn = min(RBX_K, top_k_active - k0);
		float part[RBX_K];
		#pragma unroll
		for (int j = 0; j < RBX_K; j++) {
			part[j] = 0.0f;
		}
		for (int v = threadIdx.x; v < nvec; v += ROW_THREADS) {
			float b[8];
			unpack8(g[v], b);
			#pragma unroll
			for (int j = 0; j < RBX_K; j++) {
				if (j < kn) {
					float a[8];
					unpack8(__builtin_nontemporal_load(((const u32x4 *) (expert_out + (size_t) rows[k0 + j] * model_dim)) + v), a);
					#pragma unroll
					for (int i = 0; i < 8; i++) {
						part[j] = __builtin_fmaf(a[i], b[i], part[j]);
					}
				}
			}
		}
		block_sum<RBX_K>(part, scratch);
		if (threadIdx.x < kn) {
			int j = threadIdx.x;
			float s = 0.0f;
			#pragma unroll
			for (int jj = 0; jj < RBX_K; jj++) {
				if (jj == j) {
					s = part[jj];
				}
			}
			dX_routed[(size_t) t * num_routed_experts + ids[k0 + j]] = f32_to_bf16(s);
		}
		/* every lane has finished reading the expert_out rows it is about to overwrite (block_sum synchronises) */
		for (int v = threadIdx.x; v < nvec; v += ROW_THREADS) {
			u32x4 gv = g[v];
			#pragma unroll
			for (int j = 0; j < RBX_K; j++) {
				if (j < kn) {
					float w = wts[k0 + j];
					if (w != 0.0f) {
						((u32x4 *) (dX_expert_out + (size_t) rows[k0 + j] * model_dim))[v] = scale8(gv, bf16_to_f32(f32_to_bf16(w)));
					}
				}
			}
		}
		__syncthreads();
	}
}

/* ------------------------------------------------------------------ backward without the recompute (additions) */

/* expert_zones[token_mapping[t,k], :] = bf16(X[t, :] * bf16(w[t,k])): the dispatch gather above with the row scaled by
 * the slot's routing weight on the way, one bf16 rounding per element as in router_bwd_x.cu:83-86.  It produces the
 * w-scaled upstream rows of the backward pass directly from dY, without the expert outputs that router_bwd_x reads.
 * Algorithmic HBM bytes: 2*T*D + 8*T*K read, 2*T*K*D written.   Launch: grid = T, block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
amd_prepare_experts_scaled_bf16_bf16_kernel(int total_tokens, int model_dim, int num_selected_experts,
											const bf16_t * __restrict__ X, const int * __restrict__ token_mapping,
											const float * __restrict__ token_expert_weights, bf16_t * __restrict__ expert_zones) {
	const int t = blockIdx.x;
	if (t >= total_tokens) {
		return;
	}
	const int nvec = model_dim >> 3;
	const u32x4 * src = (const u32x4 *) (X + (size_t) t * model_dim);
	const int * rows = token_mapping + (size_t) t * num_selected_experts;
	const float * wts = token_expert_weights + (size_t) t * num_selected_experts;

	for (int v0 = 0; v0 < nvec; v0 += ROW_THREADS * MAX_VEC_PER_THREAD) {
		u32x4 r[MAX_VEC_PER_THREAD];
		#pragma unroll
		for (int j = 0; j < MAX_VEC_PER_THREAD; j++) {
			int v = v0 + j * ROW_THREADS + threadIdx.x;
			if (v < nvec) {
				r[j] = src[v];
			}
		}
		for (int k = 0; k < num_selected_experts; k++) {
			u32x4 * dst = (u32x4 *) (expert_zones + (size_t) rows[k] * model_dim);
			const float wb = bf16_to_f32(f32_to_bf16(wts[k]));
			#pragma unroll
			for (int j = 0; j < MAX_VEC_PER_THREAD; j++) {
				int v = v0 + j * ROW_THREADS + threadIdx.x;
				if (v < nvec) {
					dst[v] = scale8(r[j], wb);
				}
			}
		}
	}
}

/* default_swiglu for activations whose rows are not packed: row r of x_w1 / x_w3 starts x_row_stride elements after
 * row r-1 (x_row_stride >= num_cols, a multiple of 8); out is packed [num_rows][num_cols].  With x_w3 = x_w1 + num_cols
 * and x_row_stride = 2 * num_cols the two up-projections of a row lie side by side, which is how one GEMM over the
 * stacked w1 / w3 matrices writes them.  Same expressions as default_swiglu: same bits.
 * Launch: grid = ceil(rows*cols/8 / 256), block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
amd_swiglu_strided_bf16_kernel(int num_rows, int num_cols, int x_row_stride, const bf16_t * x_w1, const bf16_t * x_w3, bf16_t * out) {
	const int per_row = num_cols >> 3;
	const size_t nvec = (size_t) num_rows * (size_t) per_row;
	const size_t v = (size_t) blockIdx.x * ROW_THREADS + threadIdx.x;
	if (v >= nvec) {
		return;
	}
	const size_t r = v / (size_t) per_row;
	const size_t src = (r * (size_t) x_row_stride >> 3) + (v - r * (size_t) per_row);
	float a[8], b[8], o[8];
	unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w1) + src), a);
	unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w3) + src), b);
	#pragma unroll
	for (int i = 0; i < 8; i++) {
		float silu = a[i] / (1.0f + __expf(-a[i]));
		o[i] = silu * b[i];
	}
	((u32x4 *) out)[v] = pack8(o);
}

/* What remains of the expert-side backward between the hidden-gradient GEMM and the input-gradient GEMMs when the
 * expert outputs are not recomputed.  The reference recomputes y = h W2^T to form the router gradient <y_r, dY_t>
 * (dataflow_transformer.c:3494-3535, router_bwd_x.cu:52-66).  With g_r = wb * dY_t the w-scaled upstream row and
 * dh_r = g_r W2 the hidden gradient that the backward computes anyway,
 *     <y_r, dY_t> = <h_r W2^T, dY_t> = <h_r, dY_t W2> = <h_r, dh_r> / wb,
 * a dot product over the expert dimension.  For routed row r (token t = expert_mapping[r], slot k with
 * token_mapping[t,k] == r, expert e = chosen_experts[t,k], wb = bf16(w[t,k])):
 *     h_out[r,:]     = bf16(silu(x1[r,:]) * x3[r,:])                 the SwiGLU output, as swiglu.cu:66-151
 *     dX_routed[t,e] = bf16(<h_out[r,:], dh[r,:]> / wb)              fp32 accumulation; 0 where wb == 0 (the softmax
 *                                                                    gate backward multiplies it by that weight)
 *     dX_w3[r,:] = bf16(dh * silu(x1)),  dX_w1[r,:] = bf16(dh * x3 * (s + x1 s (1 - s)))      (swiglu_bwd_x.cu:111-256)
 * Rows of x1 / x3 start x_row_stride elements apart and rows of dX_w1 / dX_w3 dx_row_stride elements apart (multiples
 * of 8, >= num_cols; see amd_swiglu_strided above); dh and h_out are packed.  With dx_row_stride == num_cols dX_w1 may
 * alias dh: every lane reads its elements of dh before it writes them.
 * Algorithmic HBM bytes: 12 * rows * cols (three rows read, three written).
 * Launch: one wave per routed row, 4 rows per 256-thread work-group: grid = ceil(rows / 4). */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
amd_swiglu_bwd_x_routed_bf16_bf16_kernel(int num_rows, int num_cols, int num_routed_experts, int top_k_active,
										 int x_row_stride, int dx_row_stride,
										 const int * __restrict__ expert_mapping, const int * __restrict__ token_mapping,
										 const uint16_t * __restrict__ chosen_experts, const float * __restrict__ token_expert_weights,
										 const bf16_t * x_w1, const bf16_t * x_w3, const bf16_t * dh,
										 bf16_t * dX_routed, bf16_t * dX_w1, bf16_t * dX_w3, bf16_t * h_out) {
	const int lane = threadIdx.x & (WAVE - 1);
	const int r = blockIdx.x * ROW_WAVES + (threadIdx.x / WAVE);
	if (r >= num_rows) {
		return;
	}
	const int t = expert_mapping[r];
	/* the slot of this row: lanes 0..K-1 look at one slot each (K <= 64 is checked at submit) */
	const bool mine = lane < top_k_active && token_mapping[(size_t) t * top_k_active + lane] == r;
	const uint64_t found = __ballot(mine);
	int e = -1;
	float wb = 0.0f;
	if (found != 0) {                                  /* 0: mappings that do not belong together; no router gradient then */
		const int k = __ffsll((long long) found) - 1;
		e = chosen_experts[(size_t) t * top_k_active + k];
		wb = bf16_to_f32(f32_to_bf16(token_expert_weights[(size_t) t * top_k_active + k]));
	}

	const int nvec = num_cols >> 3;
	const size_t row = (size_t) r * (size_t) nvec;
	const size_t x_row = (size_t) r * (size_t) (x_row_stride >> 3);
	const size_t dx_row = (size_t) r * (size_t) (dx_row_stride >> 3);
	float dot = 0.0f;
	for (int v = lane; v < nvec; v += WAVE) {
		float a[8], b[8], g[8], d1[8], d3[8], h[8];
		unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w1) + x_row + v), a);
		unpack8(__builtin_nontemporal_load(((const u32x4 *) x_w3) + x_row + v), b);
		unpack8(__builtin_nontemporal_load(((const u32x4 *) dh) + row + v), g);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			/* the same expressions as default_swiglu / default_swiglu_bwd_x above, so that h, dX_w1 and dX_w3 come out
			 * bit for bit as from those kernels */
			const float s = sigmoid_f32(a[i]);
			const float silu_fwd = a[i] / (1.0f + __expf(-a[i]));
			h[i] = silu_fwd * b[i];
			const float silu = a[i] * s;
			d3[i] = g[i] * silu;
			const float ds = s * (1.0f - s);
			const float dsilu = s + a[i] * ds;
			d1[i] = g[i] * b[i] * dsilu;
		}
		const u32x4 hv = pack8(h);
		float hr[8];
		unpack8(hv, hr);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			dot = __builtin_fmaf(hr[i], g[i], dot);
		}
		((u32x4 *) dX_w1)[dx_row + v] = pack8(d1);
		((u32x4 *) dX_w3)[dx_row + v] = pack8(d3);
		((u32x4 *) h_out)[row + v] = hv;
	}
	dot = wave_sum(dot);
	if (lane == 0 && e >= 0) {
		dX_routed[(size_t) t * num_routed_experts + e] = f32_to_bf16(wb != 0.0f ? dot / wb : 0.0f);
	}
}
