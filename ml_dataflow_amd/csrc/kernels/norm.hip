/*
 * norm.hip -- RMS norm around the MoE layer: forward, forward from saved statistics, backward w.r.t. the
 * input and w.r.t. the scale (bf16 data, fp32 arithmetic).  Included by hip_kernels.hip after movement.hip.
 *
 * Semantics follow backends/nvidia/src/ops/src/native/src/norm/{rms_norm.cu:226-340, rms_norm_recompute.cu:63-135,
 * rms_norm_bwd_x.cu:241-393, rms_norm_bwd_w.cu:225-324, rms_norm_bwd_w_combine.cu:200-294}:
 *   r[row]   = rsqrt(mean(x^2) + eps)                    (saved in rms_vals: the reciprocal, not the rms)
 *   out      = bf16((x * r) * w)                          in this order of fp32 products
 *   bwd_x:   y = (x * r) * w (fp32, unrounded);  C = sum_i y_i * g_i;
 *            dX_i = bf16(float(dX_i) + r * (g_i * w_i - (C / n) * (x_i * r)));  X_out = bf16(y) if requested
 *   bwd_w:   dW_i = bf16(float(dW_i) + sum_rows g_i * x_i * r[row])   through per-work-group fp32 partial sums
 * Sums run over a row (or over rows) in fp32 in an order the reference leaves to its launch shape; results agree
 * within fp32 rounding of the sums.
 *
 * All kernels are bandwidth-bound: one 256-thread work-group per row, 16 bytes per lane per access, the row kept
 * in registers between the reduction and the second use (rows up to 8192 elements; longer rows are read twice).
 */

#define NORM_MAX_VEC 4

/* r[row], out = bf16((x * r) * w).  Launch: grid = n_rows, block = 256.
 * Algorithmic HBM bytes: 2*n_rows*n_cols read, 2*n_rows*n_cols + 4*n_rows written (w stays in cache). */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_rms_norm_bf16_kernel(int n_rows, int n_cols, float eps, const bf16_t * __restrict__ rms_weight,
							 const bf16_t * __restrict__ X, bf16_t * __restrict__ out, float * __restrict__ rms_vals) {
	__shared__ float scratch[ROW_WAVES];
	const int row = blockIdx.x;
	if (row >= n_rows) {
		return;
	}
	const int nvec = n_cols >> 3;
	const u32x4 * x = (const u32x4 *) (X + (size_t) row * n_cols);
	u32x4 * o = (u32x4 *) (out + (size_t) row * n_cols);
	const u32x4 * w = (const u32x4 *) rms_weight;

	u32x4 keep[NORM_MAX_VEC];
	float part[1] = {0.0f};
	int j = 0;
	for (int v = threadIdx.x; v < nvec; v += ROW_THREADS, j++) {
		const u32x4 q = x[v];
		if (j < NORM_MAX_VEC) {
			keep[j] = q;
		}
		float f[8];
		unpack8(q, f);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			part[0] = __builtin_fmaf(f[i], f[i], part[0]);
		}
	}
	block_sum<1>(part, scratch);
	const float r = rsqrtf(part[0] * (1.0f / (float) n_cols) + eps);
	if (threadIdx.x == 0 && rms_vals) {
		rms_vals[row] = r;
	}
	j = 0;
	for (int v = threadIdx.x; v < nvec; v += ROW_THREADS, j++) {
		float f[8], g[8], y[8];
		unpack8(j < NORM_MAX_VEC ? keep[j] : x[v], f);
		unpack8(w[v], g);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			y[i] = (f[i] * r) * g[i];
		}
		o[v] = pack8(y);
	}
}

/* out = bf16((x * r) * w) with r read from rms_vals.  Launch: grid = n_rows, block = 256. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_rms_norm_recompute_bf16_kernel(int n_rows, int n_cols, const bf16_t * __restrict__ rms_weight,
									   const float * __restrict__ rms_vals, const bf16_t * __restrict__ X, bf16_t * __restrict__ out) {
	const int row = blockIdx.x;
	if (row >= n_rows) {
		return;
	}
	const int nvec = n_cols >> 3;
	const float r = rms_vals[row];
	const u32x4 * x = (const u32x4 *) (X + (size_t) row * n_cols);
	u32x4 * o = (u32x4 *) (out + (size_t) row * n_cols);
	const u32x4 * w = (const u32x4 *) rms_weight;
	for (int v = threadIdx.x; v < nvec; v += ROW_THREADS) {
		float f[8], g[8], y[8];
		unpack8(x[v], f);
		unpack8(w[v], g);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			y[i] = (f[i] * r) * g[i];
		}
		o[v] = pack8(y);
	}
}

/* Backward w.r.t. the input, accumulated into dX; X_out (nullable) receives the recomputed forward output.
 * Launch: grid = n_rows, block = 256.
 * Algorithmic HBM bytes: 6*n_rows*n_cols read (x, g, dX), 2*n_rows*n_cols written (+2*n_rows*n_cols for X_out). */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_rms_norm_bwd_x_bf16_bf16_kernel(int n_rows, int n_cols, float eps, const float * __restrict__ fwd_rms_vals,
										const bf16_t * __restrict__ rms_weight, const bf16_t * __restrict__ X_inp,
										const bf16_t * __restrict__ upstream_dX, bf16_t * dX, bf16_t * X_out) {
	__shared__ float scratch[ROW_WAVES];
	(void) eps;
	const int row = blockIdx.x;
	if (row >= n_rows) {
		return;
	}
	const int nvec = n_cols >> 3;
	const float r = fwd_rms_vals[row];
	const u32x4 * x = (const u32x4 *) (X_inp + (size_t) row * n_cols);
	const u32x4 * g = (const u32x4 *) (upstream_dX + (size_t) row * n_cols);
	const u32x4 * w = (const u32x4 *) rms_weight;
	u32x4 * d = (u32x4 *) (dX + (size_t) row * n_cols);
	u32x4 * xo = X_out ? (u32x4 *) (X_out + (size_t) row * n_cols) : nullptr;

	u32x4 keep_x[NORM_MAX_VEC], keep_g[NORM_MAX_VEC];
	float part[1] = {0.0f};
	int j = 0;
	for (int v = threadIdx.x; v < nvec; v += ROW_THREADS, j++) {
		const u32x4 qx = x[v];
		const u32x4 qg = __builtin_nontemporal_load(g + v);
		if (j < NORM_MAX_VEC) {
			keep_x[j] = qx;
			keep_g[j] = qg;
		}
		float fx[8], fg[8], fw[8], y[8];
		unpack8(qx, fx);
		unpack8(qg, fg);
		unpack8(w[v], fw);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			y[i] = (fx[i] * r) * fw[i];
			part[0] = __builtin_fmaf(y[i], fg[i], part[0]);
		}
		if (xo) {
			xo[v] = pack8(y);
		}
	}
	block_sum<1>(part, scratch);
	const float c_div_n = part[0] / (float) n_cols;
	j = 0;
	for (int v = threadIdx.x; v < nvec; v += ROW_THREADS, j++) {
		float fx[8], fg[8], fw[8], fd[8];
		unpack8(j < NORM_MAX_VEC ? keep_x[j] : x[v], fx);
		unpack8(j < NORM_MAX_VEC ? keep_g[j] : g[v], fg);
		unpack8(w[v], fw);
		unpack8(d[v], fd);
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			fd[i] += r * (fg[i] * fw[i] - c_div_n * (fx[i] * r));
		}
		d[v] = pack8(fd);
	}
}

/* Backward w.r.t. the scale, first half: work-group b sums g * x * r over its share of the rows (a contiguous
 * range, as in the reference) into dW_workspace[b][n_cols] (fp32) and records the number of work-groups.
 * Launch: grid x <= n_rows (chosen so that the workspace holds grid.x * n_cols floats), grid y = column slabs of
 * 2048, block = 256: every thread owns 8 columns and walks down its work-group's rows with 16 loads in flight.
 * Algorithmic HBM bytes: 4*n_rows*n_cols read, 4*grid*n_cols written. */
extern "C" __global__ void __launch_bounds__(ROW_THREADS)
default_rms_norm_bwd_w_bf16_bf16_kernel(int n_rows, int n_cols, float eps, const float * __restrict__ fwd_rms_vals,
										const bf16_t * __restrict__ X_inp, const bf16_t * __restrict__ upstream_dX,
										float * __restrict__ dW_workspace, int * __restrict__ ret_num_blocks_launched) {
	(void) eps;
	if (blockIdx.x == 0 && threadIdx.x == 0) {
		*ret_num_blocks_launched = (int) gridDim.x;
	}
	const int b = blockIdx.x;
	int rows = n_rows / (int) gridDim.x;
	const int extra = n_rows % (int) gridDim.x;
	int first;
	if (b < extra) {
		rows += 1;
		first = b * rows;
	} else {
		first = b * rows + extra;
	}
	const int nvec = n_cols >> 3;
	typedef float f32x4 __attribute__((ext_vector_type(4)));
	const int v = blockIdx.y * ROW_THREADS + threadIdx.x;   /* one 8-column vector per thread, column slabs along grid y */
	if (v >= nvec) {
		return;
	}
	float acc[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
	#pragma unroll 8
	for (int i = 0; i < rows; i++) {
		const size_t off = (size_t) (first + i) * n_cols;
		const float r = fwd_rms_vals[first + i];
		float fx[8], fg[8];
		unpack8(__builtin_nontemporal_load(((const u32x4 *) (X_inp + off)) + v), fx);
		unpack8(__builtin_nontemporal_load(((const u32x4 *) (upstream_dX + off)) + v), fg);
		#pragma unroll
		for (int e = 0; e < 8; e++) {
			acc[e] += (fg[e] * fx[e]) * r;
		}
	}
	f32x4 * dst = (f32x4 *) (dW_workspace + (size_t) b * n_cols + (size_t) v * 8);
	dst[0] = f32x4{acc[0], acc[1], acc[2], acc[3]};
	dst[1] = f32x4{acc[4], acc[5], acc[6], acc[7]};
}

/* Second half: dW_i = bf16(float(dW_i) + sum over the recorded work-groups of dW_workspace[b][i]).
 * Launch: grid = ceil(model_dim / 64), block = 1024: a work-group owns 64 columns, each of its 16 waves sums a
 * sixteenth of the partial rows (lanes along the columns, so reads are contiguous; the loads of a wave are
 * independent of each other), then the waves are added.  The kernel is latency-bound: a few dependent rounds. */
#define COMBINE_WAVES 16
extern "C" __global__ void __launch_bounds__(COMBINE_WAVES * WAVE)
default_rms_norm_bwd_w_combine_bf16_kernel(const int * __restrict__ num_orig_blocks_launched, int model_dim,
										   const float * __restrict__ dW_workspace, bf16_t * dW) {
	__shared__ float partial[COMBINE_WAVES][WAVE];
	const int lane = threadIdx.x & (WAVE - 1);
	const int wave = threadIdx.x / WAVE;
	const int col = blockIdx.x * WAVE + lane;
	const int nb = *num_orig_blocks_launched;
	float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
	if (col < model_dim) {
		int b = wave;
		for (; b + 3 * COMBINE_WAVES < nb; b += 4 * COMBINE_WAVES) {
			s0 += dW_workspace[(size_t) b * model_dim + col];
			s1 += dW_workspace[(size_t) (b + COMBINE_WAVES) * model_dim + col];
			s2 += dW_workspace[(size_t) (b + 2 * COMBINE_WAVES) * model_dim + col];
			s3 += dW_workspace[(size_t) (b + 3 * COMBINE_WAVES) * model_dim + col];
		}
		for (; b < nb; b += COMBINE_WAVES) {
			s0 += dW_workspace[(size_t) b * model_dim + col];
		}
	}
	partial[wave][lane] = (s0 + s1) + (s2 + s3);
	__syncthreads();
	if (wave == 0 && col < model_dim) {
		float t = bf16_to_f32(dW[col]);
		#pragma unroll
		for (int w = 0; w < COMBINE_WAVES; w++) {
			t += partial[w][lane];
		}
		dW[col] = f32_to_bf16(t);
	}
}
