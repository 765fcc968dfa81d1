/*
 * optimizer.hip -- AdamW step on bf16 parameters, gradients and moments (fp32 arithmetic).
 * Included by hip_kernels.hip after movement.hip.
 *
 * Semantics of backends/nvidia/src/ops/src/native/src/optimizer/adamw_step.cu:6-65, element by element:
 *   m = beta1 * mean + (1 - beta1) * g;        v = beta2 * var + (1 - beta2) * g * g
 *   m_hat = m / (1 - beta1^step);              v_hat = v / (1 - beta2^step)
 *   param = bf16(param - lr * (m_hat / (sqrt(v_hat) + eps) + weight_decay * param));  mean = bf16(m);  var = bf16(v)
 * Bandwidth-bound: 8 bytes read and 6 written per element.  Each lane handles 8 consecutive elements (16-byte
 * accesses) when the four arrays are 16-byte aligned, single elements otherwise and for the tail.
 */

__device__ __forceinline__ void adamw_element(float & p, float g, float & m, float & v, float lr, float beta1, float beta2,
											  float weight_decay, float epsilon, float corr1, float corr2) {
	const float m_t = beta1 * m + (1.0f - beta1) * g;
	const float v_t = beta2 * v + (1.0f - beta2) * g * g;
	const float m_hat = m_t / corr1;
	const float v_hat = v_t / corr2;
	p = p - lr * (m_hat / (sqrtf(v_hat) + epsilon) + weight_decay * p);
	m = m_t;
	v = v_t;
}

/* Launch: grid = min(ceil(num_els / 2048), 8192), block = 256, grid-stride over 8-element vectors. */
extern "C" __global__ void __launch_bounds__(256)
default_adamw_step_bf16_bf16_bf16_bf16_kernel(uint64_t num_els, int step_num, float lr, float beta1, float beta2, float weight_decay,
											  float epsilon, bf16_t * param, const bf16_t * grad, bf16_t * mean, bf16_t * var) {
	const float corr1 = 1.0f - powf(beta1, (float) step_num);
	const float corr2 = 1.0f - powf(beta2, (float) step_num);
	const uint64_t tid = (uint64_t) blockIdx.x * 256 + threadIdx.x;
	const uint64_t nthreads = (uint64_t) gridDim.x * 256;
	const bool aligned = ((((uintptr_t) param) | ((uintptr_t) grad) | ((uintptr_t) mean) | ((uintptr_t) var)) & 15) == 0;
	const uint64_t nvec = aligned ? (num_els >> 3) : 0;
	for (uint64_t i = tid; i < nvec; i += nthreads) {
		float p[8], g[8], m[8], v[8];
		unpack8(((const u32x4 *) param)[i], p);
		unpack8(__builtin_nontemporal_load(((const u32x4 *) grad) + i), g);
		unpack8(((const u32x4 *) mean)[i], m);
		unpack8(((const u32x4 *) var)[i], v);
		#pragma unroll
		for (int e = 0; e < 8; e++) {
			adamw_element(p[e], g[e], m[e], v[e], lr, beta1, beta2, weight_decay, epsilon, corr1, corr2);
		}
		((u32x4 *) param)[i] = pack8(p);
		((u32x4 *) mean)[i] = pack8(m);
		((u32x4 *) var)[i] = pack8(v);
	}
	for (uint64_t i = (nvec << 3) + tid; i < num_els; i += nthreads) {
		float p = bf16_to_f32(param[i]), m = bf16_to_f32(mean[i]), v = bf16_to_f32(var[i]);
		adamw_element(p, bf16_to_f32(grad[i]), m, v, lr, beta1, beta2, weight_decay, epsilon, corr1, corr2);
		param[i] = f32_to_bf16(p);
		mean[i] = f32_to_bf16(m);
		var[i] = f32_to_bf16(v);
	}
}
