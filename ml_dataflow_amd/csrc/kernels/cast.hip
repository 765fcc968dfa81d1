/*
 * cast.hip -- the two conversion ops the reference registers beside the optimizer step.
 * Included by hip_kernels.hip after optimizer.hip.
 *
 *   default_cast_bf16_fp32              dst[i] = float(src[i])                      (cast.cu:11-47)
 *   default_cast_and_add_fp32_bf16_bf16 C[i] = bf16(alpha * A[i]) + bf16(beta) * B[i], the product and the sum each
 *                                       rounded to bf16 as the reference's bf16 intrinsics do (cast.cu:61-113): this is
 *                                       how an fp32 gradient is folded into a bf16 accumulator
 * Both are bandwidth-bound (6 and 8 bytes per element): grid-stride over 8-element vectors (16 bytes of bf16, two
 * 16-byte accesses of fp32) when the arrays are aligned for them, single elements otherwise and for the tail.
 */

typedef float f32x4_v __attribute__((ext_vector_type(4)));

/* Launch: grid = min(ceil(num_elements / 2048), 8192), block = 256. */
extern "C" __global__ void __launch_bounds__(256)
default_cast_bf16_fp32_kernel(uint64_t num_elements, const bf16_t * src, float * dst) {
	const uint64_t tid = (uint64_t) blockIdx.x * 256 + threadIdx.x;
	const uint64_t nthreads = (uint64_t) gridDim.x * 256;
	const bool aligned = ((((uintptr_t) src) | ((uintptr_t) dst)) & 15) == 0;
	const uint64_t nvec = aligned ? (num_elements >> 3) : 0;
	for (uint64_t i = tid; i < nvec; i += nthreads) {
		float f[8];
		unpack8(__builtin_nontemporal_load(((const u32x4 *) src) + i), f);
		((f32x4_v *) dst)[2 * i] = f32x4_v{f[0], f[1], f[2], f[3]};
		((f32x4_v *) dst)[2 * i + 1] = f32x4_v{f[4], f[5], f[6], f[7]};
	}
	for (uint64_t i = (nvec << 3) + tid; i < num_elements; i += nthreads) {
		dst[i] = bf16_to_f32(src[i]);
	}
}

/* one element: every intermediate is a bf16 value, as with the reference's __float2bfloat16_rn / __hmul2 / __hadd2 */
__device__ __forceinline__ float cast_and_add_element(float a, float b, float alpha, float beta_bf16) {
	const float t1 = bf16_to_f32(f32_to_bf16(alpha * a));
	const float t2 = bf16_to_f32(f32_to_bf16(beta_bf16 * b));       /* the product of two bf16 values is exact in fp32 */
	return t1 + t2;                                                 /* exact in fp32 wherever both terms matter; rounded by the caller */
}

/* Launch: as above.  C may alias B (the accumulate-in-place use). */
extern "C" __global__ void __launch_bounds__(256)
default_cast_and_add_fp32_bf16_bf16_kernel(int64_t num_elements, float alpha, const float * A, float beta, const bf16_t * B, bf16_t * C) {
	const float beta_bf16 = bf16_to_f32(f32_to_bf16(beta));
	const uint64_t n = num_elements > 0 ? (uint64_t) num_elements : 0;
	const uint64_t tid = (uint64_t) blockIdx.x * 256 + threadIdx.x;
	const uint64_t nthreads = (uint64_t) gridDim.x * 256;
	const bool aligned = ((((uintptr_t) A) | ((uintptr_t) B) | ((uintptr_t) C)) & 15) == 0;
	const uint64_t nvec = aligned ? (n >> 3) : 0;
	for (uint64_t i = tid; i < nvec; i += nthreads) {
		const f32x4_v a0 = __builtin_nontemporal_load(((const f32x4_v *) A) + 2 * i);
		const f32x4_v a1 = __builtin_nontemporal_load(((const f32x4_v *) A) + 2 * i + 1);
		const float a[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
		float b[8], c[8];
		unpack8(((const u32x4 *) B)[i], b);
		#pragma unroll
		for (int e = 0; e < 8; e++) {
			c[e] = cast_and_add_element(a[e], b[e], alpha, beta_bf16);
		}
		((u32x4 *) C)[i] = pack8(c);
	}
	for (uint64_t i = (nvec << 3) + tid; i < n; i += nthreads) {
		C[i] = f32_to_bf16(cast_and_add_element(A[i], bf16_to_f32(B[i]), alpha, beta_bf16));
	}
}
