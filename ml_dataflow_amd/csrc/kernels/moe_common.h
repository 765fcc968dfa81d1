/*
 * moe_common.h -- device helpers shared by the gfx950 MoE kernels (wave64 only).
 */
#ifndef MOE_COMMON_H
#define MOE_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

typedef uint16_t bf16_t;                                       /* raw bf16 bits */
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));    /* 16 bytes = 8 bf16 */

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
	return __uint_as_float(((uint32_t) v) << 16);
}

/* round to nearest even; NaN stays NaN */
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
	uint32_t bits = __float_as_uint(f);
	if ((bits & 0x7fffffffu) > 0x7f800000u) {
		return (bf16_t) ((bits >> 16) | 0x0040u);
	}
	bits += 0x7fffu + ((bits >> 16) & 1u);
	return (bf16_t) (bits >> 16);
}

/* low / high half of a packed pair as float */
__device__ __forceinline__ float lo_f32(uint32_t pair) { return __uint_as_float(pair << 16); }
__device__ __forceinline__ float hi_f32(uint32_t pair) { return __uint_as_float(pair & 0xffff0000u); }
/* two fp32 -> packed pair of bf16, round to nearest even, one v_cvt_pk_bf16_f32 */
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
	const f32x2_t v = {lo, hi};
	return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

__device__ __forceinline__ void unpack8(const u32x4 & v, float f[8]) {
	f[0] = lo_f32(v.x); f[1] = hi_f32(v.x);
	f[2] = lo_f32(v.y); f[3] = hi_f32(v.y);
	f[4] = lo_f32(v.z); f[5] = hi_f32(v.z);
	f[6] = lo_f32(v.w); f[7] = hi_f32(v.w);
}

__device__ __forceinline__ u32x4 pack8(const float f[8]) {
	u32x4 v;
	v.x = pack_bf16(f[0], f[1]);
	v.y = pack_bf16(f[2], f[3]);
	v.z = pack_bf16(f[4], f[5]);
	v.w = pack_bf16(f[6], f[7]);
	return v;
}

/* sum over the 64 lanes of a wave; every lane gets the total */
__device__ __forceinline__ float wave_sum(float v) {
	#pragma unroll
	for (int off = 32; off > 0; off >>= 1) {
		v += __shfl_xor(v, off, WAVE);
	}
	return v;
}

__device__ __forceinline__ uint64_t lanemask_lt() {
	return (1ULL << (threadIdx.x & (WAVE - 1))) - 1ULL;
}

#endif
