/*
 * gemm_typed_kernel.h -- the matmul for the element types beside all-bf16 that the reference's matmul accepts with
 * fp32 accumulation (backends/nvidia/src/ops/src/external/matmul_helper/src/matmul_helper.c:168-296):
 *
 *     A, B fp32            C, D fp32
 *     A, B fp16            C, D fp16 or fp32
 *     A, B bf16            C, D fp32          (bf16 C, D is the gemm_kernel.h family)
 *
 * One kernel for any shape, layout and alignment: 128 x 128 output tiles, four waves with 64 x 64 wave tiles, operand
 * tiles fetched element by element into registers one k-tile ahead and multiplied out of LDS with
 * v_mfma_f32_16x16x4_f32 / v_mfma_f32_16x16x16_f16 / v_mfma_f32_16x16x16_bf16.  Products of 16-bit operands are exact
 * in fp32 and fp32 products are rounded once, as in an fp32 fused multiply-add; the sum over k is kept in fp32 and
 * rounded once to the output type after alpha and beta.  No configuration of the MoE layer uses these types, so the
 * kernel is written for correctness on every shape, not for the last third of the matrix pipe.
 *
 * Conventions as in gemm_kernel.h: P is the M-side operand, Q the N-side one, the output is [N][M] with m contiguous;
 * an operand is k-contiguous ([rows][K]) or k-major ([K][rows]).
 */
#ifndef GEMM_TYPED_KERNEL_H
#define GEMM_TYPED_KERNEL_H

#include "gemm_kernel.h"

typedef _Float16 f16x4_t __attribute__((ext_vector_type(4)));

struct TypedGemmParams {
	const void * P;
	const void * Q;
	const void * C;                /* NULL: no C operand */
	void * D;
	int M, N, K;
	int p_kmajor, q_kmajor;
	float alpha, beta;
};

/* per operand type: LDS element, how many consecutive k a lane feeds to one MFMA, and the MFMA itself */
template <typename E> struct TypedOperand;

template <> struct TypedOperand<float> {
	static constexpr int KPACK = 1;
	typedef float frag_t;
	static __device__ __forceinline__ float zero() { return 0.0f; }
	static __device__ __forceinline__ frag_t read(const float * s) { return *s; }
	static __device__ __forceinline__ f32x4_t mfma(frag_t a, frag_t b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
};

template <> struct TypedOperand<_Float16> {
	static constexpr int KPACK = 4;
	typedef f16x4_t frag_t;
	static __device__ __forceinline__ _Float16 zero() { return (_Float16) 0.0f; }
	static __device__ __forceinline__ frag_t read(const _Float16 * s) { return *((const f16x4_t *) s); }
	static __device__ __forceinline__ f32x4_t mfma(frag_t a, frag_t b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x16f16(a, b, c, 0, 0, 0); }
};

/* bf16 travels as its 16 bits */
template <> struct TypedOperand<bf16_t> {
	static constexpr int KPACK = 4;
	typedef s16x4 frag_t;
	static __device__ __forceinline__ bf16_t zero() { return (bf16_t) 0; }
	static __device__ __forceinline__ frag_t read(const bf16_t * s) { return *((const s16x4 *) s); }
	static __device__ __forceinline__ f32x4_t mfma(frag_t a, frag_t b, f32x4_t c) { return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, b, c, 0, 0, 0); }
};

template <typename O> struct TypedOutput;
template <> struct TypedOutput<float> {
	static __device__ __forceinline__ float load(const float * p) { return *p; }
	static __device__ __forceinline__ void store(float * p, float v) { *p = v; }
};
template <> struct TypedOutput<_Float16> {
	static __device__ __forceinline__ float load(const _Float16 * p) { return (float) *p; }
	static __device__ __forceinline__ void store(_Float16 * p, float v) { *p = (_Float16) v; }      /* round to nearest even */
};

#define TYPED_TILE 128
#define TYPED_THREADS 256

/* One operand's share of a k-tile: TYPED_TILE rows x BKT k, PER elements per thread, read so that consecutive threads
 * walk the operand's contiguous direction.  Elements outside the operand read as zero. */
template <typename E, int BKT>
struct TypedStage {
	static constexpr int PER = TYPED_TILE * BKT / TYPED_THREADS;
	E regs[PER];

	__device__ __forceinline__ void load(const E * base, bool kmajor, int row0, int rows_total, int k0, int K, int tid) {
		#pragma unroll
		for (int i = 0; i < PER; i++) {
			const int id = i * TYPED_THREADS + tid;
			const int row = kmajor ? id % TYPED_TILE : id / BKT;
			const int k = kmajor ? id / TYPED_TILE : id % BKT;
			const bool ok = (row0 + row < rows_total) && (k0 + k < K);
			const long long off = kmajor ? (long long) (k0 + k) * rows_total + (row0 + row) : (long long) (row0 + row) * K + (k0 + k);
			regs[i] = ok ? base[off] : TypedOperand<E>::zero();
		}
	}

	/* LDS tile [TYPED_TILE][LDK], k contiguous */
	template <int LDK>
	__device__ __forceinline__ void store(E * tile, bool kmajor, int tid) const {
		#pragma unroll
		for (int i = 0; i < PER; i++) {
			const int id = i * TYPED_THREADS + tid;
			const int row = kmajor ? id % TYPED_TILE : id / BKT;
			const int k = kmajor ? id / TYPED_TILE : id % BKT;
			tile[row * LDK + k] = regs[i];
		}
	}
};

template <typename E, typename O>
__global__ void __launch_bounds__(TYPED_THREADS)
gemm_typed_kernel(TypedGemmParams p) {
	typedef TypedOperand<E> Op;
	constexpr int KPACK = Op::KPACK;
	constexpr int BKT = 16 * KPACK;                         /* k-tile: four MFMA k-steps */
	constexpr int LDK = BKT + (KPACK == 1 ? 1 : 4);         /* padded row, keeps 8-byte alignment of the packed reads */
	constexpr int TM = 4, TN = 4;                           /* 16 x 16 blocks of a 64 x 64 wave tile */

	__shared__ __attribute__((aligned(16))) E sP[TYPED_TILE * LDK];
	__shared__ __attribute__((aligned(16))) E sQ[TYPED_TILE * LDK];

	const int tid = threadIdx.x;
	const int lane = tid & 63;
	const int wave = tid >> 6;
	const int wm = (wave & 1) * 64;
	const int wn = (wave >> 1) * 64;
	const int tiles_m = (p.M + TYPED_TILE - 1) / TYPED_TILE;
	const int m0 = (int) (blockIdx.x % tiles_m) * TYPED_TILE;
	const int n0 = (int) (blockIdx.x / tiles_m) * TYPED_TILE;
	const E * P = (const E *) p.P;
	const E * Q = (const E *) p.Q;
	const bool pk = p.p_kmajor != 0;
	const bool qk = p.q_kmajor != 0;

	f32x4_t acc[TM][TN];
	#pragma unroll
	for (int i = 0; i < TM; i++) {
		#pragma unroll
		for (int j = 0; j < TN; j++) {
			acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
		}
	}

	const int k_tiles = (p.K + BKT - 1) / BKT;
	TypedStage<E, BKT> stP, stQ;
	if (k_tiles > 0) {
		stP.load(P, pk, m0, p.M, 0, p.K, tid);
		stQ.load(Q, qk, n0, p.N, 0, p.K, tid);
	}
	const int r16 = lane & 15;
	const int g = lane >> 4;
	for (int kt = 0; kt < k_tiles; kt++) {
		__syncthreads();                                    /* the multiplies of the k-tile before are done with the LDS */
		stP.template store<LDK>(sP, pk, tid);
		stQ.template store<LDK>(sQ, qk, tid);
		__syncthreads();
		if (kt + 1 < k_tiles) {
			stP.load(P, pk, m0, p.M, (kt + 1) * BKT, p.K, tid);
			stQ.load(Q, qk, n0, p.N, (kt + 1) * BKT, p.K, tid);
		}
		#pragma unroll
		for (int s = 0; s < 4; s++) {
			/* lane (r16, g) feeds row r16 of a block with k = KPACK * (4 s + g) ... + KPACK - 1 */
			typename Op::frag_t fa[TM], fb[TN];
			#pragma unroll
			for (int i = 0; i < TM; i++) {
				fa[i] = Op::read(sP + (wm + 16 * i + r16) * LDK + KPACK * (4 * s + g));
			}
			#pragma unroll
			for (int j = 0; j < TN; j++) {
				fb[j] = Op::read(sQ + (wn + 16 * j + r16) * LDK + KPACK * (4 * s + g));
			}
			#pragma unroll
			for (int i = 0; i < TM; i++) {
				#pragma unroll
				for (int j = 0; j < TN; j++) {
					acc[i][j] = Op::mfma(fa[i], fb[j], acc[i][j]);
				}
			}
		}
	}

	/* a lane holds m = 16 i + 4 g + 0..3 of column n = 16 j + r16 */
	const O * C = (const O *) p.C;
	O * D = (O *) p.D;
	#pragma unroll
	for (int j = 0; j < TN; j++) {
		const int n = n0 + wn + 16 * j + r16;
		if (n >= p.N) {
			continue;
		}
		#pragma unroll
		for (int i = 0; i < TM; i++) {
			#pragma unroll
			for (int e = 0; e < 4; e++) {
				const int m = m0 + wm + 16 * i + 4 * g + e;
				if (m < p.M) {
					const long long off = (long long) n * p.M + m;
					float v = p.alpha * acc[i][j][e];
					if (C) {
						v = __builtin_fmaf(p.beta, TypedOutput<O>::load(C + off), v);
					}
					TypedOutput<O>::store(D + off, v);
				}
			}
		}
	}
}

#endif
