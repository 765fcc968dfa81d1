/*
 * amd_matmul.hip -- bf16 GEMM family for gfx950 behind the reference's external matmul op.
 *
 *   amd_matmul           the "default_matmul" op: replaces cublas_matmul
 *                        (backends/nvidia/src/ops/src/external/matmul_helper/src/matmul_helper.c:774-946)
 *   amd_grouped_matmul   one launch for all experts of a ragged group (an addition: the reference loops
 *                        over experts on the host, dataflow_transformer.c:2848-2940, 3460-3641, 4101-4148)
 *
 * Semantics (column-major BLAS view, matmul_helper.c:345-425):  D[M,N] = alpha*op(A)[M,K]*op(B)[K,N] + beta*C.
 * Read as row-major arrays: A is [M][K] (to_trans_a=1) or [K][M]; B is [N][K] (to_trans_b=0) or [K][N];
 * C and D are [N][M].  bf16 in and out, fp32 accumulation on the matrix cores, one rounding to bf16.
 *
 * Kernel: work-group tile BM x BN x 64, 4 or 8 waves, v_mfma_f32_32x32x16_bf16.  The M-side operand feeds
 * the MFMA "A" input and the N-side operand the "B" input, so each lane ends up holding four consecutive
 * m for one n -- contiguous in the [N][M] output -- and stores them as one 8-byte access.
 * Both LDS tiles are kept k-contiguous ([row][64] bf16, 16-byte chunks XOR-swizzled by row) so every MFMA
 * operand is one ds_read_b128; operands that are stored k-major in memory are transposed on the way in.
 */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "dataflow_amd.h"
#include "dataflow_amd_ops.h"

typedef uint16_t bf16_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define BK 64
#define CHUNKS_PER_ROW (BK / 8)

enum { MODE_SINGLE = 0, MODE_RAGGED_N = 1, MODE_RAGGED_K = 2 };

struct GemmParams {
	const bf16_t * A;
	const bf16_t * B;
	const bf16_t * C;
	bf16_t * D;
	int M, K, N;
	float alpha, beta;
	int num_groups;
	const int * cumsum;            /* inclusive prefix sum of group rows (device) */
	long long strideA;             /* elements between groups (ragged-N: of A; ragged-K: unused) */
	long long strideD;             /* elements between groups of C/D (ragged-K) */
};

struct Tile {
	const bf16_t * P;              /* M-side operand of this problem */
	const bf16_t * Q;              /* N-side operand */
	const bf16_t * C;
	bf16_t * D;
	int M, N, K;
	int m0, n0;
};

__device__ __forceinline__ float bf2f(uint32_t v16) { return __uint_as_float(v16 << 16); }
__device__ __forceinline__ uint32_t f2bf(float f) {
	uint32_t bits = __float_as_uint(f);
	if ((bits & 0x7fffffffu) > 0x7f800000u) {
		return (bits >> 16) | 0x0040u;
	}
	bits += 0x7fffu + ((bits >> 16) & 1u);
	return bits >> 16;
}

/* element offset of 16-byte chunk c of row r inside a [rows][64] bf16 LDS tile */
__device__ __forceinline__ int lds_chunk_off(int r, int c) {
	return r * BK + ((c ^ (r & 7)) << 3);
}

/* Work-groups are dealt to the 8 accelerator dies round-robin by linear id; give each die one contiguous
 * range of tiles so the tiles that run together share operands in that die's L2. */
__device__ __forceinline__ long xcd_remap(long b, long total) {
	long chunk = (total + 7) >> 3;
	if ((b >> 3) >= chunk) {
		return total;                                 /* surplus work-group of an over-sized grid */
	}
	return (b & 7) * chunk + (b >> 3);
}

template <int BM, int BN, int MODE>
__device__ __forceinline__ bool resolve_tile(const GemmParams & p, Tile & t) {
	const int tiles_m = (p.M + BM - 1) / BM;
	if (MODE == MODE_SINGLE) {
		const int tiles_n = (p.N + BN - 1) / BN;
		long total = (long) tiles_m * tiles_n;
		long id = xcd_remap(blockIdx.x, total);
		if (id >= total) {
			return false;
		}
		t.P = p.A; t.Q = p.B; t.C = p.C; t.D = p.D;
		t.M = p.M; t.N = p.N; t.K = p.K;
		t.m0 = (int) (id % tiles_m) * BM;
		t.n0 = (int) (id / tiles_m) * BN;
		return true;
	}
	if (MODE == MODE_RAGGED_N) {
		/* tile order: group, then n-tile, then m-tile (fastest) */
		long total_n_tiles = 0;
		int prev = 0;
		for (int g = 0; g < p.num_groups; g++) {
			int c = p.cumsum[g];
			total_n_tiles += (c - prev + BN - 1) / BN;
			prev = c;
		}
		long total = total_n_tiles * tiles_m;
		long id = xcd_remap(blockIdx.x, total);
		if (id >= total) {
			return false;
		}
		long nt = id / tiles_m;
		int tm = (int) (id % tiles_m);
		prev = 0;
		int g = 0;
		int n_g = 0;
		for (; g < p.num_groups; g++) {
			int c = p.cumsum[g];
			n_g = c - prev;
			long tg = (n_g + BN - 1) / BN;
			if (nt < tg) {
				break;
			}
			nt -= tg;
			prev = c;
		}
		t.P = p.A + (long long) g * p.strideA;
		t.Q = p.B + (long long) prev * p.K;
		t.C = p.C ? p.C + (long long) prev * p.M : nullptr;
		t.D = p.D + (long long) prev * p.M;
		t.M = p.M; t.N = n_g; t.K = p.K;
		t.m0 = tm * BM;
		t.n0 = (int) nt * BN;
		return true;
	}
	/* MODE_RAGGED_K: tile order: group, n-tile, m-tile */
	const int tiles_n = (p.N + BN - 1) / BN;
	long per_group = (long) tiles_m * tiles_n;
	long total = per_group * p.num_groups;
	long id = xcd_remap(blockIdx.x, total);
	if (id >= total) {
		return false;
	}
	int g = (int) (id / per_group);
	long r = id % per_group;
	int hi = p.cumsum[g];
	int lo = g ? p.cumsum[g - 1] : 0;
	if (hi - lo <= 0) {
		return false;                                 /* no rows: D keeps its value */
	}
	t.P = p.A + (long long) lo * p.M;
	t.Q = p.B + (long long) lo * p.N;
	t.C = p.C ? p.C + (long long) g * p.strideD : nullptr;
	t.D = p.D + (long long) g * p.strideD;
	t.M = p.M; t.N = p.N; t.K = hi - lo;
	t.m0 = (int) (r % tiles_m) * BM;
	t.n0 = (int) (r / tiles_m) * BN;
	return true;
}

/* ---- global -> registers -> LDS staging of one [ROWS][64] operand tile ---- */

/* operand stored [row][K] (k contiguous): one 16-byte chunk = 8 k of one row */
template <int ROWS, int THREADS>
struct StageKContig {
	static constexpr int CHUNKS = ROWS * CHUNKS_PER_ROW;
	static constexpr int PER_THREAD = (CHUNKS + THREADS - 1) / THREADS;
	u32x4 r[PER_THREAD];

	__device__ __forceinline__ void load(const bf16_t * src, int row0, int rows_total, int k0, int K, bool vec_ok) {
		#pragma unroll
		for (int i = 0; i < PER_THREAD; i++) {
			int id = i * THREADS + threadIdx.x;
			int row = id / CHUNKS_PER_ROW;
			int c = id % CHUNKS_PER_ROW;
			int gr = row0 + row;
			int gk = k0 + c * 8;
			u32x4 v = {0u, 0u, 0u, 0u};
			if (id < CHUNKS && gr < rows_total && gk < K) {
				const bf16_t * ptr = src + (long long) gr * K + gk;
				if (vec_ok && gk + 8 <= K) {
					v = *((const u32x4 *) ptr);
				} else {
					uint32_t e[8];
					#pragma unroll
					for (int j = 0; j < 8; j++) {
						e[j] = (gk + j < K) ? (uint32_t) ptr[j] : 0u;
					}
					v.x = e[0] | (e[1] << 16); v.y = e[2] | (e[3] << 16); v.z = e[4] | (e[5] << 16); v.w = e[6] | (e[7] << 16);
				}
			}
			r[i] = v;
		}
	}

	__device__ __forceinline__ void store(bf16_t * lds) const {
		#pragma unroll
		for (int i = 0; i < PER_THREAD; i++) {
			int id = i * THREADS + threadIdx.x;
			if (id < CHUNKS) {
				int row = id / CHUNKS_PER_ROW;
				int c = id % CHUNKS_PER_ROW;
				*((u32x4 *) (lds + lds_chunk_off(row, c))) = r[i];
			}
		}
	}
};

/* operand stored [K][rows_total] (row index contiguous): one 16-byte chunk = 8 rows at one k; it is
 * scattered into the k-contiguous LDS tile element by element */
template <int ROWS, int THREADS>
struct StageKMajor {
	static constexpr int CHUNKS = BK * (ROWS / 8);
	static constexpr int PER_THREAD = (CHUNKS + THREADS - 1) / THREADS;
	u32x4 r[PER_THREAD];

	__device__ __forceinline__ void load(const bf16_t * src, int row0, int rows_total, int k0, int K, bool vec_ok) {
		#pragma unroll
		for (int i = 0; i < PER_THREAD; i++) {
			int id = i * THREADS + threadIdx.x;
			int k = id / (ROWS / 8);
			int rc = id % (ROWS / 8);
			int gk = k0 + k;
			int gr = row0 + rc * 8;
			u32x4 v = {0u, 0u, 0u, 0u};
			if (id < CHUNKS && gk < K && gr < rows_total) {
				const bf16_t * ptr = src + (long long) gk * rows_total + gr;
				if (vec_ok && gr + 8 <= rows_total) {
					v = *((const u32x4 *) ptr);
				} else {
					uint32_t e[8];
					#pragma unroll
					for (int j = 0; j < 8; j++) {
						e[j] = (gr + j < rows_total) ? (uint32_t) ptr[j] : 0u;
					}
					v.x = e[0] | (e[1] << 16); v.y = e[2] | (e[3] << 16); v.z = e[4] | (e[5] << 16); v.w = e[6] | (e[7] << 16);
				}
			}
			r[i] = v;
		}
	}

	__device__ __forceinline__ void store(bf16_t * lds) const {
		#pragma unroll
		for (int i = 0; i < PER_THREAD; i++) {
			int id = i * THREADS + threadIdx.x;
			if (id < CHUNKS) {
				int k = id / (ROWS / 8);
				int rc = id % (ROWS / 8);
				uint32_t w[4] = {r[i].x, r[i].y, r[i].z, r[i].w};
				#pragma unroll
				for (int j = 0; j < 8; j++) {
					int row = rc * 8 + j;
					lds[lds_chunk_off(row, k >> 3) + (k & 7)] = (bf16_t) ((w[j >> 1] >> ((j & 1) * 16)) & 0xffffu);
				}
			}
		}
	}
};

template <bool KMAJOR, int ROWS, int THREADS> struct StagePick { typedef StageKContig<ROWS, THREADS> type; };
template <int ROWS, int THREADS> struct StagePick<true, ROWS, THREADS> { typedef StageKMajor<ROWS, THREADS> type; };

/* ---- the kernel ---- */

template <int BM, int BN, int WAVES_M, int WAVES_N, bool P_KMAJOR, bool Q_KMAJOR, int MODE>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_bf16_kernel(GemmParams p) {
	constexpr int THREADS = WAVES_M * WAVES_N * 64;
	constexpr int WTM = BM / WAVES_M;
	constexpr int WTN = BN / WAVES_N;
	constexpr int TM = WTM / 32;
	constexpr int TN = WTN / 32;
	static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be a multiple of the 32x32 MFMA tile");

	extern __shared__ __attribute__((aligned(16))) bf16_t lds[];
	constexpr int STAGE = (BM + BN) * BK;            /* elements per pipeline stage: P tile then Q tile */

	Tile t;
	if (!resolve_tile<BM, BN, MODE>(p, t)) {
		return;
	}

	const int lane = threadIdx.x & 63;
	const int wave = threadIdx.x >> 6;
	const int wm = (wave % WAVES_M) * WTM;
	const int wn = (wave / WAVES_M) * WTN;

	/* 16-byte global accesses need the contiguous extent to be a multiple of 8 elements and an aligned base */
	const bool p_vec = P_KMAJOR ? (((t.M & 7) == 0) && ((((uintptr_t) t.P) & 15) == 0)) : (((t.K & 7) == 0) && ((((uintptr_t) t.P) & 15) == 0));
	const bool q_vec = Q_KMAJOR ? (((t.N & 7) == 0) && ((((uintptr_t) t.Q) & 15) == 0)) : (((t.K & 7) == 0) && ((((uintptr_t) t.Q) & 15) == 0));

	typename StagePick<P_KMAJOR, BM, THREADS>::type stP;
	typename StagePick<Q_KMAJOR, BN, THREADS>::type stQ;

	f32x16 acc[TM][TN];
	#pragma unroll
	for (int i = 0; i < TM; i++) {
		#pragma unroll
		for (int j = 0; j < TN; j++) {
			#pragma unroll
			for (int r = 0; r < 16; r++) {
				acc[i][j][r] = 0.0f;
			}
		}
	}

	const int k_tiles = (t.K + BK - 1) / BK;
	stP.load(t.P, t.m0, t.M, 0, t.K, p_vec);
	stQ.load(t.Q, t.n0, t.N, 0, t.K, q_vec);
	stP.store(lds);
	stQ.store(lds + BM * BK);
	__syncthreads();

	for (int kt = 0; kt < k_tiles; kt++) {
		const int cur = kt & 1;
		if (kt + 1 < k_tiles) {
			stP.load(t.P, t.m0, t.M, (kt + 1) * BK, t.K, p_vec);
			stQ.load(t.Q, t.n0, t.N, (kt + 1) * BK, t.K, q_vec);
		}
		const bf16_t * cp = lds + cur * STAGE;
		const bf16_t * cq = cp + BM * BK;
		#pragma unroll
		for (int s = 0; s < BK / 16; s++) {
			bf16x8 a[TM], b[TN];
			const int c = 2 * s + (lane >> 5);
			#pragma unroll
			for (int i = 0; i < TM; i++) {
				a[i] = *((const bf16x8 *) (cp + lds_chunk_off(wm + i * 32 + (lane & 31), c)));
			}
			#pragma unroll
			for (int j = 0; j < TN; j++) {
				b[j] = *((const bf16x8 *) (cq + lds_chunk_off(wn + j * 32 + (lane & 31), c)));
			}
			#pragma unroll
			for (int i = 0; i < TM; i++) {
				#pragma unroll
				for (int j = 0; j < TN; j++) {
					acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
				}
			}
		}
		if (kt + 1 < k_tiles) {
			/* the other buffer was last read in iteration kt-1, and every wave passed the barrier below since */
			stP.store(lds + (cur ^ 1) * STAGE);
			stQ.store(lds + (cur ^ 1) * STAGE + BM * BK);
		}
		__syncthreads();
	}

	/* epilogue: lane holds n = lane%32 and, per register group q, m = 8q + 4*(lane/32) + {0,1,2,3} */
	const bool use_c = (t.C != nullptr) && (p.beta != 0.0f);
	const bool m_vec = ((t.M & 3) == 0) && ((((uintptr_t) t.D) & 7) == 0) && (!use_c || ((((uintptr_t) t.C) & 7) == 0));
	#pragma unroll
	for (int j = 0; j < TN; j++) {
		const int n = t.n0 + wn + j * 32 + (lane & 31);
		if (n >= t.N) {
			continue;
		}
		#pragma unroll
		for (int i = 0; i < TM; i++) {
			#pragma unroll
			for (int q = 0; q < 4; q++) {
				const int m = t.m0 + wm + i * 32 + q * 8 + ((lane >> 5) << 2);
				if (m >= t.M) {
					continue;
				}
				float v[4];
				#pragma unroll
				for (int e = 0; e < 4; e++) {
					v[e] = p.alpha * acc[i][j][q * 4 + e];
				}
				const long long off = (long long) n * t.M + m;
				if (m_vec && m + 4 <= t.M) {
					if (use_c) {
						u32x2 cv = *((const u32x2 *) (t.C + off));
						v[0] = __builtin_fmaf(p.beta, bf2f(cv.x & 0xffffu), v[0]);
						v[1] = __builtin_fmaf(p.beta, bf2f(cv.x >> 16), v[1]);
						v[2] = __builtin_fmaf(p.beta, bf2f(cv.y & 0xffffu), v[2]);
						v[3] = __builtin_fmaf(p.beta, bf2f(cv.y >> 16), v[3]);
					}
					u32x2 o;
					o.x = f2bf(v[0]) | (f2bf(v[1]) << 16);
					o.y = f2bf(v[2]) | (f2bf(v[3]) << 16);
					*((u32x2 *) (t.D + off)) = o;
				} else {
					#pragma unroll
					for (int e = 0; e < 4; e++) {
						if (m + e < t.M) {
							float r = v[e];
							if (use_c) {
								r = __builtin_fmaf(p.beta, bf2f(t.C[off + e]), r);
							}
							t.D[off + e] = (bf16_t) f2bf(r);
						}
					}
				}
			}
		}
	}
}

/* ------------------------------------------------------------------ host side */

struct MatmulExtra {
	int cu_count;
	int lds_optin;
};

template <int BM, int BN, int WAVES_M, int WAVES_N, bool PK, bool QK, int MODE>
static int launch_variant(const GemmParams & p, long grid, hipStream_t stream) {
	constexpr int threads = WAVES_M * WAVES_N * 64;
	constexpr size_t lds_bytes = 2 * (BM + BN) * BK * sizeof(bf16_t);
	auto kernel = gemm_bf16_kernel<BM, BN, WAVES_M, WAVES_N, PK, QK, MODE>;
	static bool attr_done = false;
	if (lds_bytes > 65536 && !attr_done) {
		hipError_t e = hipFuncSetAttribute((const void *) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_bytes);
		if (e != hipSuccess) {
			fprintf(stderr, "Error: could not raise dynamic LDS limit to %zu bytes: %s...\n", lds_bytes, hipGetErrorString(e));
			return -1;
		}
		attr_done = true;
	}
	if (grid <= 0) {
		return 0;
	}
	hipLaunchKernelGGL(kernel, dim3((unsigned int) grid), dim3(threads), lds_bytes, stream, p);
	hipError_t e = hipGetLastError();
	if (e != hipSuccess) {
		fprintf(stderr, "Error: gemm kernel launch failed: %s...\n", hipGetErrorString(e));
		return -1;
	}
	return 0;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int MODE>
static int launch_layout(const GemmParams & p, int transa, int transb, long grid, hipStream_t stream) {
	/* to_trans_a = 1 means A is stored [M][K] (k contiguous); to_trans_b = 1 means B is stored [K][N] (k-major) */
	const bool pk = !transa;
	const bool qk = transb != 0;
	if (!pk && !qk) { return launch_variant<BM, BN, WAVES_M, WAVES_N, false, false, MODE>(p, grid, stream); }
	if (pk && !qk) { return launch_variant<BM, BN, WAVES_M, WAVES_N, true, false, MODE>(p, grid, stream); }
	if (pk && qk) { return launch_variant<BM, BN, WAVES_M, WAVES_N, true, true, MODE>(p, grid, stream); }
	return launch_variant<BM, BN, WAVES_M, WAVES_N, false, true, MODE>(p, grid, stream);
}

static long round_up8(long v) { return (v + 7) & ~7L; }

static int check_dtypes(DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
						DataflowDatatype compute_dt, const void * C, float beta) {
	if (a_dt != DATAFLOW_BF16 || b_dt != DATAFLOW_BF16 || d_dt != DATAFLOW_BF16) {
		fprintf(stderr, "Error: this matmul implements BF16 operands and output only (got A=%s B=%s D=%s)...\n",
				dataflow_datatype_as_string(a_dt), dataflow_datatype_as_string(b_dt), dataflow_datatype_as_string(d_dt));
		return -1;
	}
	if (c_dt != DATAFLOW_NONE && c_dt != DATAFLOW_BF16 && C != NULL && beta != 0.0f) {
		fprintf(stderr, "Error: this matmul implements a BF16 C only (got %s)...\n", dataflow_datatype_as_string(c_dt));
		return -1;
	}
	if (compute_dt != DATAFLOW_FP32 && compute_dt != DATAFLOW_BF16 && compute_dt != DATAFLOW_NONE) {
		fprintf(stderr, "Error: unsupported compute type %s; accumulation is always fp32...\n", dataflow_datatype_as_string(compute_dt));
		return -1;
	}
	return 0;
}

static int resolve_stream(Dataflow_Handle * handle, int stream_id, hipStream_t * stream) {
	if (stream_id == -1) {
		*stream = NULL;
		return 0;
	}
	if (stream_id < 0 || stream_id >= handle->num_streams) {
		fprintf(stderr, "Error: trying to dispatch matmul on stream id %d, but only have %d streams...\n", stream_id, handle->num_streams);
		return -1;
	}
	*stream = ((hipStream_t *) handle->streams)[stream_id];
	return 0;
}

extern "C" int amd_matmul_init(Dataflow_Handle * dataflow_handle, void * op_table_value) {
	Hip_Function * fn = (Hip_Function *) op_table_value;
	MatmulExtra * extra = (MatmulExtra *) calloc(1, sizeof(MatmulExtra));
	if (!extra) {
		fprintf(stderr, "Error: malloc failed for matmul op extra...\n");
		return -1;
	}
	Hip_Device_Info * info = (Hip_Device_Info *) dataflow_handle->device_info;
	extra->cu_count = info ? info->cu_count : 256;
	extra->lds_optin = info ? info->optin_max_lds_per_block : 65536;
	fn->op_extra = extra;
	return 0;
}

extern "C" int amd_matmul(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra) {
	(void) op_extra;
	void ** a = op->op_args;
	DataflowDatatype a_dt = *((DataflowDatatype *) a[1]);
	DataflowDatatype b_dt = *((DataflowDatatype *) a[2]);
	DataflowDatatype c_dt = *((DataflowDatatype *) a[3]);
	DataflowDatatype d_dt = *((DataflowDatatype *) a[4]);
	DataflowDatatype compute_dt = *((DataflowDatatype *) a[5]);
	int transa = *((int *) a[6]);
	int transb = *((int *) a[7]);
	GemmParams p;
	memset(&p, 0, sizeof(p));
	p.M = *((int *) a[8]);
	p.K = *((int *) a[9]);
	p.N = *((int *) a[10]);
	p.alpha = *((float *) a[11]);
	p.beta = *((float *) a[12]);
	p.A = (const bf16_t *) *((uint64_t *) a[13]);
	p.B = (const bf16_t *) *((uint64_t *) a[14]);
	p.C = (const bf16_t *) *((uint64_t *) a[15]);
	p.D = (bf16_t *) *((uint64_t *) a[16]);
	if (c_dt == DATAFLOW_NONE || p.beta == 0.0f) {
		p.C = NULL;
	}
	if (check_dtypes(a_dt, b_dt, c_dt, d_dt, compute_dt, p.C, p.beta)) {
		return -1;
	}
	if (p.M < 0 || p.N < 0 || p.K < 0 || !p.D || ((p.M > 0 && p.N > 0 && p.K > 0) && (!p.A || !p.B))) {
		fprintf(stderr, "Error: bad matmul arguments M=%d K=%d N=%d A=%p B=%p D=%p...\n", p.M, p.K, p.N, (void *) p.A, (void *) p.B, (void *) p.D);
		return -1;
	}
	if (p.M == 0 || p.N == 0) {
		return 0;
	}
	hipStream_t stream;
	if (resolve_stream(dataflow_handle, stream_id, &stream)) {
		return -1;
	}
	if (hipSetDevice(dataflow_handle->device_id) != hipSuccess) {
		fprintf(stderr, "Error: hipSetDevice failed in matmul...\n");
		return -1;
	}
	/* small problems: 128x128 tiles fill the device better; large ones amortise operand traffic with 256x256 */
	long tiles_big = (long) ((p.M + 255) / 256) * ((p.N + 255) / 256);
	if (tiles_big >= 256 && p.M >= 256 && p.N >= 256) {
		return launch_layout<256, 256, 2, 2, MODE_SINGLE>(p, transa, transb, round_up8(tiles_big), stream);
	}
	long tiles = (long) ((p.M + 127) / 128) * ((p.N + 127) / 128);
	return launch_layout<128, 128, 2, 2, MODE_SINGLE>(p, transa, transb, round_up8(tiles), stream);
}

extern "C" int amd_grouped_matmul(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra) {
	(void) op_extra;
	void ** a = op->op_args;
	DataflowDatatype a_dt = *((DataflowDatatype *) a[1]);
	DataflowDatatype b_dt = *((DataflowDatatype *) a[2]);
	DataflowDatatype c_dt = *((DataflowDatatype *) a[3]);
	DataflowDatatype d_dt = *((DataflowDatatype *) a[4]);
	DataflowDatatype compute_dt = *((DataflowDatatype *) a[5]);
	int transa = *((int *) a[6]);
	int transb = *((int *) a[7]);
	int ragged = *((int *) a[8]);
	GemmParams p;
	memset(&p, 0, sizeof(p));
	p.M = *((int *) a[9]);
	p.K = *((int *) a[10]);
	p.N = *((int *) a[11]);
	p.num_groups = *((int *) a[12]);
	p.cumsum = (const int *) *((uint64_t *) a[13]);
	p.alpha = *((float *) a[14]);
	p.beta = *((float *) a[15]);
	p.A = (const bf16_t *) *((uint64_t *) a[16]);
	uint64_t strideA_bytes = *((uint64_t *) a[17]);
	p.B = (const bf16_t *) *((uint64_t *) a[18]);
	p.C = (const bf16_t *) *((uint64_t *) a[19]);
	p.D = (bf16_t *) *((uint64_t *) a[20]);
	uint64_t strideD_bytes = *((uint64_t *) a[21]);
	if (c_dt == DATAFLOW_NONE || p.beta == 0.0f) {
		p.C = NULL;
	}
	if (check_dtypes(a_dt, b_dt, c_dt, d_dt, compute_dt, p.C, p.beta)) {
		return -1;
	}
	if (p.num_groups < 1 || !p.cumsum || !p.A || !p.B || !p.D || p.M < 1 || (strideA_bytes & 1) || (strideD_bytes & 1)) {
		fprintf(stderr, "Error: bad grouped matmul arguments (groups=%d M=%d K=%d N=%d)...\n", p.num_groups, p.M, p.K, p.N);
		return -1;
	}
	p.strideA = (long long) (strideA_bytes / 2);
	p.strideD = (long long) (strideD_bytes / 2);
	hipStream_t stream;
	if (resolve_stream(dataflow_handle, stream_id, &stream)) {
		return -1;
	}
	if (hipSetDevice(dataflow_handle->device_id) != hipSuccess) {
		fprintf(stderr, "Error: hipSetDevice failed in grouped matmul...\n");
		return -1;
	}
	if (ragged == AMD_GROUPED_RAGGED_N) {
		if (transb != 0 || p.K < 1 || p.N < 0) {
			fprintf(stderr, "Error: ragged-N grouped matmul needs to_trans_b == 0 and K >= 1...\n");
			return -1;
		}
		if (p.N == 0) {
			return 0;
		}
		/* upper bound of n-tiles: every group may end in one partial tile */
		long tiles_m = (p.M + 255) / 256;
		long tiles = tiles_m * ((long) p.N / 256 + p.num_groups);
		return launch_layout<256, 256, 2, 2, MODE_RAGGED_N>(p, transa, transb, round_up8(tiles), stream);
	}
	if (ragged == AMD_GROUPED_RAGGED_K) {
		if (transa != 0 || transb != 1 || p.N < 1) {
			fprintf(stderr, "Error: ragged-K grouped matmul needs to_trans_a == 0 and to_trans_b == 1...\n");
			return -1;
		}
		long tiles = (long) ((p.M + 255) / 256) * ((p.N + 255) / 256) * p.num_groups;
		return launch_layout<256, 256, 2, 2, MODE_RAGGED_K>(p, transa, transb, round_up8(tiles), stream);
	}
	fprintf(stderr, "Error: unknown ragged dimension %d...\n", ragged);
	return -1;
}
