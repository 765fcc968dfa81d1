/*
 * gemm_kernel.h -- device code of the bf16 GEMM family for gfx950 (see amd_matmul.hip for the semantics).
 *
 * Three kernels share the tile resolver:
 *
 *   gemm_bf16_stream_kernel   the fast path for large problems (256 x 256 tiles, or 256 x 288 for the token rows of a
 *       ragged-N launch without a C operand): one persistent work-group per
 *       compute unit walks over many output tiles with the operand stream of the direct kernel below, the MFMA
 *       operands one k-step ahead in registers, and a line-coalesced epilogue through its own LDS scratch.
 *
 *   gemm_bf16_direct_kernel   one work-group per output tile (128 x 128 tiles, small problems).  Operand tiles go from global memory straight into LDS with
 *       16-byte buffer loads (no VGPR staging); out-of-range rows and the k tail are zero-filled by the buffer
 *       bounds check.  Two LDS stages: the loads of k-tile i+1 are in flight while k-tile i is multiplied.
 *       Operands stored k-contiguous are kept [row][64] in LDS (16-byte chunks XOR-swizzled by row) and read
 *       with ds_read_b128; operands stored k-major are kept [64][rows] (32-byte groups XOR-swizzled by k) and
 *       read with the transposing ds_read_b64_tr_b16, so no layout needs an explicit transpose.
 *       Needs the contiguous extent of each operand to be a multiple of 8 elements and 16-byte aligned bases.
 *
 *   gemm_bf16_staged_kernel   any shape / alignment: global -> registers -> LDS with element-wise fallbacks.
 *
 * All use v_mfma_f32_16x16x32_bf16 with the M-side operand as MFMA input A and the N-side operand as
 * input B: a lane then holds four consecutive m for one n, contiguous in the [N][M] output.
 */
#ifndef GEMM_KERNEL_H
#define GEMM_KERNEL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

#define BK 64
#define CHUNKS_PER_ROW (BK / 8)
#define LDS_PTR(p) ((__attribute__((address_space(3))) void *) (p))

enum { MODE_SINGLE = 0, MODE_RAGGED_N = 1, MODE_RAGGED_K = 2 };
/* which operand of a grouped problem is fetched through a row map (GemmParams::gather) */
enum { GATHER_NONE = 0, GATHER_Q_ROWS = 1, GATHER_P_KROWS = 2 };

struct GemmParams {
	const bf16_t * A;
	const bf16_t * B;
	const bf16_t * C;
	bf16_t * D;
	int M, K, N;
	float alpha, beta;
	int num_groups;
	const int * cumsum;            /* inclusive prefix sum of group rows (device) */
	long long strideA;             /* elements between groups of A (ragged-N) */
	long long strideD;             /* elements between groups of C/D (ragged-K) */
	/* gathered token rows: row i of group g of the operand whose rows are the groups' rows (B in ragged-N, where a row
	 * is K elements; A in ragged-K, where a row is M elements) is row gather[base_g + i] of that operand, an array of
	 * gather_rows rows (below 4 GiB in all); NULL: the rows are packed in the operand itself */
	const int * gather;
	int gather_rows;
	/* split-K (single problems on the direct kernel only): work-group b computes k-tiles
	 * [ks * kt_per_split, (ks+1) * kt_per_split) of tile b % tiles, ks = b / tiles, and writes its fp32 partial sums
	 * (no alpha, beta or C) to partial[ks][n * M + m]; splitk_reduce_kernel turns them into D */
	float * partial;
	int split_k;                   /* 0 or 1: off */
	int kt_per_split;              /* even */
	/* Ragged-N launches without C that both the eight-wave kernel (token rows in tiles of 288) and the four-wave
	 * kernel with the 256 x 384 tile can take are launched on both; each work-group counts the tiles of the two tilings
	 * from the device prefix sum (ragged_n_prefers_384) and the kernel that loses returns at once.
	 * 0: run; ARBITRATE_NARROW: run unless the 384 tiling wins; ARBITRATE_WIDE: run only if it wins */
	int arbitrate;
};
enum { ARBITRATE_NONE = 0, ARBITRATE_NARROW = 1, ARBITRATE_WIDE = 2 };

struct Tile {
	const bf16_t * P;              /* M-side operand of this problem */
	const bf16_t * Q;              /* N-side operand */
	const int * Qmap;              /* gathered N-side operand (ragged-N): row n of the problem is row Qmap[n] of Q; else NULL */
	const int * Pmap;              /* gathered M-side operand (ragged-K): its row k is row Pmap[k] of P; else NULL */
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

/* two fp32 -> one packed pair of bf16 (round to nearest even) in a single v_cvt_pk_bf16_f32 */
typedef float f32x2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack2_bf16(float lo, float hi) {
	const f32x2_t v = {lo, hi};
	return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

/* Element offset of 16-byte chunk c of row r inside a k-contiguous [rows][64] LDS tile.  A row is 128 bytes, so
 * two rows span the 64 banks; XOR-ing the chunk index with bits 1..3 of the row makes the sixteen 16-byte reads of
 * any 16 consecutive rows at one k land on sixteen different bank groups. */
__device__ __forceinline__ int lds_chunk_off(int r, int c) {
	return r * BK + ((c ^ ((r >> 1) & 7)) << 3);
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

/* number of tiles of the launch (ragged-N: read from the device prefix sum) */
template <int BM, int BN, int MODE>
__device__ __forceinline__ long count_tiles(const GemmParams & p) {
	const int tiles_m = (p.M + BM - 1) / BM;
	if (MODE == MODE_SINGLE) {
		return (long) tiles_m * ((p.N + BN - 1) / BN);
	}
	if (MODE == MODE_RAGGED_K) {
		return (long) tiles_m * ((p.N + BN - 1) / BN) * p.num_groups;
	}
	const int lane = threadIdx.x & 63;
	long total_n_tiles = 0;
	int carry_rows = 0;
	for (int base = 0; base < p.num_groups; base += 64) {
		const int g = base + lane;
		const int c = (g < p.num_groups) ? p.cumsum[g] : 0;
		int prev = __shfl_up(c, 1, 64);
		if (lane == 0) {
			prev = carry_rows;
		}
		int tiles = (g < p.num_groups) ? (c - prev + BN - 1) / BN : 0;
		#pragma unroll
		for (int off = 1; off < 64; off <<= 1) {
			int up = __shfl_up(tiles, off, 64);
			if (lane >= off) {
				tiles += up;
			}
		}
		total_n_tiles += __shfl(tiles, 63, 64);
		carry_rows = __shfl(c, min(63, p.num_groups - base - 1), 64);
	}
	return (long) __builtin_amdgcn_readfirstlane((int) total_n_tiles) * tiles_m;
}

/* Which tiling of the token rows is cheaper for this launch.  A launch takes (rounds of tiles over the work-groups) x
 * (time of a tile), and a k-tile step is paced by the bytes it fetches: 256 + 288 rows against 256 + 384 rows of 128
 * bytes, the larger tile at 3 % fewer bytes per clock plus what 1.6 k-tiles take per tile (its tiles change over
 * with fewer loads in flight; measured over group sizes of 256-2048 rows, K of 1024-4096 and the layer's launches: 3-7 %
 * at 64 k-tiles, 7-15 % at 16).  The 384 tiling wins where the groups are long enough to fill its tiles and the rounds
 * come out even; with short or very uneven groups the narrower tile wastes less.  Every work-group of both launches
 * computes the same answer.  Both sides are scaled by the k-tiles of a tile. */
#define WIDE_TILE_COST(rounds, k_tiles) ((rounds) * (256 + 384) * (103 * (k_tiles) + 160))
#define NARROW_TILE_COST(rounds, k_tiles) ((rounds) * (256 + 288) * 100 * (k_tiles))
__device__ __forceinline__ bool ragged_n_prefers_384(const GemmParams & p) {
	const long groups = gridDim.x;
	const long narrow = (count_tiles<256, 288, MODE_RAGGED_N>(p) + groups - 1) / groups;
	const long wide = (count_tiles<256, 384, MODE_RAGGED_N>(p) + groups - 1) / groups;
	const long k_tiles = (p.K + BK - 1) / BK;
	return WIDE_TILE_COST(wide, k_tiles) < NARROW_TILE_COST(narrow, k_tiles);
}

/* Order of the tiles of one problem (tiles_m x tiles_n of them, `lid` counts them): the work-groups of a die run 32
 * consecutive tiles at a time, and what they fetch is one operand panel per distinct m-tile plus one per distinct
 * n-tile among those 32; a panel that k of them share is fetched once and the k work-groups that wait for its lines
 * move in step.  The order walks blocks of 8 m-tiles x 4 n-tiles, inside a block m by m with n fastest: 32 consecutive
 * tiles then hold 8 + 4 panels, each M-side panel (the weights: the operand that always comes from HBM) shared by all
 * the n-tiles it has in the block.  Where tiles_n is not a multiple of 4 the last n-tiles form a narrower block, so
 * with 3 n-tiles (groups of about 1024 rows in tiles of 384) every M-side panel is still shared three ways, and not
 * by one tile in one round and two in the next. */
__device__ __forceinline__ void tile_in_problem(int lid, int tiles_m, int tiles_n, int & tm, int & tn) {
	const int mb = (tiles_m > 8 && (tiles_m & 7) == 0) ? 8 : tiles_m;
	const int per_block = mb * tiles_n;
	const int blk = lid / per_block;
	const int rem = lid - blk * per_block;
	const int whole = (tiles_n >> 2) * 4 * mb;              /* tiles of the m-block that lie in full groups of 4 n-tiles */
	if (rem < whole) {
		const int grp = rem / (4 * mb);
		const int r = rem - grp * 4 * mb;
		tm = blk * mb + (r >> 2);
		tn = grp * 4 + (r & 3);
	} else {
		const int last = tiles_n & 3;
		const int r = rem - whole;
		tm = blk * mb + r / last;
		tn = (tiles_n & ~3) + r % last;
	}
}

/* tile `id` (0 <= id < count_tiles) of the launch; false if it has nothing to do */
template <int BM, int BN, int MODE>
__device__ __forceinline__ bool resolve_tile_id(const GemmParams & p, long id, Tile & t) {
	const int tiles_m = (p.M + BM - 1) / BM;
	if (MODE == MODE_SINGLE) {
		t.P = p.A; t.Q = p.B; t.Qmap = nullptr; t.Pmap = nullptr; t.C = p.C; t.D = p.D;
		t.M = p.M; t.N = p.N; t.K = p.K;
		int tm_, tn_;
		tile_in_problem((int) id, tiles_m, (p.N + BN - 1) / BN, tm_, tn_);
		t.m0 = tm_ * BM;
		t.n0 = tn_ * BN;
		return true;
	}
	if (MODE == MODE_RAGGED_N) {
		const int lane = threadIdx.x & 63;
		const int nt = (int) (id / tiles_m);                /* finds the group: a group owns tiles_m * (its n-tiles) consecutive ids */
		int found_g = 0, found_prev = 0, found_rows = 0, found_nt = 0;
		int tiles_before = 0;
		int carry_rows = 0;
		for (int base = 0; base < p.num_groups; base += 64) {
			const int g = base + lane;
			const int c = (g < p.num_groups) ? p.cumsum[g] : 0;
			int prev = __shfl_up(c, 1, 64);
			if (lane == 0) {
				prev = carry_rows;
			}
			const int mine = (g < p.num_groups) ? (c - prev + BN - 1) / BN : 0;
			int incl = mine;
			#pragma unroll
			for (int off = 1; off < 64; off <<= 1) {
				int up = __shfl_up(incl, off, 64);
				if (lane >= off) {
					incl += up;
				}
			}
			const uint64_t past = __ballot((g < p.num_groups) && (tiles_before + incl > nt));
			if (past) {
				const int src = __ffsll((long long) past) - 1;
				found_g = base + src;
				found_prev = __shfl(prev, src, 64);
				found_rows = __shfl(c - prev, src, 64);
				found_nt = nt - (tiles_before + __shfl(incl - mine, src, 64));
				break;
			}
			tiles_before += __shfl(incl, 63, 64);
			carry_rows = __shfl(c, min(63, p.num_groups - base - 1), 64);
		}
		found_g = __builtin_amdgcn_readfirstlane(found_g);
		found_prev = __builtin_amdgcn_readfirstlane(found_prev);
		found_rows = __builtin_amdgcn_readfirstlane(found_rows);
		found_nt = __builtin_amdgcn_readfirstlane(found_nt);
		/* found_nt counted whole rows of tiles_m ids inside the group; redo the split with the blocked order */
		int tm, tn;
		tile_in_problem(found_nt * tiles_m + (int) (id % tiles_m), tiles_m, (found_rows + BN - 1) / BN, tm, tn);
		found_nt = tn;
		t.P = p.A + (long long) found_g * p.strideA;
		t.Q = p.gather ? p.B : p.B + (long long) found_prev * p.K;
		t.Qmap = p.gather ? p.gather + found_prev : nullptr;
		t.Pmap = nullptr;
		t.C = p.C ? p.C + (long long) found_prev * p.M : nullptr;
		t.D = p.D + (long long) found_prev * p.M;
		t.M = p.M; t.N = found_rows; t.K = p.K;
		t.m0 = tm * BM;
		t.n0 = found_nt * BN;
		return true;
	}
	const int tiles_n = (p.N + BN - 1) / BN;
	const long per_group = (long) tiles_m * tiles_n;
	const int g = (int) (id / per_group);
	const long r = id % per_group;
	const int hi = p.cumsum[g];
	const int lo = g ? p.cumsum[g - 1] : 0;
	if (hi - lo <= 0) {
		return false;                                 /* no rows: D keeps its value */
	}
	t.P = p.gather ? p.A : p.A + (long long) lo * p.M;
	t.Pmap = p.gather ? p.gather + lo : nullptr;
	t.Q = p.B + (long long) lo * p.N;
	t.Qmap = nullptr;
	t.C = p.C ? p.C + (long long) g * p.strideD : nullptr;
	t.D = p.D + (long long) g * p.strideD;
	t.M = p.M; t.N = p.N; t.K = hi - lo;
	int tm_, tn_;
	tile_in_problem((int) r, tiles_m, tiles_n, tm_, tn_);
	t.m0 = tm_ * BM;
	t.n0 = tn_ * BN;
	return true;
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
		t.P = p.A; t.Q = p.B; t.Qmap = nullptr; t.Pmap = nullptr; t.C = p.C; t.D = p.D;
		t.M = p.M; t.N = p.N; t.K = p.K;
		t.m0 = (int) (id % tiles_m) * BM;
		t.n0 = (int) (id / tiles_m) * BN;
		return true;
	}
	if (MODE == MODE_RAGGED_N) {
		/* Tile order: group, then n-tile, then m-tile (fastest).  The per-group tile counts come from the device-side
		 * prefix sum; every wave scans them on its own, 64 groups per step with one coalesced load and shuffles,
		 * instead of walking the array with dependent scalar loads. */
		const int lane = threadIdx.x & 63;
		long total_n_tiles = 0;
		int carry_rows = 0;
		for (int base = 0; base < p.num_groups; base += 64) {
			const int g = base + lane;
			const int c = (g < p.num_groups) ? p.cumsum[g] : 0;
			int prev = __shfl_up(c, 1, 64);
			if (lane == 0) {
				prev = carry_rows;
			}
			int tiles = (g < p.num_groups) ? (c - prev + BN - 1) / BN : 0;
			#pragma unroll
			for (int off = 1; off < 64; off <<= 1) {
				int up = __shfl_up(tiles, off, 64);
				if (lane >= off) {
					tiles += up;
				}
			}
			total_n_tiles += __shfl(tiles, 63, 64);
			carry_rows = __shfl(c, min(63, p.num_groups - base - 1), 64);
		}
		total_n_tiles = __builtin_amdgcn_readfirstlane((int) total_n_tiles);
		const long total = total_n_tiles * tiles_m;
		const long id = xcd_remap(blockIdx.x, total);
		if (id >= total) {
			return false;
		}
		const int nt = (int) (id / tiles_m);
		const int tm = (int) (id % tiles_m);
		int found_g = 0, found_prev = 0, found_rows = 0, found_nt = 0;
		int tiles_before = 0;
		carry_rows = 0;
		for (int base = 0; base < p.num_groups; base += 64) {
			const int g = base + lane;
			const int c = (g < p.num_groups) ? p.cumsum[g] : 0;
			int prev = __shfl_up(c, 1, 64);
			if (lane == 0) {
				prev = carry_rows;
			}
			const int mine = (g < p.num_groups) ? (c - prev + BN - 1) / BN : 0;
			int incl = mine;
			#pragma unroll
			for (int off = 1; off < 64; off <<= 1) {
				int up = __shfl_up(incl, off, 64);
				if (lane >= off) {
					incl += up;
				}
			}
			const uint64_t past = __ballot((g < p.num_groups) && (tiles_before + incl > nt));
			if (past) {
				const int src = __ffsll((long long) past) - 1;
				found_g = base + src;
				found_prev = __shfl(prev, src, 64);
				found_rows = __shfl(c - prev, src, 64);
				found_nt = nt - (tiles_before + __shfl(incl - mine, src, 64));
				break;
			}
			tiles_before += __shfl(incl, 63, 64);
			carry_rows = __shfl(c, min(63, p.num_groups - base - 1), 64);
		}
		found_g = __builtin_amdgcn_readfirstlane(found_g);
		found_prev = __builtin_amdgcn_readfirstlane(found_prev);
		found_rows = __builtin_amdgcn_readfirstlane(found_rows);
		found_nt = __builtin_amdgcn_readfirstlane(found_nt);
		t.P = p.A + (long long) found_g * p.strideA;
		t.Q = p.gather ? p.B : p.B + (long long) found_prev * p.K;
		t.Qmap = p.gather ? p.gather + found_prev : nullptr;
		t.Pmap = nullptr;
		t.C = p.C ? p.C + (long long) found_prev * p.M : nullptr;
		t.D = p.D + (long long) found_prev * p.M;
		t.M = p.M; t.N = found_rows; t.K = p.K;
		t.m0 = tm * BM;
		t.n0 = found_nt * BN;
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
	t.P = p.gather ? p.A : p.A + (long long) lo * p.M;
	t.Pmap = p.gather ? p.gather + lo : nullptr;
	t.Q = p.B + (long long) lo * p.N;
	t.Qmap = nullptr;
	t.C = p.C ? p.C + (long long) g * p.strideD : nullptr;
	t.D = p.D + (long long) g * p.strideD;
	t.M = p.M; t.N = p.N; t.K = hi - lo;
	t.m0 = (int) (r % tiles_m) * BM;
	t.n0 = (int) (r / tiles_m) * BN;
	return true;
}

/* Accumulator layout of v_mfma_f32_16x16x32_bf16, for block (i, j) of a wave tile (TM x TN blocks of 16 x 16):
 * lane holds n = 16 j + lane % 16 and m = 16 i + 4 * (lane / 16) + {0, 1, 2, 3}. */

/* D = alpha*acc + beta*C, bf16, for the accumulators of one wave */
template <int TM, int TN>
__device__ __forceinline__ void store_accumulators(const Tile & t, const GemmParams & p, f32x4_t (&acc)[TM][TN], int wm, int wn, int lane) {
	const bool use_c = (t.C != nullptr) && (p.beta != 0.0f);
	const bool m_vec = ((t.M & 3) == 0) && ((((uintptr_t) t.D) & 7) == 0) && (!use_c || ((((uintptr_t) t.C) & 7) == 0));
	#pragma unroll
	for (int j = 0; j < TN; j++) {
		const int n = t.n0 + wn + j * 16 + (lane & 15);
		if (n >= t.N) {
			continue;
		}
		#pragma unroll
		for (int i = 0; i < TM; i++) {
			const int m = t.m0 + wm + i * 16 + ((lane >> 4) << 2);
			if (m >= t.M) {
				continue;
			}
			float v[4];
			#pragma unroll
			for (int e = 0; e < 4; e++) {
				v[e] = p.alpha * acc[i][j][e];
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
				o.x = pack2_bf16(v[0], v[1]);
				o.y = pack2_bf16(v[2], v[3]);
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

/* fp32 partial sums of one split of K, straight from the accumulator layout (16 bytes per lane and store) */
template <int TM, int TN>
__device__ __forceinline__ void store_partial(const Tile & t, float * dst, f32x4_t (&acc)[TM][TN], int wm, int wn, int lane) {
	const bool m_vec = ((t.M & 3) == 0) && ((((uintptr_t) dst) & 15) == 0);
	#pragma unroll
	for (int j = 0; j < TN; j++) {
		const int n = t.n0 + wn + j * 16 + (lane & 15);
		if (n >= t.N) {
			continue;
		}
		#pragma unroll
		for (int i = 0; i < TM; i++) {
			const int m = t.m0 + wm + i * 16 + ((lane >> 4) << 2);
			const long long off = (long long) n * t.M + m;
			if (m_vec && m + 4 <= t.M) {
				*((f32x4_t *) (dst + off)) = acc[i][j];
			} else {
				#pragma unroll
				for (int e = 0; e < 4; e++) {
					if (m + e < t.M) {
						dst[off + e] = acc[i][j][e];
					}
				}
			}
		}
	}
}

/* D = bf16(alpha * sum over splits of partial + beta * C); one element per thread and step, neighbours coalesce */
__global__ void __launch_bounds__(256) splitk_reduce_kernel(const float * __restrict__ partial, int splits, long long count,
															  float alpha, float beta, const bf16_t * C, bf16_t * D) {
	const long long stride = (long long) gridDim.x * blockDim.x;
	for (long long i = (long long) blockIdx.x * blockDim.x + threadIdx.x; i < count; i += stride) {
		float sum = 0.0f;
		for (int s = 0; s < splits; s++) {
			sum += partial[(long long) s * count + i];
		}
		float r = alpha * sum;
		if (C != nullptr && beta != 0.0f) {
			r = __builtin_fmaf(beta, bf2f(C[i]), r);
		}
		D[i] = (bf16_t) f2bf(r);
	}
}

/* The same result written through LDS so that global accesses are whole 128-byte lines: each wave stages 16 output
 * rows (n) x WTM columns (m) of fp32 at a time (one row of 16 x 16 blocks) in its own LDS scratch, then every lane
 * fetches 8 consecutive m of one row, applies alpha / beta*C and stores 16 bytes; the lanes of a row cover it
 * contiguously.  The direct epilogue above issues 8-byte pieces to 16 different rows per instruction, which is bound
 * by the number of L2 requests, not by bytes.  Row pitch WTM+4 floats keeps both the 16-byte writes (one row per lane)
 * and the reads (WTM/8 lanes per row) free of bank conflicts.
 * Needs M % 8 == 0 and 16-byte aligned C / D; `scratch` is STAGED_EPILOGUE_FLOATS(WTM) floats per wave. */
#define STAGED_EPILOGUE_FLOATS(wtm) (16 * ((wtm) + 4))
template <int TM, int TN>
__device__ __forceinline__ void store_accumulators_staged(const Tile & t, const GemmParams & p, f32x4_t (&acc)[TM][TN],
														  int wm, int wn, int lane, float * scratch) {
	constexpr int WTM = TM * 16;
	constexpr int PITCH = WTM + 4;
	constexpr int LANES_PER_ROW = WTM / 8;
	constexpr int ROWS_PER_STEP = 64 / LANES_PER_ROW;
	static_assert(16 % ROWS_PER_STEP == 0, "the lanes of a wave must cover whole rows of the staged block");
	const bool use_c = (t.C != nullptr) && (p.beta != 0.0f);
	#pragma unroll
	for (int j = 0; j < TN; j++) {
		const int n_first = t.n0 + wn + j * 16;
		if (n_first >= t.N) {
			break;                                         /* wave-uniform: rows only grow with j */
		}
		#pragma unroll
		for (int i = 0; i < TM; i++) {
			*((f32x4_t *) (scratch + (lane & 15) * PITCH + i * 16 + ((lane >> 4) << 2))) = p.alpha * acc[i][j];
		}
		__builtin_amdgcn_wave_barrier();
		#pragma unroll
		for (int r = 0; r < 16 / ROWS_PER_STEP; r++) {
			const int row = r * ROWS_PER_STEP + lane / LANES_PER_ROW;
			const int c = lane % LANES_PER_ROW;
			const f32x4_t lo = *((const f32x4_t *) (scratch + row * PITCH + c * 8));
			const f32x4_t hi = *((const f32x4_t *) (scratch + row * PITCH + c * 8 + 4));
			const int n = n_first + row;
			const int m = t.m0 + wm + c * 8;
			if (n < t.N && m < t.M) {
				float v[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
				const long long off = (long long) n * t.M + m;
				if (use_c) {
					const u32x4 cv = *((const u32x4 *) (t.C + off));
					const uint32_t cw[4] = {cv.x, cv.y, cv.z, cv.w};
					#pragma unroll
					for (int e = 0; e < 4; e++) {
						v[2 * e] = __builtin_fmaf(p.beta, bf2f(cw[e] & 0xffffu), v[2 * e]);
						v[2 * e + 1] = __builtin_fmaf(p.beta, bf2f(cw[e] >> 16), v[2 * e + 1]);
					}
				}
				u32x4 o;
				o.x = pack2_bf16(v[0], v[1]);
				o.y = pack2_bf16(v[2], v[3]);
				o.z = pack2_bf16(v[4], v[5]);
				o.w = pack2_bf16(v[6], v[7]);
				*((u32x4 *) (t.D + off)) = o;
			}
		}
		__builtin_amdgcn_wave_barrier();
	}
}

/* Epilogue of the streaming kernel for a 64 (m) x 128 (n) wave tile (4 x 8 blocks): the same line-coalesced write as
 * above, through 4 KiB of LDS per wave with XOR swizzles instead of row padding, in as few dependent steps as possible.
 *   No C operand: the accumulators are converted to bf16 first and staged 32 rows (n) x 64 (m) at a time (two rows of
 *   blocks) -- a row is 128 bytes; the 16-byte chunk c of row r sits at chunk c ^ ((r >> 1) & 7).  The four passes are
 *   software-pipelined: pass p+1 is converted and written to LDS while the reads of pass p are in flight (the LDS
 *   executes a wave's instructions in order, so re-using the same 4 KiB needs no wait).
 *   With C (beta != 0): fp32 staging, 16 rows x 64 at a time (one row of blocks), a row is 256 bytes with the 16-byte
 *   chunk c at c ^ row.
 * Stores are non-temporal: the output is not read again by this kernel and should not displace the operand panels
 * from the L2.  `before_stores` runs once, after the first LDS traffic is issued and before the first global store.
 * Needs M % 8 == 0 and 16-byte aligned C / D. */
template <int TM, int TN, int BPP, typename F>
__device__ __forceinline__ void store_tile_swizzled(const Tile & t, const GemmParams & p, f32x4_t (&acc)[TM][TN], int wm, int wn,
													int lane, void * scratch, F before_stores) {
	static_assert(TM == 4 && (BPP == 1 || BPP == 2) && TN % BPP == 0, "written for a 64-wide (m) wave tile, one or two 16-row blocks a pass");
	const bool use_c = (t.C != nullptr) && (p.beta != 0.0f);
	char * const sb = (char *) scratch;
	const int col = lane & 15;                        /* the n this lane holds inside a block */
	const int g = lane >> 4;                          /* its group of four m */
	const int m_lane = t.m0 + wm + ((lane & 7) << 3); /* first of the 8 consecutive m this lane stores */
	const bool m_ok = m_lane < t.M;
	if (!use_c) {
		constexpr int PASSES = TN / BPP;
		constexpr int PASS_ROWS = 16 * BPP;
		/* the lane's 8 bytes of block (i, jj) of a pass: row 16 jj + col, m = 16 i + 4 g -> chunk 2 i + (g >> 1), half g & 1 */
#define EPI_WRITE_BF16(pp) do { \
			_Pragma("unroll") \
			for (int jj = 0; jj < BPP; jj++) { \
				const int row_ = jj * 16 + col; \
				_Pragma("unroll") \
				for (int i = 0; i < TM; i++) { \
					u32x2 v_; \
					v_.x = pack2_bf16(p.alpha * acc[i][BPP * (pp) + jj][0], p.alpha * acc[i][BPP * (pp) + jj][1]); \
					v_.y = pack2_bf16(p.alpha * acc[i][BPP * (pp) + jj][2], p.alpha * acc[i][BPP * (pp) + jj][3]); \
					*((u32x2 *) (sb + row_ * 128 + (((2 * i + (g >> 1)) ^ ((row_ >> 1) & 7)) << 4) + ((g & 1) << 3))) = v_; \
				} \
			} \
		} while (0)
#define EPI_READ_BF16(dst) do { \
			_Pragma("unroll") \
			for (int r = 0; r < 2 * BPP; r++) { \
				const int row_ = r * 8 + (lane >> 3); \
				dst[r] = *((const u32x4 *) (sb + row_ * 128 + (((lane & 7) ^ ((row_ >> 1) & 7)) << 4))); \
			} \
		} while (0)
#define EPI_STORE_BF16(pp, src) do { \
			_Pragma("unroll") \
			for (int r = 0; r < 2 * BPP; r++) { \
				const int n_ = t.n0 + wn + (pp) * PASS_ROWS + r * 8 + (lane >> 3); \
				if (n_ < t.N && m_ok) { \
					__builtin_nontemporal_store(src[r], (u32x4 *) (t.D + (long long) n_ * t.M + m_lane)); \
				} \
			} \
		} while (0)
		u32x4 ra[2 * BPP], rb[2 * BPP];
		EPI_WRITE_BF16(0);
		__builtin_amdgcn_wave_barrier();
		EPI_READ_BF16(ra);
		__builtin_amdgcn_wave_barrier();
		before_stores();
		if (PASSES > 1 && t.n0 + wn + PASS_ROWS < t.N) {
			EPI_WRITE_BF16(1);
			__builtin_amdgcn_wave_barrier();
		}
		EPI_STORE_BF16(0, ra);
		#pragma unroll
		for (int pp = 1; pp < PASSES; pp++) {
			if (t.n0 + wn + pp * PASS_ROWS >= t.N) {
				break;                                     /* wave-uniform: rows only grow with the pass */
			}
			EPI_READ_BF16(rb);
			__builtin_amdgcn_wave_barrier();
			if (pp + 1 < PASSES && t.n0 + wn + (pp + 1) * PASS_ROWS < t.N) {
				EPI_WRITE_BF16(pp + 1);
				__builtin_amdgcn_wave_barrier();
			}
			EPI_STORE_BF16(pp, rb);
		}
#undef EPI_WRITE_BF16
#undef EPI_READ_BF16
#undef EPI_STORE_BF16
		return;
	}
	/* the path with a C operand stages 16 rows of fp32: it exists in the two-block form only (4 KiB of scratch) */
	if constexpr (BPP == 2) {
	/* C is read four passes ahead of its use (a pass is 16 rows: two 16-byte loads per lane), so the latency of
	 * the loads overlaps the LDS traffic of the passes in between instead of adding up pass after pass */
	constexpr int PASSES = TN;
	constexpr int AHEAD = 4;
	u32x4 cbuf[AHEAD][2];
#define EPI_LOAD_C(pp) do { \
		_Pragma("unroll") \
		for (int st = 0; st < 2; st++) { \
			const int n_ = t.n0 + wn + (pp) * 16 + st * 8 + (lane >> 3); \
			cbuf[(pp) % AHEAD][st] = (n_ < t.N && m_ok) ? __builtin_nontemporal_load((const u32x4 *) (t.C + (long long) n_ * t.M + m_lane)) : u32x4{0u, 0u, 0u, 0u}; \
		} \
	} while (0)
	#pragma unroll
	for (int pp = 0; pp < AHEAD && pp < PASSES; pp++) {
		EPI_LOAD_C(pp);
	}
	bool first = true;
	#pragma unroll
	for (int pp = 0; pp < PASSES; pp++) {
		if (t.n0 + wn + pp * 16 >= t.N) {
			break;                                         /* wave-uniform: rows only grow with the pass */
		}
		/* row col of the pass, the four floats at m = 16 i + 4 g: chunk 4 i + g */
		#pragma unroll
		for (int i = 0; i < TM; i++) {
			*((f32x4_t *) (sb + col * 256 + (((4 * i + g) ^ col) << 4))) = p.alpha * acc[i][pp];
		}
		__builtin_amdgcn_wave_barrier();
		if (first) {
			before_stores();
			first = false;
		}
		#pragma unroll
		for (int st = 0; st < 2; st++) {
			const int rr = st * 8 + (lane >> 3);
			const int u = lane & 7;
			const f32x4_t lo = *((const f32x4_t *) (sb + rr * 256 + (((2 * u) ^ rr) << 4)));
			const f32x4_t hi = *((const f32x4_t *) (sb + rr * 256 + (((2 * u + 1) ^ rr) << 4)));
			const int n = t.n0 + wn + pp * 16 + rr;
			if (n < t.N && m_ok) {
				const long long off = (long long) n * t.M + m_lane;
				const u32x4 cv = cbuf[pp % AHEAD][st];
				u32x4 o;
				o.x = pack2_bf16(__builtin_fmaf(p.beta, bf2f(cv.x & 0xffffu), lo.x), __builtin_fmaf(p.beta, bf2f(cv.x >> 16), lo.y));
				o.y = pack2_bf16(__builtin_fmaf(p.beta, bf2f(cv.y & 0xffffu), lo.z), __builtin_fmaf(p.beta, bf2f(cv.y >> 16), lo.w));
				o.z = pack2_bf16(__builtin_fmaf(p.beta, bf2f(cv.z & 0xffffu), hi.x), __builtin_fmaf(p.beta, bf2f(cv.z >> 16), hi.y));
				o.w = pack2_bf16(__builtin_fmaf(p.beta, bf2f(cv.w & 0xffffu), hi.z), __builtin_fmaf(p.beta, bf2f(cv.w >> 16), hi.w));
				__builtin_nontemporal_store(o, (u32x4 *) (t.D + off));
			}
		}
		__builtin_amdgcn_wave_barrier();
		if (pp + AHEAD < PASSES) {
			EPI_LOAD_C(pp + AHEAD);
		}
	}
#undef EPI_LOAD_C
	}
}

/* picks the line-coalesced epilogue when alignment allows it; each wave has STAGED_EPILOGUE_FLOATS of scratch at lds_base */
template <int TM, int TN>
__device__ __forceinline__ void write_tile(const Tile & t, const GemmParams & p, f32x4_t (&acc)[TM][TN], int wm, int wn, int lane,
										   int wave, void * lds_base) {
	const bool use_c = (t.C != nullptr) && (p.beta != 0.0f);
	const bool ok = ((t.M & 7) == 0) && ((((uintptr_t) t.D) & 15) == 0) && (!use_c || ((((uintptr_t) t.C) & 15) == 0));
	if (ok) {
		float * scratch = (float *) lds_base + wave * STAGED_EPILOGUE_FLOATS(TM * 16);
		store_accumulators_staged<TM, TN>(t, p, acc, wm, wn, lane, scratch);
	} else {
		store_accumulators<TM, TN>(t, p, acc, wm, wn, lane);
	}
}

/* ============================================================================================
 * fast path: direct-to-LDS loads
 * ============================================================================================ */

typedef int i32x4 __attribute__((ext_vector_type(4)));

/* raw buffer descriptor (stride 0) over `bytes` bytes at `base`, in scalar registers */
__device__ __forceinline__ i32x4 make_raw_rsrc(const void * base, uint32_t bytes) {
	const uint64_t a = (uint64_t) base;
	i32x4 r;
	r.x = __builtin_amdgcn_readfirstlane((int) (uint32_t) a);
	r.y = __builtin_amdgcn_readfirstlane((int) (uint32_t) ((a >> 32) & 0xffffu));
	r.z = __builtin_amdgcn_readfirstlane((int) bytes);
	r.w = 0x00020000;
	return r;
}

/* One 16-byte-per-lane load from a buffer straight into LDS: lane l's data lands at lds_addr + 16*l.
 * Written as inline assembly so the loads are invisible to the compiler's wait-count bookkeeping: it would
 * otherwise drain every outstanding load (vmcnt(0)) before the first LDS read that follows, which defeats the
 * prefetch.  The kernel places its own s_waitcnt vmcnt before the barrier that publishes a stage, and issues no
 * other vector-memory loads until it has drained them (WAIT_VMCNT(0) ahead of the epilogue). */
__device__ __forceinline__ void dma_load16(uint32_t voff, i32x4 rsrc, uint32_t lds_addr) {
	asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" : : "s"(lds_addr), "v"(voff), "s"(rsrc) : "memory", "m0");
}

/* s_waitcnt vmcnt(n) with the other counters left alone (gfx9 encoding: vmcnt in bits 3:0 and 15:14) */
#define WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | 0x0F70)

#define VOFF_INVALID 0xFFFFFFFFu

/* k-major LDS tile ([64 k][ROWS]): the 16-byte chunk (8 rows) c of k-row k sits at chunk c ^ kmajor_swizzle(k).  A
 * fragment read takes, per 16-lane group, 32 bytes (16 rows) of each of four consecutive k-rows, and the groups that
 * are served together read k-rows 8 apart: bits 0-1 of k spread the four k-rows of a group over the banks, bit 3 the
 * two groups. */
__device__ __forceinline__ int kmajor_swizzle(int k) {
	return ((k & 3) << 2) ^ (((k >> 3) & 1) << 1);
}

/* Loads one operand panel (ROWS rows of the operand, all of K) k-tile by k-tile into its LDS tile layout.
 *
 * Addressing is 64-bit where sizes are not bounded by a tile: the buffer descriptor of k-tile kt starts at the
 * panel's own first element advanced by kt k-tiles, and covers what is left of the operand from there (clamped to
 * the 32 bits a descriptor can express).  Per-lane offsets then only span one k-tile of one panel
 * (lane_voff + i * step, with the second term wave-uniform), so an operand -- or one group of a ragged operand -- can
 * have any size; only K itself is bounded (K <= 2^22, checked on the host), so that ROWS rows of K elements stay
 * below 4 GiB.
 *
 * k-contiguous operand ([rows_total][K] in memory, [ROWS][64] in LDS): LDS chunk id -> (row = id/8, slot = id%8)
 *   holds global chunk slot ^ ((row >> 1) & 7) of that row.  Consecutive loads of a lane are THREADS/8 rows apart.
 *   Rows past rows_total fall behind the end of the buffer and read as zero; the k tail needs a check.
 * k-major operand ([K][rows_total] in memory, [64][ROWS] in LDS): LDS chunk id -> (k = id/(ROWS/8), slot)
 *   holds global row-chunk slot ^ kmajor_swizzle(k) of that k.  Consecutive loads are THREADS/(ROWS/8) k apart: 8 (the
 *   swizzle then alternates between a lane's even and odd loads, which are two chunks apart in the row) or 16.
 *   k past K falls behind the end of the buffer; rows past rows_total need a check (fixed per lane).
 * A lane whose chunk is not valid loads from offset 0xFFFFFFFF, which is out of range of any descriptor.

 * GATHER, k-contiguous: the panel's rows are scattered over a source array, row r of the panel at source row
 *   map[r]; every load of a lane then has its own offset from the source's first element (a lane's loads are
 *   THREADS/8 rows apart, PER_THREAD of them per k-tile), the same for every k-tile but for the k advance.
 * GATHER, k-major: the k-rows are scattered, k-row k of the operand at source row map[k].  Lane l of a wave keeps
 *   map[64 kt + l] for the k-tile it is about to load (fetched one k-tile ahead, behind the loads of the k-tile
 *   before, so that its latency overlaps the multiplies) and every load takes its k-row's entry from the lane that
 *   holds it. */
template <bool KMAJOR, int ROWS, int THREADS, bool GATHER = false>
struct TileLoader {
	static constexpr int CHUNKS = ROWS * CHUNKS_PER_ROW;
	static constexpr int PER_THREAD = CHUNKS / THREADS;
	static_assert(CHUNKS % THREADS == 0, "tile must split evenly over the work-group");
	static constexpr int KSTEP = THREADS / (ROWS / 8);       /* k-major: k-rows between consecutive loads of a lane */
	static_assert(!KMAJOR || KSTEP == 8 || KSTEP % 16 == 0, "k-major swizzle needs a k step of 8 or a multiple of 16");
	static_assert(KMAJOR || ((THREADS / 8) % 16 == 0), "k-contiguous swizzle needs the row step to be a multiple of 16");

	uint32_t lane_voff;      /* VGPR: this lane's first chunk inside a k-tile of the panel */
	uint32_t step;           /* uniform: bytes between consecutive loads of a lane */
	uint64_t ktile;          /* uniform: bytes between consecutive k-tiles of the panel */
	uint64_t base;           /* uniform: address of the panel's first element */
	uint64_t extent;         /* uniform: bytes from there to the end of the operand */
	int kchunk;              /* k-contiguous only: first k (within the tile) of this lane's chunk */
	bool lane_ok;            /* k-major only: this lane's rows exist */
	bool lane_ok_odd;        /* k-major with a k step of 8: the same for the lane's odd loads */
	uint32_t odd_delta;      /* k-major with a k step of 8: bytes from an even load's chunk to the odd loads' chunk (+-32) */
	uint32_t gather_voff[(GATHER && !KMAJOR) ? PER_THREAD : 1];   /* VGPRs, k-contiguous GATHER: offset of each of this lane's chunks */
	const int * kmap;        /* uniform, k-major GATHER: source row of every k-row of the operand */
	int kmap_val;            /* VGPR, k-major GATHER: kmap[64 * kmap_kt + lane] */
	int kmap_kt;             /* uniform */
	uint32_t row_bytes;      /* uniform, k-major GATHER: bytes of one source row */
	uint32_t kmap_rows;      /* uniform, k-major GATHER: rows of the source */

	/* `operand`: first element of the operand (of this group); row0: first of the panel's rows; row0 < rows_total */
	__device__ __forceinline__ void init(const bf16_t * operand, int row0, int rows_total, int K) {
		const int tid = threadIdx.x % THREADS;
		if (!KMAJOR) {
			const int row = tid >> 3;
			const int c = (tid & 7) ^ ((row >> 1) & 7);
			kchunk = c << 3;
			lane_ok = true;
			lane_ok_odd = true;
			odd_delta = 0;
			base = (uint64_t) (operand + (uint64_t) row0 * (uint64_t) K);
			extent = (uint64_t) (rows_total - row0) * (uint64_t) K * 2u;
			lane_voff = ((uint32_t) row * (uint32_t) K + (uint32_t) kchunk) * 2u;
			step = (uint32_t) (THREADS / 8) * (uint32_t) K * 2u;
			ktile = BK * 2u;
		} else {
			constexpr int CPR = ROWS / 8;
			const int k = tid / CPR;
			const int mc = (tid % CPR) ^ kmajor_swizzle(k);
			const int mc_odd = (tid % CPR) ^ kmajor_swizzle(k + KSTEP);
			kchunk = 0;
			lane_ok = row0 + (mc << 3) < rows_total;
			lane_ok_odd = row0 + (mc_odd << 3) < rows_total;
			odd_delta = (uint32_t) ((mc_odd - mc) * 16);
			base = (uint64_t) (operand + row0);
			extent = (uint64_t) K * (uint64_t) rows_total * 2u - (uint64_t) row0 * 2u;
			lane_voff = ((uint32_t) k * (uint32_t) rows_total + (uint32_t) (mc << 3)) * 2u;
			step = (uint32_t) (THREADS / CPR) * (uint32_t) rows_total * 2u;
			ktile = (uint64_t) BK * (uint64_t) rows_total * 2u;
		}
	}

	/* GATHER: `source` has source_rows rows of K elements (below 4 GiB in all); map[r] is the source row of the panel's
	 * row r, for row0 <= r < rows_total */
	__device__ __forceinline__ void init_gather(const bf16_t * source, const int * map, int row0, int rows_total, int K, int source_rows) {
		const int tid = threadIdx.x % THREADS;
		const int row = tid >> 3;
		const int c = (tid & 7) ^ ((row >> 1) & 7);
		kchunk = c << 3;
		lane_ok = true;
		lane_ok_odd = true;
		odd_delta = 0;
		base = (uint64_t) source;
		extent = (uint64_t) source_rows * (uint64_t) K * 2u;
		lane_voff = 0;
		step = 0;
		ktile = BK * 2u;
		#pragma unroll
		for (int i = 0; i < ((GATHER && !KMAJOR) ? PER_THREAD : 1); i++) {
			const int r = row0 + row + i * (THREADS / 8);
			/* a map entry outside the source (negative, stale) reads zeros, like a row past the panel's end */
			const uint32_t src = r < rows_total ? (uint32_t) map[r] : 0xFFFFFFFFu;
			gather_voff[i] = src < (uint32_t) source_rows ? (src * (uint32_t) K + (uint32_t) kchunk) * 2u : VOFF_INVALID;
		}
	}

	__device__ __forceinline__ void fetch_kmap(int kt, int K) {
		/* an entry outside the source (negative, stale) becomes the row one past its end: out of the buffer, zeros */
		kmap_val = (int) min((uint32_t) kmap[min(kt * BK + (int) (threadIdx.x & 63), K - 1)], kmap_rows);
		kmap_kt = kt;
	}

	/* k-major GATHER: `source` has source_rows rows of rows_total elements (below 4 GiB in all); map[k] is the source
	 * row of the operand's k-row k, 0 <= k < K, K >= 1 */
	__device__ __forceinline__ void init_gather_k(const bf16_t * source, const int * map, int row0, int rows_total, int K, int source_rows,
													bool have_first = false, int first = 0) {
		constexpr int CPR = ROWS / 8;
		const int tid = threadIdx.x % THREADS;
		const int k = tid / CPR;
		const int mc = (tid % CPR) ^ kmajor_swizzle(k);
		const int mc_odd = (tid % CPR) ^ kmajor_swizzle(k + KSTEP);
		kchunk = 0;
		lane_ok = row0 + (mc << 3) < rows_total;
		lane_ok_odd = row0 + (mc_odd << 3) < rows_total;
		odd_delta = (uint32_t) ((mc_odd - mc) * 16);
		base = (uint64_t) (source + row0);
		extent = (uint64_t) source_rows * (uint64_t) rows_total * 2u - (uint64_t) row0 * 2u;
		lane_voff = (uint32_t) (mc << 3) * 2u;
		step = 0;
		ktile = 0;
		row_bytes = (uint32_t) rows_total * 2u;
		kmap = map;
		kmap_rows = (uint32_t) source_rows;
		if (have_first) {
			kmap_val = (int) min((uint32_t) first, kmap_rows);   /* map[min(lane, K - 1)], fetched ahead by the caller */
			kmap_kt = 0;
		} else {
			fetch_kmap(0, K);
		}
	}

	/* `tile_addr`: LDS byte address of the tile; `wave`: wave index among the loading waves (uniform) */
	__device__ __forceinline__ void issue(uint32_t tile_addr, int kt, int K, int wave, bool live = true) {
		if (GATHER && KMAJOR) {
			constexpr int CPR = ROWS / 8;
			const int k_lane = (int) (threadIdx.x % THREADS) / CPR;       /* this lane's k-row inside the k-tile, first load */
			if (live && kmap_kt != kt) {
				fetch_kmap(kt, K);
			}
			const i32x4 rsrc = make_raw_rsrc((const void *) base, extent > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t) extent);
			#pragma unroll
			for (int i = 0; i < PER_THREAD; i++) {
				const int k_in = k_lane + i * (THREADS / CPR);
				const uint32_t src = (uint32_t) __builtin_amdgcn_ds_bpermute(k_in << 2, kmap_val);
				const bool ok = live && ((i & 1) ? lane_ok_odd : lane_ok) && (kt * BK + k_in < K);
				const uint32_t voff = ok ? src * row_bytes + lane_voff + ((i & 1) ? odd_delta : 0u) : VOFF_INVALID;
				dma_load16(voff, rsrc, tile_addr + (uint32_t) (i * THREADS + wave * 64) * 16u);
			}
			if (live && (kt + 1) * BK < K) {
				fetch_kmap(kt + 1, K);
			}
			return;
		}
		/* k-contiguous: chunks that start at or past K exist only in the last k-tile; `live` false: nothing to load,
		 * every lane reads out of range (zeros) */
		const bool ok = live && (KMAJOR ? (kt * BK < K) : (kt * BK + kchunk < K));
		const uint64_t advance = (uint64_t) kt * ktile;
		const uint64_t left = extent > advance ? extent - advance : 0;
		const i32x4 rsrc = make_raw_rsrc((const void *) (base + advance), left > 0xFFFFFFFFull ? 0xFFFFFFFFu : (uint32_t) left);
		#pragma unroll
		for (int i = 0; i < PER_THREAD; i++) {
			const bool ok_i = ok && (!KMAJOR || ((i & 1) ? lane_ok_odd : lane_ok));
			const uint32_t voff = ok_i ? ((GATHER && !KMAJOR) ? gather_voff[i] : lane_voff + (uint32_t) i * step + ((KMAJOR && (i & 1)) ? odd_delta : 0u))
									   : VOFF_INVALID;
			dma_load16(voff, rsrc, tile_addr + (uint32_t) (i * THREADS + wave * 64) * 16u);
		}
	}
};

/* MFMA operand of one lane for v_mfma_f32_16x16x32_bf16: rows [row_base, row_base+16) x k [32s, 32s+32) of the tile;
 * lane l holds row l % 16 and the eight k from 32s + 8 * (l / 16) on */
template <bool KMAJOR, int ROWS>
__device__ __forceinline__ bf16x8 read_fragment(const bf16_t * tile, int row_base, int s, int lane) {
	if (!KMAJOR) {
		const int row = row_base + (lane & 15);
		return *((const bf16x8 *) (tile + lds_chunk_off(row, 4 * s + (lane >> 4))));
	} else {
		/* each 16-lane group loads a 4(k) x 16(row) block, 8 bytes per lane, and gets it back transposed:
		 * lane j of the group receives row j's elements of the 4 consecutive k */
		const int lg = lane & 15;
		const int r0 = row_base + ((lg & 3) << 2);
		const int k_lo = 32 * s + ((lane >> 4) << 3) + (lg >> 2), k_hi = k_lo + 4;
		s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *) LDS_PTR(tile + k_lo * ROWS + (r0 ^ (kmajor_swizzle(k_lo) << 3))));
		s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) s16x4 *) LDS_PTR(tile + k_hi * ROWS + (r0 ^ (kmajor_swizzle(k_hi) << 3))));
		s16x8 both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
		return __builtin_bit_cast(bf16x8, both);
	}
}

/* STAGES: 2, or 4 for the launches that split K over otherwise idle compute units (few tiles, the router's GEMMs): those
 * are short streams of operand bytes with nothing to reuse, and what one k-tile in flight per compute unit fetches in a
 * memory round trip is a third of what HBM delivers; with four stages three k-tiles are in flight.  A split then has to
 * be a multiple of four k-tiles long. */
template <int BM, int BN, int WAVES_M, int WAVES_N, bool P_KMAJOR, bool Q_KMAJOR, int MODE, int GATHER = 0, int STAGES = 2>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_bf16_direct_kernel(GemmParams p) {
	static_assert(STAGES == 2 || STAGES == 4, "two stages, or four");
	constexpr int THREADS = WAVES_M * WAVES_N * 64;
	constexpr int WTM = BM / WAVES_M;
	constexpr int WTN = BN / WAVES_N;
	constexpr int TM = WTM / 16;
	constexpr int TN = WTN / 16;
	constexpr int LOADS_PER_STAGE = (BM + BN) * CHUNKS_PER_ROW / THREADS;
	static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be a multiple of the 16x16 MFMA tile");
	static_assert(LOADS_PER_STAGE < 64, "vmcnt is a 6-bit counter");

	/* the pipeline stages; the epilogue reuses the memory as per-wave fp32 scratch */
	__shared__ __attribute__((aligned(16))) bf16_t stages[STAGES][(BM + BN) * BK];
	static_assert(WAVES_M * WAVES_N * STAGED_EPILOGUE_FLOATS(WTM) * 4 <= 2 * (BM + BN) * BK * 2, "epilogue scratch must fit in the stages");
	bf16_t * const stage0 = stages[0];
	bf16_t * const stage1 = stages[1];

	Tile t;
	int kt_begin = 0;
	int split = -1;
	if (MODE == MODE_SINGLE && p.split_k > 1) {
		const long tiles = (long) ((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN);
		split = (int) (blockIdx.x / tiles);
		if (split >= p.split_k || !resolve_tile_id<BM, BN, MODE>(p, blockIdx.x - split * tiles, t)) {
			return;
		}
		kt_begin = split * p.kt_per_split;
	} else if (!resolve_tile<BM, BN, MODE>(p, t)) {
		return;
	}

	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int wm = (wave % WAVES_M) * WTM;
	const int wn = (wave / WAVES_M) * WTN;

	const uint32_t stage0_addr = (uint32_t) (uintptr_t) LDS_PTR(stage0);
	const uint32_t stage1_addr = (uint32_t) (uintptr_t) LDS_PTR(stage1);

	f32x4_t acc[TM][TN];
	#pragma unroll
	for (int i = 0; i < TM; i++) {
		#pragma unroll
		for (int j = 0; j < TN; j++) {
			acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
		}
	}

	/* a split of K is an even number of k-tiles, so the stage that the loop multiplies beyond an odd count only
	 * ever holds k-tiles past K (zeros), never the next split's */
	int k_tiles = (t.K + BK - 1) / BK;
	if (split >= 0) {
		k_tiles = min(k_tiles, kt_begin + p.kt_per_split);
	}

	TileLoader<P_KMAJOR, BM, THREADS, GATHER == GATHER_P_KROWS> ldP;
	TileLoader<Q_KMAJOR, BN, THREADS, GATHER == GATHER_Q_ROWS> ldQ;
	if (GATHER == GATHER_P_KROWS) {
		ldP.init_gather_k(t.P, t.Pmap, t.m0, t.M, t.K, p.gather_rows);
	} else {
		ldP.init(t.P, t.m0, t.M, t.K);
	}
	if (GATHER == GATHER_Q_ROWS) {
		ldQ.init_gather(t.Q, t.Qmap, t.n0, t.N, t.K, p.gather_rows);
	} else {
		ldQ.init(t.Q, t.n0, t.N, t.K);
	}

	/* the descriptors end with the operand of this problem: anything outside reads as zero */
#define ISSUE_STAGE(addr, kt_) do { \
		ldP.issue((addr), (kt_), t.K, wave); \
		ldQ.issue((addr) + BM * BK * 2, (kt_), t.K, wave); \
	} while (0)

	/* multiply one k-tile out of an LDS stage; the compiler interleaves the LDS reads of step s+1 with the MFMAs of step s */
#define COMPUTE_STAGE(buf) do { \
		const bf16_t * cp = (buf); \
		const bf16_t * cq = (buf) + BM * BK; \
		_Pragma("unroll") \
		for (int s = 0; s < BK / 32; s++) { \
			bf16x8 a[TM], b[TN]; \
			_Pragma("unroll") \
			for (int i = 0; i < TM; i++) { a[i] = read_fragment<P_KMAJOR, BM>(cp, wm + i * 16, s, lane); } \
			_Pragma("unroll") \
			for (int j = 0; j < TN; j++) { b[j] = read_fragment<Q_KMAJOR, BN>(cq, wn + j * 16, s, lane); } \
			_Pragma("unroll") \
			for (int i = 0; i < TM; i++) { \
				_Pragma("unroll") \
				for (int j = 0; j < TN; j++) { \
					acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0); \
				} \
			} \
		} \
	} while (0)

	/* One barrier per k-tile.  Iteration kt: wait for this wave's loads of k-tile kt (issued one iteration
	 * earlier), barrier -- after it every wave's share of the tile is in LDS and every wave has finished reading
	 * the other stage -- then immediately start the loads of k-tile kt+1 into that other stage and multiply
	 * k-tile kt.  The loads have the whole multiply phase to land.
	 * Loads past the last k-tile are out of range of the buffer and fill LDS with zeros: an odd tile count
	 * costs one multiply of a zero tile instead of control flow around 256 live accumulators. */
	if constexpr (STAGES == 2) {
		ISSUE_STAGE(stage0_addr, kt_begin);
		for (int kt = kt_begin; kt < k_tiles; kt += 2) {
			WAIT_VMCNT(0);
			__syncthreads();
			ISSUE_STAGE(stage1_addr, kt + 1);
			COMPUTE_STAGE(stage0);
			WAIT_VMCNT(0);
			__syncthreads();
			ISSUE_STAGE(stage0_addr, kt + 2);
			COMPUTE_STAGE(stage1);
		}
	} else {
		/* Iteration for k-tile kt (stage kt mod 4): the loads of kt, kt+1, kt+2 are out; wait until only the two younger
		 * ones are (loads complete in order), barrier -- kt is visible, and nobody reads the stage of kt-1 any more --
		 * start kt+3 into that stage, multiply kt.  The split is a multiple of four k-tiles (or ends with K), so what is
		 * multiplied past its end are k-tiles past K: zeros; the loads that run ahead into the next split's k-tiles are
		 * never multiplied. */
		constexpr uint32_t STAGE_BYTES = (BM + BN) * BK * 2;
		ISSUE_STAGE(stage0_addr, kt_begin);
		ISSUE_STAGE(stage0_addr + STAGE_BYTES, kt_begin + 1);
		ISSUE_STAGE(stage0_addr + 2 * STAGE_BYTES, kt_begin + 2);
		for (int kt = kt_begin; kt < k_tiles; kt += 4) {
			#pragma unroll
			for (int u = 0; u < 4; u++) {
				WAIT_VMCNT(2 * LOADS_PER_STAGE);
				__syncthreads();
				ISSUE_STAGE(stage0_addr + ((u + 3) & 3) * STAGE_BYTES, kt + u + 3);
				COMPUTE_STAGE(stages[u]);
			}
		}
	}
	WAIT_VMCNT(0);                             /* drain the trailing (zero-filling) loads before the LDS is released */
	__syncthreads();
#undef ISSUE_STAGE
#undef COMPUTE_STAGE

	if (split >= 0) {
		store_partial<TM, TN>(t, p.partial + (long long) split * t.M * t.N, acc, wm, wn, lane);
		return;
	}
	write_tile<TM, TN>(t, p, acc, wm, wn, lane, wave, (void *) stages);
}

/* --------------------------------------------------------------------------------------------
 * streaming form: persistent work-groups, operands of every MFMA group in registers one k-step ahead
 *
 * With 128 KiB of LDS in two stages only one work-group fits on a compute unit, so a fresh work-group per tile
 * would pay the launch, the first (unhidden) load round trip and the epilogue serially.  Here the grid is one
 * work-group per compute unit and each walks over many tiles; tiles are dealt so that the 32 compute units of one
 * die work on neighbouring tiles: die x owns tiles [x*chunk, (x+1)*chunk), its work-groups take them round-robin.
 * The direct kernel above meets at a barrier once per k-tile and only then starts reading the fresh stage: for
 * the length of a barrier plus an LDS round trip no wave has operands and the matrix pipes idle.  Here the
 * operands of k-step s+1 are read from LDS while the MFMAs of k-step s run, also from one k-tile to the next, and
 * the one barrier per k-tile sits between the MFMAs of k-steps 2 and 3:
 *
 *     k-tile g of the stream of k-tiles (across output tiles), LDS stage g & 1; F(g,0) is in registers:
 *         F(g,1) <- LDS;  MFMAs on F(g,0)
 *         F(g,2) <- LDS;  MFMAs on F(g,1)
 *         F(g,3) <- LDS;  MFMAs on F(g,2)
 *         wait for this wave's loads of k-tile g+1; barrier
 *             -> k-tile g+1 is visible to all, and nobody reads stage g & 1 any more
 *         loader waves start the loads of k-tile g+2 into stage g & 1 (they have until the next barrier to land,
 *         so they go out first); first MFMAs on F(g,3); F(g+1,0) <- LDS; remaining MFMAs on F(g,3)
 *
 * A load has a whole k-tile of multiplies to land.  Rows of k-contiguous operands are fetched 128 bytes (one
 * cache line) at a time: the L1 of a compute unit tracks a bounded number of lines in flight, so half-line
 * requests would halve the bytes in flight.
 * The stream runs across output tiles: the loader moves on to the next tile of this work-group while the last
 * k-tiles of the current one are multiplied.  Every output tile is given at least two k-tiles (k-tiles past K read
 * as zero), so the loader is never more than one tile ahead; when the tiles run out it issues loads that are out
 * of range (they write zeros to a free stage) to keep the count of outstanding loads uniform.
 * The epilogue has its own LDS scratch (one region per wave): it needs no barrier and never waits for a stage.
 * -------------------------------------------------------------------------------------------- */
template <int BM, int BN, int WAVES_M, int WAVES_N, bool P_KMAJOR, bool Q_KMAJOR, int MODE, int GATHER = 0>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_bf16_stream_kernel(GemmParams p) {
	constexpr int THREADS = WAVES_M * WAVES_N * 64;
	constexpr int WTM = BM / WAVES_M;
	constexpr int WTN = BN / WAVES_N;
	constexpr int TM = WTM / 16;
	constexpr int TN = WTN / 16;
	constexpr int STAGE_ELEMS = (BM + BN) * BK;
	constexpr int BPP = (TN & 1) ? 1 : 2;                  /* 16-row blocks per epilogue pass */
	constexpr int EPI_WAVE_FLOATS = 512 * BPP;             /* 2 or 4 KiB per wave */
	constexpr int EPI_FLOATS = WAVES_M * WAVES_N * EPI_WAVE_FLOATS;
	static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be a multiple of the 16x16 MFMA tile");
	static_assert(STAGE_ELEMS * 4 + EPI_FLOATS * 4 <= 160 * 1024, "two stages and the epilogue scratch must fit in the LDS");

	__shared__ __attribute__((aligned(16))) bf16_t stages[2][STAGE_ELEMS];
	__shared__ __attribute__((aligned(16))) float epilogue_scratch[EPI_FLOATS];

	const int lane = threadIdx.x & 63;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int wm = (wave % WAVES_M) * WTM;
	const int wn = (wave / WAVES_M) * WTN;

	if (MODE == MODE_RAGGED_N && p.arbitrate == ARBITRATE_NARROW && ragged_n_prefers_384(p)) {
		return;                                             /* the 256 x 384 launch behind this one does the work */
	}
	const long total = count_tiles<BM, BN, MODE>(p);
	const long chunk = (total + 7) >> 3;                    /* tiles per die */
	const long die = blockIdx.x & 7;
	const long stride = gridDim.x >> 3;                     /* work-groups per die (the grid is a multiple of 8) */
	long local = blockIdx.x >> 3;

	Tile cur;
	bool have = false;
	for (; local < chunk; local += stride) {
		const long id = die * chunk + local;
		if (id < total && resolve_tile_id<BM, BN, MODE>(p, id, cur)) {
			have = true;
			break;
		}
	}
	if (!have) {
		return;
	}

	const uint32_t stages_addr = (uint32_t) (uintptr_t) LDS_PTR(stages);

	/* the loader: a cursor (tile, k-tile) two k-tiles ahead of the multiplies */
	constexpr int LD_THREADS = THREADS / 2;                 /* the first half of the waves does all the loading */
	TileLoader<P_KMAJOR, BM, LD_THREADS, GATHER == GATHER_P_KROWS> ldP;
	TileLoader<Q_KMAJOR, BN, LD_THREADS, GATHER == GATHER_Q_ROWS> ldQ;
	bool peeked = false;                                    /* gathered k-rows: peek_val holds the next tile's first row-map entries */
	int peek_val = 0;
	/* the waves that never load skip the row-map reads of a gathered operand (their offsets are never used) */
#define ST_INIT_LOADERS(tile_) do { \
		if (GATHER != GATHER_P_KROWS) { \
			ldP.init(tile_.P, tile_.m0, tile_.M, tile_.K); \
		} else if (wave < (WAVES_M * WAVES_N) / 2) { \
			ldP.init_gather_k(tile_.P, tile_.Pmap, tile_.m0, tile_.M, tile_.K, p.gather_rows, peeked, peek_val); \
			peeked = false; \
		} \
		if (GATHER != GATHER_Q_ROWS) { \
			ldQ.init(tile_.Q, tile_.n0, tile_.N, tile_.K); \
		} else if (wave < (WAVES_M * WAVES_N) / 2) { \
			ldQ.init_gather(tile_.Q, tile_.Qmap, tile_.n0, tile_.N, tile_.K, p.gather_rows); \
		} \
	} while (0)
	ST_INIT_LOADERS(cur);
	int ld_K = cur.K;
	int ld_kt = 0;
	int ld_tiles = max(2, (cur.K + BK - 1) / BK);
	bool ld_live = true;
	Tile nxt;
	bool has_next = false;
	uint32_t ld_g = 0;                                      /* k-tiles issued so far; ld_g & 1 is the stage */

	/* Gathered k-rows: the row-map entries of a tile's first k-tile are fetched while the last k-tile of the tile before
	 * is issued, one call ahead of the switch (a tile has at least two k-tiles), so the switch does not wait for them.
	 * The look-ahead resolves the next tile a second time and leaves `nxt` alone: the multiplies may not have taken
	 * it over yet. */
#define ST_PEEK_NEXT() do { \
		if (GATHER == GATHER_P_KROWS && wave < (WAVES_M * WAVES_N) / 2 && ld_live && ld_kt == ld_tiles - 1) { \
			Tile ahead_; \
			for (long l_ = local + stride; l_ < chunk; l_ += stride) { \
				const long id_ = die * chunk + l_; \
				if (id_ < total && resolve_tile_id<BM, BN, MODE>(p, id_, ahead_)) { \
					peek_val = ahead_.Pmap[min(lane, ahead_.K - 1)]; \
					peeked = true; \
					break; \
				} \
			} \
		} \
	} while (0)
#define ST_ISSUE_NEXT() do { \
		ST_PEEK_NEXT(); \
		if (ld_live && ld_kt == ld_tiles) { \
			has_next = false; \
			for (local += stride; local < chunk; local += stride) { \
				const long id_ = die * chunk + local; \
				if (id_ < total && resolve_tile_id<BM, BN, MODE>(p, id_, nxt)) { \
					has_next = true; \
					break; \
				} \
			} \
			ld_live = has_next; \
			if (has_next) { \
				ST_INIT_LOADERS(nxt); \
				ld_K = nxt.K; \
				ld_kt = 0; \
				ld_tiles = max(2, (nxt.K + BK - 1) / BK); \
			} \
		} \
		if (loader) { \
			const uint32_t addr_ = stages_addr + (ld_g & 1u) * (uint32_t) (STAGE_ELEMS * 2); \
			ldP.issue(addr_, ld_kt, ld_K, wave % (LD_THREADS / 64), ld_live); \
			ldQ.issue(addr_ + BM * BK * 2, ld_kt, ld_K, wave % (LD_THREADS / 64), ld_live); \
		} \
		ld_kt++; \
		ld_g++; \
	} while (0)
	/* A k-tile is two k-steps of 32 (one MFMA deep each); a k-step is multiplied in two halves of the wave tile's
	 * columns, TN / 2 blocks each: sub-step (s, h) takes the TM fragments of P for k-step s (read once per k-step) and the
	 * TN / 2 fragments of Q for columns [h * TN / 2, (h + 1) * TN / 2), and issues TM * TN / 2 MFMAs. */
	constexpr int TNH = (TN + 1) / 2;                       /* blocks of the first half; the second has TN - TNH (one less if TN is odd) */
#define ST_HALF(h_) ((h_) ? TN - TNH : TNH)
	static_assert(BK == 64 && TN >= 2, "the schedule below is written for two k-steps of two halves per k-tile");
#define ST_READ_P(fa, g_, s_) do { \
		const bf16_t * sp_ = stages[(g_) & 1u]; \
		_Pragma("unroll") \
		for (int i = 0; i < TM; i++) { fa[i] = read_fragment<P_KMAJOR, BM>(sp_, wm + i * 16, (s_), lane); } \
	} while (0)
#define ST_READ_Q(fb, g_, s_, h_) do { \
		const bf16_t * sq_ = stages[(g_) & 1u] + BM * BK; \
		_Pragma("unroll") \
		for (int j = 0; j < ST_HALF(h_); j++) { fb[j] = read_fragment<Q_KMAJOR, BN>(sq_, wn + ((h_) * TNH + j) * 16, (s_), lane); } \
	} while (0)
	/* the MFMAs of sub-step (., h) on column blocks [j0, j1) of the half */
#define ST_MFMA(fa, fb, h_, j0, j1) do { \
		_Pragma("unroll") \
		for (int j = (j0); j < (j1); j++) { \
			_Pragma("unroll") \
			for (int i = 0; i < TM; i++) { \
				acc[i][(h_) * TNH + j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i][(h_) * TNH + j], 0, 0, 0); \
			} \
		} \
	} while (0)

	/* Order inside a sub-step: the LDS reads of the next sub-step's operands go out two at a time behind the first
	 * MFMAs, so their issue overlaps the matrix pipe and their data has the rest of the sub-step to arrive (left to
	 * itself the compiler sinks the reads to the end and the next sub-step starts by waiting for them). */
	constexpr int READS_P = TM * (P_KMAJOR ? 2 : 1);
#define ST_READS_Q(h_) (ST_HALF(h_) * (Q_KMAJOR ? 2 : 1))
	/* `reads_` LDS reads behind the first of the `mfmas_` MFMAs of a sub-step */
#define ST_INTERLEAVE(reads_, mfmas_) do { \
		_Pragma("unroll") \
		for (int r_ = 0; r_ < ((reads_) + 1) / 2; r_++) { \
			__builtin_amdgcn_sched_group_barrier(0x008, 1, 0); \
			__builtin_amdgcn_sched_group_barrier(0x100, 2, 0); \
		} \
		__builtin_amdgcn_sched_group_barrier(0x008, (mfmas_) - ((reads_) + 1) / 2, 0); \
	} while (0)

	/* The first half of the waves (one per SIMD) issues all loads.  A wave that issues a load while the memory
	 * pipeline of the compute unit is busy waits until the load is accepted and issues no MFMA meanwhile; and of the
	 * two waves that share a SIMD the older one (lower index) wins the matrix pipe whenever both have an MFMA ready.
	 * So the older wave of each SIMD loads the whole k-tile g+2 right after the barrier of k-tile g, and the younger
	 * one, which never loads, has the matrix pipe to itself for that long. */
	const bool loader = wave < (WAVES_M * WAVES_N) / 2;
	/* prologue: the first k-tile landed and visible, its first k-step in registers, one more k-tile in flight */
	ST_ISSUE_NEXT();
	ST_ISSUE_NEXT();
	WAIT_VMCNT((BM + BN) * CHUNKS_PER_ROW / LD_THREADS);
	__syncthreads();
	bf16x8 pa[TM], pb[TM], qa[TNH], qb[TNH];                /* P fragments of k-step 0 / 1, Q fragments of alternating sub-steps */
	uint32_t g = 0;                                         /* k-tiles multiplied so far */
	bool landed = false;                                    /* this wave's loads of the next k-tile are known to be complete */
	ST_READ_P(pa, g, 0);
	ST_READ_Q(qa, g, 0, 0);

	while (true) {
		f32x4_t acc[TM][TN];
		#pragma unroll
		for (int i = 0; i < TM; i++) {
			#pragma unroll
			for (int j = 0; j < TN; j++) {
				acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
			}
		}
		const int k_tiles = max(2, (cur.K + BK - 1) / BK);
		for (int kt = 0; kt < k_tiles; kt++) {
			ST_READ_Q(qb, g, 0, 1);
			ST_MFMA(pa, qa, 0, 0, ST_HALF(0));
			ST_INTERLEAVE(ST_READS_Q(1), TM * ST_HALF(0));
			__builtin_amdgcn_sched_barrier(0);
			ST_READ_P(pb, g, 1);
			ST_READ_Q(qa, g, 1, 0);
			ST_MFMA(pa, qb, 1, 0, ST_HALF(1));
			ST_INTERLEAVE(READS_P + ST_READS_Q(0), TM * ST_HALF(1));
			__builtin_amdgcn_sched_barrier(0);
			ST_READ_Q(qb, g, 1, 1);
			ST_MFMA(pb, qa, 0, 0, ST_HALF(0));
			ST_INTERLEAVE(ST_READS_Q(1), TM * ST_HALF(0));
			__builtin_amdgcn_sched_barrier(0);
			if (!landed) {
				WAIT_VMCNT(0);
			}
			landed = false;
			__syncthreads();
			ST_ISSUE_NEXT();                                /* k-tile g+2 into the stage of k-tile g, free since the barrier */
			__builtin_amdgcn_sched_barrier(0);
			ST_MFMA(pb, qb, 1, 0, 1);
			__builtin_amdgcn_sched_barrier(0);
			ST_READ_P(pa, g + 1, 0);
			ST_READ_Q(qa, g + 1, 0, 0);
			__builtin_amdgcn_sched_barrier(0);
			ST_MFMA(pb, qb, 1, 1, ST_HALF(1));
			g++;
		}
		{
			/* The loads of the next k-tile are waited for here, before the first store, and not at the next barrier:
			 * a wait there would also wait for the stores just issued (one counter covers both). */
			const bool use_c = (cur.C != nullptr) && (p.beta != 0.0f);
			const bool fast = ((cur.M & 7) == 0) && ((((uintptr_t) cur.D) & 15) == 0) && (!use_c || ((((uintptr_t) cur.C) & 15) == 0));
			/* The epilogue's per-lane offsets are derived from a lane id the compiler cannot see through, so that it
			 * computes them here and does not keep them in registers across the k-loop. */
			int lane_e;
			asm volatile("v_mov_b32 %0, %1" : "=v"(lane_e) : "v"(lane));
			if (fast && (BPP == 2 || !use_c)) {
				store_tile_swizzled<TM, TN, BPP>(cur, p, acc, wm, wn, lane_e, (void *) (epilogue_scratch + wave * EPI_WAVE_FLOATS), [&]() { WAIT_VMCNT(0); });
			} else {
				WAIT_VMCNT(0);
				store_accumulators<TM, TN>(cur, p, acc, wm, wn, lane_e);
			}
			landed = true;
		}
		if (!has_next) {
			break;
		}
		cur = nxt;
		has_next = false;
	}
	WAIT_VMCNT(0);
#undef ST_INIT_LOADERS
#undef ST_PEEK_NEXT
#undef ST_ISSUE_NEXT
#undef ST_READ_P
#undef ST_READ_Q
#undef ST_MFMA
#undef ST_INTERLEAVE
#undef ST_HALF
#undef ST_READS_Q
}

/* ============================================================================================
 * general path: global -> registers -> LDS, any shape or alignment
 * ============================================================================================ */

/* operand stored [row][K] (k contiguous): one 16-byte chunk = 8 k of one row */
template <int ROWS, int THREADS>
struct StageKContig {
	static constexpr int CHUNKS = ROWS * CHUNKS_PER_ROW;
	static constexpr int PER_THREAD = (CHUNKS + THREADS - 1) / THREADS;
	u32x4 r[PER_THREAD];

	/* map: NULL, or the source row of every row of the problem (a gathered operand) */
	__device__ __forceinline__ void load(const bf16_t * src, int row0, int rows_total, int k0, int K, bool vec_ok, const int * map = nullptr) {
		#pragma unroll
		for (int i = 0; i < PER_THREAD; i++) {
			int id = i * THREADS + threadIdx.x;
			int row = id / CHUNKS_PER_ROW;
			int c = id % CHUNKS_PER_ROW;
			int gr = row0 + row;
			int gk = k0 + c * 8;
			u32x4 v = {0u, 0u, 0u, 0u};
			if (id < CHUNKS && gr < rows_total && gk < K) {
				const bf16_t * ptr = src + (long long) (map ? map[gr] : gr) * K + gk;
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

	/* map: NULL, or the source row of every k-row of the problem (a gathered operand) */
	__device__ __forceinline__ void load(const bf16_t * src, int row0, int rows_total, int k0, int K, bool vec_ok, const int * map = nullptr) {
		#pragma unroll
		for (int i = 0; i < PER_THREAD; i++) {
			int id = i * THREADS + threadIdx.x;
			int k = id / (ROWS / 8);
			int rc = id % (ROWS / 8);
			int gk = k0 + k;
			int gr = row0 + rc * 8;
			u32x4 v = {0u, 0u, 0u, 0u};
			if (id < CHUNKS && gk < K && gr < rows_total) {
				const bf16_t * ptr = src + (long long) (map ? map[gk] : gk) * rows_total + gr;
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

template <int BM, int BN, int WAVES_M, int WAVES_N, bool P_KMAJOR, bool Q_KMAJOR, int MODE>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_bf16_staged_kernel(GemmParams p) {
	constexpr int THREADS = WAVES_M * WAVES_N * 64;
	constexpr int WTM = BM / WAVES_M;
	constexpr int WTN = BN / WAVES_N;
	constexpr int TM = WTM / 16;
	constexpr int TN = WTN / 16;
	static_assert(WTM % 16 == 0 && WTN % 16 == 0, "wave tile must be a multiple of the 16x16 MFMA tile");

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

	f32x4_t acc[TM][TN];
	#pragma unroll
	for (int i = 0; i < TM; i++) {
		#pragma unroll
		for (int j = 0; j < TN; j++) {
			acc[i][j] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
		}
	}

	const int k_tiles = (t.K + BK - 1) / BK;
	stP.load(t.P, t.m0, t.M, 0, t.K, p_vec, t.Pmap);
	stQ.load(t.Q, t.n0, t.N, 0, t.K, q_vec, t.Qmap);
	stP.store(lds);
	stQ.store(lds + BM * BK);
	__syncthreads();

	for (int kt = 0; kt < k_tiles; kt++) {
		const int cur = kt & 1;
		if (kt + 1 < k_tiles) {
			stP.load(t.P, t.m0, t.M, (kt + 1) * BK, t.K, p_vec, t.Pmap);
			stQ.load(t.Q, t.n0, t.N, (kt + 1) * BK, t.K, q_vec, t.Qmap);
		}
		const bf16_t * cp = lds + cur * STAGE;
		const bf16_t * cq = cp + BM * BK;
		#pragma unroll
		for (int s = 0; s < BK / 32; s++) {
			bf16x8 a[TM], b[TN];
			#pragma unroll
			for (int i = 0; i < TM; i++) {
				a[i] = read_fragment<false, BM>(cp, wm + i * 16, s, lane);
			}
			#pragma unroll
			for (int j = 0; j < TN; j++) {
				b[j] = read_fragment<false, BN>(cq, wn + j * 16, s, lane);
			}
			#pragma unroll
			for (int j = 0; j < TN; j++) {
				#pragma unroll
				for (int i = 0; i < TM; i++) {
					acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
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

	store_accumulators<TM, TN>(t, p, acc, wm, wn, lane);
}

#endif
