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
 * The kernels live in gemm_kernel.h (eight waves), gemm_w4_kernel.h (four waves) and gemm_typed_kernel.h (element
 * types beside all-bf16); this file decodes the op arguments, checks them on the host and picks a kernel: the
 * direct-to-LDS kernels when every operand is 16-byte aligned with a contiguous extent that is a multiple of 8
 * elements, the register-staged kernel otherwise; for large ragged-N launches without a C operand the choice between
 * the eight-wave kernel and the four-wave 256 x 384 one is left to the device (launch_gemm).
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "dataflow_amd.h"
#include "dataflow_amd_ops.h"
#include "amd_matmul.h"
#include "gemm_kernel.h"
#include "gemm_w4_kernel.h"
#include "gemm_typed_kernel.h"

/* ------------------------------------------------------------------ host side */

struct MatmulExtra {
	int cu_count;
	int lds_optin;
};

/* Scratch of amd_matmul_no_alloc: the fp32 partial sums of a split along K, which amd_matmul keeps in the caller's
 * workspace.  A file-scope device array: every GPU the library runs on holds its own copy at its own address until the
 * process ends.  In host code the name is only a handle for hipGetSymbolAddress; the address of each device's copy is
 * looked up once per device in amd_matmul_init and everything below uses that pointer. */
#define AMD_MATMUL_SCRATCH_BYTES (8u << 20)
#define AMD_MATMUL_MAX_DEVICES 64
static __device__ __align__(256) unsigned char scratch[AMD_MATMUL_SCRATCH_BYTES];
static void * scratch_of_device[AMD_MATMUL_MAX_DEVICES];

static int check_launch(void) {
	hipError_t e = hipGetLastError();
	if (e != hipSuccess) {
		fprintf(stderr, "Error: gemm kernel launch failed: %s...\n", hipGetErrorString(e));
		return -1;
	}
	return 0;
}

/* register-staged kernel: dynamic LDS, two stages */
template <int BM, int BN, int WAVES_M, int WAVES_N, bool PK, bool QK, int MODE>
static int launch_staged(const GemmParams & p, long grid, hipStream_t stream) {
	constexpr int threads = WAVES_M * WAVES_N * 64;
	constexpr size_t lds_bytes = 2 * (BM + BN) * BK * sizeof(bf16_t);
	auto kernel = gemm_bf16_staged_kernel<BM, BN, WAVES_M, WAVES_N, PK, QK, MODE>;
	static bool attr_done = false;
	if (lds_bytes > 65536 && !attr_done) {
		hipError_t e = hipFuncSetAttribute((const void *) kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int) lds_bytes);
		if (e != hipSuccess) {
			fprintf(stderr, "Error: could not raise dynamic LDS limit to %zu bytes: %s...\n", lds_bytes, hipGetErrorString(e));
			return -1;
		}
		attr_done = true;
	}
	hipLaunchKernelGGL(kernel, dim3((unsigned int) grid), dim3(threads), lds_bytes, stream, p);
	return check_launch();
}

/* direct-to-LDS kernel: static LDS */
template <int BM, int BN, int WAVES_M, int WAVES_N, bool PK, bool QK, int MODE, int GATHER = GATHER_NONE>
static int launch_direct(const GemmParams & p, long grid, hipStream_t stream) {
	constexpr int threads = WAVES_M * WAVES_N * 64;
	hipLaunchKernelGGL((gemm_bf16_direct_kernel<BM, BN, WAVES_M, WAVES_N, PK, QK, MODE, GATHER>), dim3((unsigned int) grid), dim3(threads), 0, stream, p);
	return check_launch();
}

/* the direct kernel with four stages, for the partial products of a split along K (amd_matmul's few-tile problems) */
static int launch_split_deep(const GemmParams & p, int transa, int transb, long grid, hipStream_t stream) {
	const bool pk = !transa;
	const bool qk = transb != 0;
#define DEEP(PK, QK) do { \
		hipLaunchKernelGGL((gemm_bf16_direct_kernel<128, 128, 2, 2, PK, QK, MODE_SINGLE, GATHER_NONE, 4>), dim3((unsigned int) grid), dim3(256), 0, stream, p); \
		return check_launch(); \
	} while (0)
	if (!pk && !qk) { DEEP(false, false); }
	if (pk && !qk) { DEEP(true, false); }
	if (pk && qk) { DEEP(true, true); }
	DEEP(false, true);
#undef DEEP
}

/* streaming kernel: one persistent work-group per compute unit (LDS allows no more), a multiple of 8 so every die gets the same share */
template <int BM, int BN, int WAVES_M, int WAVES_N, bool PK, bool QK, int MODE, int GATHER = GATHER_NONE>
static int launch_stream(const GemmParams & p, long tiles_upper_bound, long cu_count, hipStream_t stream) {
	constexpr int threads = WAVES_M * WAVES_N * 64;
	long grid = cu_count & ~7L;
	if (grid < 8) {
		grid = 8;
	}
	const long need = (tiles_upper_bound + 7) & ~7L;
	if (need < grid) {
		grid = need;
	}
	hipLaunchKernelGGL((gemm_bf16_stream_kernel<BM, BN, WAVES_M, WAVES_N, PK, QK, MODE, GATHER>), dim3((unsigned int) grid), dim3(threads), 0, stream, p);
	return check_launch();
}

/* four-wave kernel (gemm_w4_kernel.h): same grid rule as the streaming kernel, 256 threads */
template <bool PK, int MODE, int GATHER = GATHER_NONE>
static int launch_w4(const GemmParams & p, long tiles_upper_bound, long cu_count, hipStream_t stream) {
	long grid = cu_count & ~7L;
	if (grid < 8) {
		grid = 8;
	}
	const long need = (tiles_upper_bound + 7) & ~7L;
	if (need < grid) {
		grid = need;
	}
	hipLaunchKernelGGL((gemm_bf16_w4_kernel<PK, MODE, GATHER>), dim3((unsigned int) grid), dim3(256), 0, stream, p);
	return check_launch();
}

/* the four symmetric waves with the 256 x 384 tile (gemm_w4_kernel.h): same grid rule */
template <bool PK, int MODE, int GATHER = GATHER_NONE>
static int launch_w4d(const GemmParams & p, long tiles_upper_bound, long cu_count, hipStream_t stream) {
	long grid = cu_count & ~7L;
	if (grid < 8) {
		grid = 8;
	}
	const long need = (tiles_upper_bound + 7) & ~7L;
	if (need < grid) {
		grid = need;
	}
	hipLaunchKernelGGL((gemm_bf16_w4d_kernel<PK, MODE, GATHER>), dim3((unsigned int) grid), dim3(256), 0, stream, p);
	return check_launch();
}

/* Which persistent kernel large problems without a C operand run: AMD_MATMUL_KERNEL_EIGHT_WAVES or
 * AMD_MATMUL_KERNEL_FOUR_WAVES (amd_matmul.h).  Process-wide; amd_matmul_select_kernel changes it, the environment
 * variable AMD_MATMUL_KERNEL ("8" or "4") sets the initial value when the op is registered. */
static int kernel_choice = AMD_MATMUL_KERNEL_DEFAULT;

extern "C" int amd_matmul_select_kernel(int which) {
	if (which != AMD_MATMUL_KERNEL_AUTO && which != AMD_MATMUL_KERNEL_EIGHT_WAVES && which != AMD_MATMUL_KERNEL_FOUR_WAVES &&
		which != AMD_MATMUL_KERNEL_FOUR_WAVES_384) {
		fprintf(stderr, "Error: amd_matmul_select_kernel: unknown kernel %d...\n", which);
		return -1;
	}
	kernel_choice = which;
	return 0;
}

/* the four-wave kernel takes whole k-tiles in pairs from k-contiguous operands, 16-byte lines of output, no C */
static bool w4_ok(const GemmParams & p) {
	return !(p.C && p.beta != 0.0f) && (p.K % 128 == 0) && p.K <= (1 << 21) &&
		   (p.M % 8 == 0) && ((((uintptr_t) p.D) & 15) == 0);
}

static long round_up8(long v) { return (v + 7) & ~7L; }
static long tiles_of(long extent, long tile) { return (extent + tile - 1) / tile; }

#define BIG_TILE 256, 256, 4, 2          /* 8 waves, wave tile 64 x 128 */
#define WIDE_TILE 256, 288, 4, 2         /* 8 waves, wave tile 64 x 144: the token side of the ragged-N launches, see launch_gemm */
#define SMALL_TILE 128, 128, 2, 2        /* 4 waves, wave tile 64 x 64 */

/* grid_big / grid_small: work-group counts for the two tile sizes; `direct` selects the fast kernel */
template <int MODE>
static int launch_gemm(const GemmParams & p, int transa, int transb, bool direct, bool big, long grid_big, long grid_small, long cu_count, hipStream_t stream,
					   long grid_wide = 0) {
	/* to_trans_a = 1 means A is stored [M][K] (k contiguous); to_trans_b = 1 means B is stored [K][N] (k-major) */
	const bool pk = !transa;
	const bool qk = transb != 0;
	if (grid_big <= 0 || grid_small <= 0) {
		return 0;
	}
	const bool four_ok = direct && big && !qk && w4_ok(p);
	const bool wide_only = kernel_choice == AMD_MATMUL_KERNEL_FOUR_WAVES_384;
	bool either = kernel_choice == AMD_MATMUL_KERNEL_AUTO;
	if (MODE == MODE_RAGGED_N && either && p.num_groups > 0) {
		/* The second launch costs a few microseconds even where it returns at once.  With all groups the same size the
		 * rule of ragged_n_prefers_384 can be evaluated here; where the narrow tiling wins then, uneven groups only make
		 * it win by more (short groups fill a 384-row tile worse), and the eight-wave kernel is launched alone. */
		const long rows = (long) p.N / p.num_groups;
		const long tiles_m = tiles_of(p.M, 256);
		long groups = cu_count & ~7L;
		groups = groups < 8 ? 8 : groups;
		const long narrow = tiles_of(tiles_m * p.num_groups * tiles_of(rows > 0 ? rows : 1, 288), groups);
		const long wide = tiles_of(tiles_m * p.num_groups * tiles_of(rows > 0 ? rows : 1, 384), groups);
		const long k_tiles = tiles_of(p.K, BK);
		if (!(WIDE_TILE_COST(wide, k_tiles) < NARROW_TILE_COST(narrow, k_tiles))) {
			either = false;
		}
	}
	if (MODE == MODE_RAGGED_N && four_ok && grid_wide > 0 && (wide_only || either)) {
		/* grid_wide counts tiles of 288 rows: an upper bound for tiles of 384.  With the choice left open both kernels
		 * are launched and the work-groups decide from the group sizes which of them runs (GemmParams::arbitrate). */
		GemmParams q = p;
		if (either) {
			q.arbitrate = ARBITRATE_NARROW;
			int r;
			if (p.gather) {
				r = pk ? launch_stream<WIDE_TILE, true, false, MODE_RAGGED_N, GATHER_Q_ROWS>(q, grid_wide, cu_count, stream)
					   : launch_stream<WIDE_TILE, false, false, MODE_RAGGED_N, GATHER_Q_ROWS>(q, grid_wide, cu_count, stream);
			} else {
				r = pk ? launch_stream<WIDE_TILE, true, false, MODE_RAGGED_N>(q, grid_wide, cu_count, stream)
					   : launch_stream<WIDE_TILE, false, false, MODE_RAGGED_N>(q, grid_wide, cu_count, stream);
			}
			if (r) {
				return r;
			}
			q.arbitrate = ARBITRATE_WIDE;
		}
		if (p.gather) {
			if (pk) { return launch_w4d<true, MODE_RAGGED_N, GATHER_Q_ROWS>(q, grid_wide, cu_count, stream); }
			return launch_w4d<false, MODE_RAGGED_N, GATHER_Q_ROWS>(q, grid_wide, cu_count, stream);
		}
		if (pk) { return launch_w4d<true, MODE_RAGGED_N>(q, grid_wide, cu_count, stream); }
		return launch_w4d<false, MODE_RAGGED_N>(q, grid_wide, cu_count, stream);
	}
	if (MODE == MODE_SINGLE && four_ok && p.split_k <= 1 && (wide_only || either)) {
		/* a single problem's tiles are known here: the same rule as for the ragged launches, against the 256 x 256 tiles
		 * the eight-wave kernel walks a single problem in */
		const long tiles = tiles_of(p.M, 256) * tiles_of(p.N, 384);
		long groups = cu_count & ~7L;
		groups = groups < 8 ? 8 : groups;
		const long wide = tiles_of(tiles, groups), narrow = tiles_of(grid_big, groups);
		const long k_tiles = tiles_of(p.K, BK);
		if (wide_only || wide * (256 + 384) * (103 * k_tiles + 160) < narrow * (256 + 256) * 100 * k_tiles) {
			if (pk) { return launch_w4d<true, MODE_SINGLE>(p, tiles, cu_count, stream); }
			return launch_w4d<false, MODE_SINGLE>(p, tiles, cu_count, stream);
		}
	}
	const bool four_one_loader = kernel_choice == AMD_MATMUL_KERNEL_FOUR_WAVES;
	if (MODE == MODE_RAGGED_N && four_ok && grid_wide > 0 && four_one_loader) {
		if (p.gather) {
			if (pk) { return launch_w4<true, MODE_RAGGED_N, GATHER_Q_ROWS>(p, grid_wide, cu_count, stream); }
			return launch_w4<false, MODE_RAGGED_N, GATHER_Q_ROWS>(p, grid_wide, cu_count, stream);
		}
		if (pk) { return launch_w4<true, MODE_RAGGED_N>(p, grid_wide, cu_count, stream); }
		return launch_w4<false, MODE_RAGGED_N>(p, grid_wide, cu_count, stream);
	}
	if (MODE == MODE_SINGLE && four_ok && p.split_k <= 1 && four_one_loader) {
		const long tiles = tiles_of(p.M, 256) * tiles_of(p.N, 288);
		if (pk) { return launch_w4<true, MODE_SINGLE>(p, tiles, cu_count, stream); }
		return launch_w4<false, MODE_SINGLE>(p, tiles, cu_count, stream);
	}
	if (MODE == MODE_RAGGED_N && direct && big && grid_wide > 0 && !qk && !(p.C && p.beta != 0.0f)) {
		/* Token rows in tiles of 288: a launch takes as long as its tiles are many (a k-tile step is paced by the
		 * latency of the operand stream, not by the multiplies), and a group of slightly more than a multiple of 256
		 * rows -- every second expert when the mean is such a multiple -- then needs no extra, nearly empty tile.
		 * Every element is accumulated over k in the same order as in the 256-row tiles: results are bit-identical. */
		if (p.gather) {
			if (pk) { return launch_stream<WIDE_TILE, true, false, MODE_RAGGED_N, GATHER_Q_ROWS>(p, grid_wide, cu_count, stream); }
			return launch_stream<WIDE_TILE, false, false, MODE_RAGGED_N, GATHER_Q_ROWS>(p, grid_wide, cu_count, stream);
		}
		if (pk) { return launch_stream<WIDE_TILE, true, false, MODE_RAGGED_N>(p, grid_wide, cu_count, stream); }
		return launch_stream<WIDE_TILE, false, false, MODE_RAGGED_N>(p, grid_wide, cu_count, stream);
	}
#define PICK(PK, QK) do { \
		if (direct) { \
			return big ? launch_stream<BIG_TILE, PK, QK, MODE>(p, grid_big, cu_count, stream) \
					   : launch_direct<SMALL_TILE, PK, QK, MODE>(p, round_up8(grid_small), stream); \
		} \
		return launch_staged<SMALL_TILE, PK, QK, MODE>(p, round_up8(grid_small), stream); \
	} while (0)
	if (MODE == MODE_RAGGED_N && p.gather) {
		/* gathered B: its rows are fetched through the row map by the loaders themselves (B is k-contiguous here) */
#define PICK_GATHER(PK) do { \
			if (direct) { \
				return big ? launch_stream<BIG_TILE, PK, false, MODE_RAGGED_N, GATHER_Q_ROWS>(p, grid_big, cu_count, stream) \
						   : launch_direct<SMALL_TILE, PK, false, MODE_RAGGED_N, GATHER_Q_ROWS>(p, round_up8(grid_small), stream); \
			} \
			return launch_staged<SMALL_TILE, PK, false, MODE_RAGGED_N>(p, round_up8(grid_small), stream); \
		} while (0)
		if (pk) { PICK_GATHER(true); }
		PICK_GATHER(false);
#undef PICK_GATHER
	}
	if (MODE == MODE_RAGGED_K && p.gather) {
		/* gathered A: the k-rows of the reduction are fetched through the row map (both operands are k-major here) */
		if (direct) {
			return big ? launch_stream<BIG_TILE, true, true, MODE_RAGGED_K, GATHER_P_KROWS>(p, grid_big, cu_count, stream)
					   : launch_direct<SMALL_TILE, true, true, MODE_RAGGED_K, GATHER_P_KROWS>(p, round_up8(grid_small), stream);
		}
		return launch_staged<SMALL_TILE, true, true, MODE_RAGGED_K>(p, round_up8(grid_small), stream);
	}
	if (!pk && !qk) { PICK(false, false); }
	if (pk && !qk) { PICK(true, false); }
	if (pk && qk) { PICK(true, true); }
	PICK(false, true);
#undef PICK
}

static bool aligned16(const void * ptr) { return (((uintptr_t) ptr) & 15) == 0; }

/* Can the operand (k-contiguous: rows of K elements; k-major: K rows of `rows` elements) be fetched with 16-byte
 * buffer loads?  Needs a 16-byte aligned base, a contiguous extent that is a multiple of 8 elements (so every row
 * starts aligned) and group bases that keep that alignment.  The kernels address one k-tile of one 256-row panel with
 * 32-bit offsets and everything above that with 64-bit pointers, so the operand's total size does not matter; the
 * contiguous extent itself is bounded (256 rows of K elements, or 64 k of `rows` elements, must stay below 4 GiB). */
static bool operand_direct_ok(const void * base, bool kmajor, long rows, long K, long group_stride_elems) {
	const long contiguous = kmajor ? rows : K;
	const long bound = kmajor ? (1L << 24) : (1L << 22);
	return aligned16(base) && (contiguous % 8 == 0) && (group_stride_elems % 8 == 0) && contiguous <= bound;
}

static int check_dtypes(DataflowDatatype a_dt, DataflowDatatype b_dt, DataflowDatatype c_dt, DataflowDatatype d_dt,
						DataflowDatatype compute_dt, const void * C, float beta) {
	if (a_dt != DATAFLOW_BF16 || b_dt != DATAFLOW_BF16 || d_dt != DATAFLOW_BF16) {
		fprintf(stderr, "Error: this matmul takes bf16 operands with a bf16 result; the single matmul also fp32 -> fp32, fp16 -> fp16 | fp32 and bf16 -> fp32 with fp32 accumulation and C in D's type (got A=%s B=%s D=%s)...\n",
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
	const int dev = dataflow_handle->device_id;
	if (dev >= 0 && dev < AMD_MATMUL_MAX_DEVICES && !scratch_of_device[dev]) {
		void * ptr = NULL;
		hipError_t e = hipSetDevice(dev);
		if (e == hipSuccess) {
			e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
		}
		if (e != hipSuccess || !ptr) {
			fprintf(stderr, "Error: could not look up the matmul scratch on device %d: %s...\n", dev, hipGetErrorString(e));
			free(extra);
			return -1;
		}
		scratch_of_device[dev] = ptr;
	}
	Hip_Device_Info * info = (Hip_Device_Info *) dataflow_handle->device_info;
	extra->cu_count = info ? info->cu_count : 256;
	extra->lds_optin = info ? info->optin_max_lds_per_block : 65536;
	fn->op_extra = extra;
	const char * env = getenv("AMD_MATMUL_KERNEL");
	if (env && (env[0] == '4' || env[0] == '8') && env[1] == 0) {
		kernel_choice = env[0] == '4' ? AMD_MATMUL_KERNEL_FOUR_WAVES : AMD_MATMUL_KERNEL_EIGHT_WAVES;
	} else if (env && strcmp(env, "384") == 0) {
		kernel_choice = AMD_MATMUL_KERNEL_FOUR_WAVES_384;
	} else if (env && strcmp(env, "auto") == 0) {
		kernel_choice = AMD_MATMUL_KERNEL_AUTO;
	}
	return 0;
}

static long extra_cu_count(void * op_extra) {
	return op_extra ? ((MatmulExtra *) op_extra)->cu_count : 256;
}

/* shared by amd_matmul and amd_matmul_no_alloc: checks, kernel choice, launch.  `workspace` (may be NULL) holds the fp32
 * partial sums of a split along K; `must_fit`: a split that the workspace cannot hold is an error instead of running
 * unsplit */
static int run_matmul(Dataflow_Handle * dataflow_handle, int stream_id, GemmParams & p, int transa, int transb,
					  float * workspace, uint64_t workspace_bytes, long cu_count, bool must_fit) {
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
	const bool direct = operand_direct_ok(p.A, !transa, p.M, p.K, 0) && operand_direct_ok(p.B, transb != 0, p.N, p.K, 0);
	/* small problems: 128x128 tiles fill the device better; large ones amortise operand traffic with 256x256 */
	const long grid_big = tiles_of(p.M, 256) * tiles_of(p.N, 256);
	const long grid_small = tiles_of(p.M, 128) * tiles_of(p.N, 128);
	const bool big = grid_big >= cu_count / 2 && p.M >= 256 && p.N >= 256;
	/* Few tiles and a long K (the router's GEMMs: 64 experts on one side): split K over the idle compute units,
	 * fp32 partial sums in the caller's workspace, one reduction pass.  Without a workspace that is large enough
	 * (and 16-byte aligned) the problem runs unsplit. */
	const long k_tiles = tiles_of(p.K, BK);
	long splits = direct && !big ? cu_count / grid_small : 1;
	if (splits >= 2 && k_tiles >= 8 && workspace && aligned16(workspace)) {
		long per = tiles_of(k_tiles, splits);
		per = per < 4 ? 4 : per;
		per = (per + 3) & ~3L;                      /* the four-stage kernel takes its k-tiles in fours */
		splits = tiles_of(k_tiles, per);
		const uint64_t count = (uint64_t) p.M * (uint64_t) p.N;
		if (splits >= 2 && must_fit && workspace_bytes / 4 / (uint64_t) splits < count) {
			fprintf(stderr, "Error: this %d x %d x %d matmul splits along K into %ld parts of %lu partial sums each, more than the %lu-byte scratch holds; use the matmul op with a workspace...\n",
					p.M, p.K, p.N, splits, (unsigned long) count, (unsigned long) workspace_bytes);
			return -1;
		}
		if (splits >= 2 && workspace_bytes / 4 / (uint64_t) splits >= count) {
			p.partial = workspace;
			p.split_k = (int) splits;
			p.kt_per_split = (int) per;
			if (launch_split_deep(p, transa, transb, (grid_small * splits + 7) & ~7L, stream)) {
				return -1;
			}
			const long blocks = (long) ((count + 255) / 256);
			hipLaunchKernelGGL(splitk_reduce_kernel, dim3((unsigned int) (blocks < 4096 ? blocks : 4096)), dim3(256), 0, stream,
							   (const float *) workspace, (int) splits, (long long) count, p.alpha, p.beta, p.C, p.D);
			return check_launch();
		}
	}
	return launch_gemm<MODE_SINGLE>(p, transa, transb, direct, big, grid_big, grid_small, cu_count, stream);
}

/* Ragged K without a C operand: D_g = alpha * (sum over no rows) = 0 for a group without rows.  The GEMM kernels give such
 * a group no tile, so its zeros are written here, by work-groups that find the group empty (the others exit at once). */
__global__ void __launch_bounds__(256) zero_empty_groups_kernel(const int * __restrict__ cumsum, int num_groups, bf16_t * __restrict__ D, long long strideD, long long count) {
	const long long step = (long long) gridDim.x * 256;
	const long long first = (long long) blockIdx.x * 256 + threadIdx.x;
	for (int g = blockIdx.y; g < num_groups; g += gridDim.y) {
		const int hi = cumsum[g];
		const int lo = g ? cumsum[g - 1] : 0;
		if (hi - lo > 0) {
			continue;
		}
		bf16_t * dst = D + (long long) g * strideD;
		const long long vecs = (((uintptr_t) dst) & 15) == 0 ? count >> 3 : 0;       /* 16-byte stores where the group's base allows them */
		for (long long i = first; i < vecs; i += step) {
			reinterpret_cast<uint4 *>(dst)[i] = uint4{0u, 0u, 0u, 0u};
		}
		for (long long i = (vecs << 3) + first; i < count; i += step) {
			dst[i] = (bf16_t) 0;
		}
	}
}

/* The element types beside all-bf16 (gemm_typed_kernel.h).  Returns 0 when the combination is not one of them, 1 after a
 * launch, -1 on an error.  A and B share a type; C, where it is used, has D's type. */
static int run_typed_matmul(Dataflow_Handle * dataflow_handle, int stream_id, DataflowDatatype ab_dt, DataflowDatatype d_dt,
							int transa, int transb, int M, int K, int N, float alpha, float beta, const void * A, const void * B,
							const void * C, void * D) {
	const bool f32_f32 = ab_dt == DATAFLOW_FP32 && d_dt == DATAFLOW_FP32;
	const bool f16_f16 = ab_dt == DATAFLOW_FP16 && d_dt == DATAFLOW_FP16;
	const bool f16_f32 = ab_dt == DATAFLOW_FP16 && d_dt == DATAFLOW_FP32;
	const bool bf16_f32 = ab_dt == DATAFLOW_BF16 && d_dt == DATAFLOW_FP32;
	if (!f32_f32 && !f16_f16 && !f16_f32 && !bf16_f32) {
		return 0;
	}
	if (M < 0 || N < 0 || K < 0 || !D || ((M > 0 && N > 0 && K > 0) && (!A || !B))) {
		fprintf(stderr, "Error: bad matmul arguments M=%d K=%d N=%d A=%p B=%p D=%p...\n", M, K, N, A, B, D);
		return -1;
	}
	if (M == 0 || N == 0) {
		return 1;
	}
	hipStream_t stream;
	if (resolve_stream(dataflow_handle, stream_id, &stream)) {
		return -1;
	}
	if (hipSetDevice(dataflow_handle->device_id) != hipSuccess) {
		fprintf(stderr, "Error: hipSetDevice failed in matmul...\n");
		return -1;
	}
	const long tiles = tiles_of(M, TYPED_TILE) * tiles_of(N, TYPED_TILE);
	if (tiles > 0x7fffffffL) {
		fprintf(stderr, "Error: %d x %d is more output tiles than one launch of this matmul takes...\n", M, N);
		return -1;
	}
	TypedGemmParams t;
	t.P = A; t.Q = B; t.C = C; t.D = D;
	t.M = M; t.N = N; t.K = K;
	t.p_kmajor = !transa;
	t.q_kmajor = transb != 0;
	t.alpha = alpha; t.beta = beta;
	const dim3 grid((unsigned int) tiles), block(TYPED_THREADS);
	if (f32_f32) {
		hipLaunchKernelGGL((gemm_typed_kernel<float, float>), grid, block, 0, stream, t);
	} else if (f16_f16) {
		hipLaunchKernelGGL((gemm_typed_kernel<_Float16, _Float16>), grid, block, 0, stream, t);
	} else if (f16_f32) {
		hipLaunchKernelGGL((gemm_typed_kernel<_Float16, float>), grid, block, 0, stream, t);
	} else {
		hipLaunchKernelGGL((gemm_typed_kernel<bf16_t, float>), grid, block, 0, stream, t);
	}
	return check_launch() ? -1 : 1;
}

extern "C" int amd_matmul(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra) {
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
	if (a_dt == b_dt && !(a_dt == DATAFLOW_BF16 && d_dt == DATAFLOW_BF16)) {
		/* fp32, fp16, or bf16 with an fp32 result: fp32 accumulation only, C in D's type */
		if ((p.C == NULL || c_dt == d_dt) && (compute_dt == DATAFLOW_FP32 || compute_dt == DATAFLOW_NONE)) {
			const int r = run_typed_matmul(dataflow_handle, stream_id, a_dt, d_dt, transa, transb, p.M, p.K, p.N, p.alpha, p.beta,
										   (const void *) p.A, (const void *) p.B, (const void *) p.C, (void *) p.D);
			if (r != 0) {
				return r < 0 ? -1 : 0;
			}
		}
	}
	if (check_dtypes(a_dt, b_dt, c_dt, d_dt, compute_dt, p.C, p.beta)) {
		return -1;
	}
	const uint64_t workspace_bytes = *((uint64_t *) a[17]);
	float * workspace = (float *) *((uint64_t *) a[18]);
	return run_matmul(dataflow_handle, stream_id, p, transa, transb, workspace, workspace_bytes, extra_cu_count(op_extra), false);
}

/* D = alpha * op(A) op(B) + beta * C like amd_matmul (same kernels, same split along K, bit-identical results), for
 * callers that cannot allocate: the split's partial sums go to the library's own scratch on the handle's device
 * instead of a caller's workspace, and the call makes no allocation of any kind.  BF16 operands and result, fp32
 * accumulation; C is ignored when NULL or beta == 0.  A problem whose split would need more than the scratch
 * (AMD_MATMUL_SCRATCH_BYTES, 8 MiB) is refused with -1.  The scratch keeps the last call's contents (nothing in it
 * has to start at zero: every partial sum is written before it is read); it is shared by every call on that device, so
 * calls that overlap on one device -- two streams, two host threads -- race on it. */
extern "C" int amd_matmul_no_alloc(Dataflow_Handle * dataflow_handle, int stream_id, int to_trans_a, int to_trans_b,
								   int M, int K, int N, float alpha, float beta, void * A, void * B, void * C, void * D) {
	if (!dataflow_handle) {
		fprintf(stderr, "Error: amd_matmul_no_alloc needs a handle...\n");
		return -1;
	}
	const int dev = dataflow_handle->device_id;
	if (dev < 0 || dev >= AMD_MATMUL_MAX_DEVICES || !scratch_of_device[dev]) {
		fprintf(stderr, "Error: amd_matmul_no_alloc on device %d before the matmul op was registered on a handle of that device...\n", dev);
		return -1;
	}
	GemmParams p;
	memset(&p, 0, sizeof(p));
	p.M = M; p.K = K; p.N = N;
	p.alpha = alpha; p.beta = beta;
	p.A = (const bf16_t *) A; p.B = (const bf16_t *) B; p.C = (beta == 0.0f) ? NULL : (const bf16_t *) C; p.D = (bf16_t *) D;
	Hip_Device_Info * info = (Hip_Device_Info *) dataflow_handle->device_info;
	return run_matmul(dataflow_handle, stream_id, p, to_trans_a, to_trans_b, (float *) scratch_of_device[dev], AMD_MATMUL_SCRATCH_BYTES,
					  info ? info->cu_count : 256, true);
}

extern "C" int amd_grouped_matmul(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra) {
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
	/* the gathered form of the op carries two more arguments: the row map and the number of rows of the gathered operand */
	if (op->op_skeleton.header.num_args == 24) {
		p.gather = (const int *) *((uint64_t *) a[22]);
		p.gather_rows = *((int *) a[23]);
		const int row_elems = ragged == AMD_GROUPED_RAGGED_N ? p.K : p.M;      /* one row of the gathered operand */
		if (!p.gather || p.gather_rows < 1 || (ragged != AMD_GROUPED_RAGGED_N && ragged != AMD_GROUPED_RAGGED_K) || row_elems < 1 ||
			(uint64_t) p.gather_rows * (uint64_t) row_elems * 2u > 0xFFFFFFFFull) {
			fprintf(stderr, "Error: bad gathered grouped matmul arguments (row map %p, %d rows of %d elements: the gathered operand must stay below 4 GiB)...\n",
					(const void *) p.gather, p.gather_rows, row_elems);
			return -1;
		}
	}
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
		/* A: one matrix per group at strideA; B: rows packed, so every group base is K-aligned */
		const bool direct = operand_direct_ok(p.A, !transa, p.M, p.K, p.strideA) && operand_direct_ok(p.B, false, p.N, p.K, 0);
		/* upper bound of n-tiles: every group may end in one partial tile */
		const long grid_big = tiles_of(p.M, 256) * ((long) p.N / 256 + p.num_groups);
		const long grid_small = tiles_of(p.M, 128) * ((long) p.N / 128 + p.num_groups);
		const bool big = p.M >= 256 && (long) p.N / 256 * tiles_of(p.M, 256) >= 128;
		const long grid_wide = tiles_of(p.M, 256) * ((long) p.N / 288 + p.num_groups);
		return launch_gemm<MODE_RAGGED_N>(p, transa, transb, direct, big, grid_big, grid_small, extra_cu_count(op_extra), stream, grid_wide);
	}
	if (ragged == AMD_GROUPED_RAGGED_K) {
		if (transa != 0 || transb != 1 || p.N < 1) {
			fprintf(stderr, "Error: ragged-K grouped matmul needs to_trans_a == 0 and to_trans_b == 1...\n");
			return -1;
		}
		/* both operands have their rows packed along k: group bases are aligned when M and N are multiples of 8 */
		const bool direct = operand_direct_ok(p.A, true, p.M, p.K, 0) && operand_direct_ok(p.B, true, p.N, p.K, 0) && (p.strideD % 4 == 0);
		const long grid_big = tiles_of(p.M, 256) * tiles_of(p.N, 256) * p.num_groups;
		const long grid_small = tiles_of(p.M, 128) * tiles_of(p.N, 128) * p.num_groups;
		const bool big = p.M >= 256 && p.N >= 256 && grid_big >= 128;
		if (p.C == nullptr) {
			const long long count = (long long) p.M * p.N;
			const long long blocks = (count / 8 + 255) / 256;
			hipLaunchKernelGGL(zero_empty_groups_kernel, dim3((unsigned int) (blocks < 64 ? (blocks < 1 ? 1 : blocks) : 64), (unsigned int) (p.num_groups < 65535 ? p.num_groups : 65535)), dim3(256), 0, stream,
							   p.cumsum, p.num_groups, p.D, p.strideD, count);
			if (check_launch()) {
				return -1;
			}
		}
		return launch_gemm<MODE_RAGGED_K>(p, transa, transb, direct, big, grid_big, grid_small, extra_cu_count(op_extra), stream);
	}
	fprintf(stderr, "Error: unknown ragged dimension %d...\n", ragged);
	return -1;
}
