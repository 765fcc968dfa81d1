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
 * The kernels live in gemm_kernel.h; this file decodes the op arguments, checks them on the host and picks
 * a kernel: the direct-to-LDS kernels when every operand is 16-byte aligned with a contiguous extent that is
 * a multiple of 8 elements, the register-staged kernel otherwise.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "dataflow_amd.h"
#include "dataflow_amd_ops.h"
#include "amd_matmul.h"
#include "gemm_kernel.h"
#include "gemm_w4_kernel.h"

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

/* Which persistent kernel large problems without a C operand run: AMD_MATMUL_KERNEL_EIGHT_WAVES or
 * AMD_MATMUL_KERNEL_FOUR_WAVES (amd_matmul.h).  Process-wide; amd_matmul_select_kernel changes it, the environment
 * variable AMD_MATMUL_KERNEL ("8" or "4") sets the initial value when the op is registered. */
static int kernel_choice = AMD_MATMUL_KERNEL_DEFAULT;

extern "C" int amd_matmul_select_kernel(int which) {
	if (which != AMD_MATMUL_KERNEL_EIGHT_WAVES && which != AMD_MATMUL_KERNEL_FOUR_WAVES) {
		fprintf(stderr, "Error: amd_matmul_select_kernel: unknown kernel %d...\n", which);
		return -1;
	}
	kernel_choice = which;
	return 0;
}

/* the four-wave kernel takes whole k-tiles in pairs from k-contiguous operands, 16-byte lines of output, no C */
static bool w4_ok(const GemmParams & p) {
	return kernel_choice == AMD_MATMUL_KERNEL_FOUR_WAVES && !(p.C && p.beta != 0.0f) && (p.K % 128 == 0) && p.K <= (1 << 21) &&
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
	if (MODE == MODE_RAGGED_N && direct && big && grid_wide > 0 && !qk && w4_ok(p)) {
		if (p.gather) {
			if (pk) { return launch_w4<true, MODE_RAGGED_N, GATHER_Q_ROWS>(p, grid_wide, cu_count, stream); }
			return launch_w4<false, MODE_RAGGED_N, GATHER_Q_ROWS>(p, grid_wide, cu_count, stream);
		}
		if (pk) { return launch_w4<true, MODE_RAGGED_N>(p, grid_wide, cu_count, stream); }
		return launch_w4<false, MODE_RAGGED_N>(p, grid_wide, cu_count, stream);
	}
	if (MODE == MODE_SINGLE && direct && big && !qk && w4_ok(p) && p.split_k <= 1) {
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
		per += per & 1;
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
			if (launch_gemm<MODE_SINGLE>(p, transa, transb, true, false, grid_big, grid_small * splits, cu_count, stream)) {
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
		return launch_gemm<MODE_RAGGED_K>(p, transa, transb, direct, big, grid_big, grid_small, extra_cu_count(op_extra), stream);
	}
	fprintf(stderr, "Error: unknown ragged dimension %d...\n", ragged);
	return -1;
}

/* ------------------------------------------------------------------ diagnostic */

/* Nothing but matrix instructions: every wave keeps independent bf16 MFMAs in flight out of registers, no loads, no
 * LDS.  What this sustains is the ceiling of any GEMM on the card under its power limit.  The power a matrix
 * instruction draws depends on its operands and on its shape, hence the modes (AMD_MFMA_PROBE_* bits):
 *   RANDOM    every lane multiplies pseudo-random values of full mantissa width in [-1, 1) (what a GEMM of real
 *             activations does); without it, small integers times a power of two, which toggle few bits;
 *   SHAPE_16  v_mfma_f32_16x16x32_bf16 (sixteen per round) instead of v_mfma_f32_32x32x16_bf16 (eight per round):
 *             the same flops per round, four times fewer accumulator registers read and written per flop;
 *   VARYING   consecutive instructions take different operand registers (four A and four B fragments in rotation, as
 *             in a GEMM's k-step) instead of the same pair every time. */
typedef float f32x4_acc __attribute__((ext_vector_type(4)));
__global__ void __launch_bounds__(512) mfma_rate_probe_kernel(float * out, int iters, int mode) {
	bf16x8 a[4], b[4];
	uint32_t h = (blockIdx.x * 512u + threadIdx.x) * 2654435761u + 12345u;
	#pragma unroll
	for (int f = 0; f < 4; f++) {
		#pragma unroll
		for (int e = 0; e < 8; e++) {
			if (mode & AMD_MFMA_PROBE_RANDOM) {
				h = h * 1664525u + 1013904223u;
				a[f][e] = (__bf16) ((float) (int) (h >> 8) * (1.0f / 8388608.0f) - 1.0f);
				h = h * 1664525u + 1013904223u;
				b[f][e] = (__bf16) ((float) (int) (h >> 8) * (1.0f / 8388608.0f) - 1.0f);
			} else {
				a[f][e] = (__bf16) ((float) ((threadIdx.x + e + f) & 15) * 0.125f);
				b[f][e] = (__bf16) ((float) ((threadIdx.x * 3 + e + f) & 15) * 0.0625f);
			}
		}
	}
	if (!(mode & AMD_MFMA_PROBE_VARYING)) {
		#pragma unroll
		for (int f = 1; f < 4; f++) {
			a[f] = a[0];
			b[f] = b[0];
		}
	}
	float s = 0.0f;
	if (mode & AMD_MFMA_PROBE_SHAPE_16) {
		f32x4_acc acc[16];
		#pragma unroll
		for (int i = 0; i < 16; i++) {
			acc[i] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};
		}
		for (int it = 0; it < iters; it++) {
			#pragma unroll
			for (int i = 0; i < 16; i++) {
				acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i >> 2], b[i & 3], acc[i], 0, 0, 0);
			}
		}
		#pragma unroll
		for (int i = 0; i < 16; i++) {
			s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
		}
	} else {
		f32x16 acc[8];
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			#pragma unroll
			for (int e = 0; e < 16; e++) {
				acc[i][e] = 0.0f;
			}
		}
		for (int it = 0; it < iters; it++) {
			#pragma unroll
			for (int i = 0; i < 8; i++) {
				acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i >> 2], b[i & 3], acc[i], 0, 0, 0);
			}
		}
		#pragma unroll
		for (int i = 0; i < 8; i++) {
			#pragma unroll
			for (int e = 0; e < 16; e++) {
				s += acc[i][e];
			}
		}
	}
	if (s == 12345.0f) {                               /* keeps the loop alive; practically never true */
		out[0] = s;
	}
}

extern "C" int amd_matmul_mfma_probe(Dataflow_Handle * dataflow_handle, int stream_id, int iters, int mode, void * device_word,
									 uint64_t * flops) {
	hipStream_t stream;
	if (!dataflow_handle || !device_word || iters < 1 || mode < 0 || mode > 7 || resolve_stream(dataflow_handle, stream_id, &stream)) {
		fprintf(stderr, "Error: bad arguments to the MFMA rate probe...\n");
		return -1;
	}
	if (hipSetDevice(dataflow_handle->device_id) != hipSuccess) {
		return -1;
	}
	Hip_Device_Info * info = (Hip_Device_Info *) dataflow_handle->device_info;
	const int grid = info ? info->cu_count : 256;
	hipLaunchKernelGGL(mfma_rate_probe_kernel, dim3((unsigned int) grid), dim3(512), 0, stream, (float *) device_word, iters, mode);
	if (flops) {
		*flops = (uint64_t) grid * 8u * (uint64_t) iters * 8u * (2ull * 32 * 32 * 16);
	}
	return check_launch();
}

/* The streaming GEMM's skeleton and nothing else: what a k-tile step costs when it consists of the operand loads, the
 * multiplies and the barrier only.  One 512-thread work-group per compute unit; per step each of waves 0-3 issues
 * sixteen 16-byte-per-lane loads straight into one of two 64 KiB LDS stages (512 rows x 128 bytes, row stride 8 KiB:
 * a k-tile of two k-contiguous 256-row panels with K = 4096), every wave issues 64 v_mfma_f32_16x16x32_bf16 on
 * constant registers, then the loading waves wait for loads and all meet at a barrier.  A region is 64 steps (4 MiB);
 * `share` work-groups of a die read the same region at the same time; every pass moves on to regions not read
 * before, so with a source larger than the caches every line comes from HBM exactly once per `share` readers.
 * SLACK 1: the loads of a step are waited for at the end of that step (what two stages allow a GEMM); 2: at the end
 * of the next step (what three stages would allow; nothing reads the LDS here, so two are enough to land them in);
 * 0: never, and no barrier.  TOUCH: wave 4 reads four bytes of each line of this work-group's 1 / share of the lines
 * two steps ahead into LDS nobody reads, so that the loads proper find them in the L2.
 * VIA_REGS: a third stage that exists, in registers.  All eight waves load their share of a step (eight 16-byte loads
 * per lane) into one of two register sets at the start of the step and write the other set, requested a step earlier,
 * to an LDS stage with ds_write_b128 behind the multiplies, in front of the barrier: two steps of slack, paid with
 * 64 registers per lane and 64 KiB of LDS writes per step. */
template <int SLACK, bool LOAD, bool MFMA, bool TOUCH, bool VIA_REGS = false>
__global__ void __launch_bounds__(512) stream_probe_kernel(const char * src, unsigned int regions, int share, int passes, float * out) {
	constexpr unsigned int REGION = 4u << 20;
	constexpr int STEPS = 64;
	__shared__ __attribute__((aligned(16))) char stages[2][65536];
	const uint32_t stages_addr = (uint32_t) (uintptr_t) LDS_PTR(stages);
	const unsigned int die = blockIdx.x & 7, idx = blockIdx.x >> 3;
	const unsigned int groups = share == 0 ? 1 : (gridDim.x >> 3) / share * 8;       /* regions read at a time */
	const unsigned int group = share == 0 ? 0 : (idx / share) * 8 + die;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int tid = threadIdx.x & 255;
	const bool loader = wave < 4;
	f32x4_acc acc[16];
	#pragma unroll
	for (int i = 0; i < 16; i++) {
		acc[i] = f32x4_acc{0.0f, 0.0f, 0.0f, 0.0f};
	}
	bf16x8 a, b;
	#pragma unroll
	for (int e = 0; e < 8; e++) {
		a[e] = (__bf16) 0.0f;
		b[e] = (__bf16) 0.0f;
	}
	asm volatile("" : "+v"(a), "+v"(b));
	unsigned int stage = 0;
	if (share != 0 && idx >= (gridDim.x >> 3) / share * share) {
		return;                                        /* work-groups beyond the last full group of sharers */
	}
	if constexpr (VIA_REGS) {
		u32x4 set_a[8], set_b[8];
		const int total_steps = passes * STEPS;
		/* step gs of the launch: step gs % 64 of the region of pass gs / 64 */
#define PROBE_FETCH(set_, gs_) do { \
			const char * region_ = src + (size_t) ((group + (unsigned int) ((gs_) / STEPS) * groups) % regions) * REGION; \
			const __amdgpu_buffer_rsrc_t rs_ = __builtin_amdgcn_make_buffer_rsrc((void *) region_, 0, (int) REGION, 0x00020000); \
			_Pragma("unroll") \
			for (int i = 0; i < 8; i++) { \
				set_[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_, (int) ((i * 64 + (threadIdx.x >> 3)) * 8192 + ((gs_) % STEPS) * 128 + (threadIdx.x & 7) * 16), 0, 0); \
			} \
		} while (0)
#define PROBE_LAND(set_, stage_) do { \
			_Pragma("unroll") \
			for (int i = 0; i < 8; i++) { \
				*((u32x4 *) (stages[stage_] + (i * 512 + threadIdx.x) * 16)) = set_[i]; \
			} \
		} while (0)
#define PROBE_MFMAS() do { \
			if (MFMA) { \
				_Pragma("unroll") \
				for (int m = 0; m < 64; m++) { \
					acc[m & 15] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[m & 15], 0, 0, 0); \
				} \
			} \
		} while (0)
		PROBE_FETCH(set_a, 0);
		for (int gs = 0; gs < total_steps; gs += 2) {              /* 64 steps a pass: total_steps is even */
			PROBE_FETCH(set_b, gs + 1);
			__builtin_amdgcn_sched_barrier(0);             /* the requests go out in front of the multiplies, not behind the writes */
			PROBE_MFMAS();
			__builtin_amdgcn_sched_barrier(0);
			PROBE_LAND(set_a, 0);
			__syncthreads();
			PROBE_FETCH(set_a, min(gs + 2, total_steps - 1));  /* the last one is fetched again and not used */
			__builtin_amdgcn_sched_barrier(0);
			PROBE_MFMAS();
			__builtin_amdgcn_sched_barrier(0);
			PROBE_LAND(set_b, 1);
			__syncthreads();
		}
#undef PROBE_FETCH
#undef PROBE_LAND
#undef PROBE_MFMAS
		float s = 0.0f;
		#pragma unroll
		for (int i = 0; i < 16; i++) {
			s += acc[i][0];
		}
		if (s != 0.0f) {
			out[0] = s;
		}
		return;
	}
	for (int p = 0; p < passes; p++) {
		const i32x4 rsrc = make_raw_rsrc(src + (size_t) ((group + (unsigned int) p * groups) % regions) * REGION, REGION);
		for (int st = 0; st < STEPS; st++) {
			if (TOUCH && wave == 4 && st + 2 < STEPS) {
				const int sc = share == 0 ? (int) gridDim.x : share;
				const int si = share == 0 ? (int) blockIdx.x : (int) (idx % share);
				const int lo = 512 * si / sc, hi = 512 * (si + 1) / sc;
				for (int r0 = lo; r0 < hi; r0 += 64) {
					const int row = r0 + (int) (threadIdx.x & 63);
					const uint32_t voff = row < hi ? (uint32_t) (row * 8192 + (st + 2) * 128) : VOFF_INVALID;
					const uint32_t dump = (uint32_t) __builtin_amdgcn_readfirstlane((int) (stages_addr + 2 * 65536 - 256));
					asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dword %1, %2, 0 offen lds" : : "s"(dump), "v"(voff), "s"(rsrc) : "memory", "m0");
				}
			}
			if (LOAD && loader) {
				#pragma unroll
				for (int i = 0; i < 16; i++) {
					const uint32_t voff = (uint32_t) ((i * 32 + (tid >> 3)) * 8192 + st * 128 + (tid & 7) * 16);
					dma_load16(voff, rsrc, stages_addr + stage * 65536u + (uint32_t) (i * 256 + wave * 64) * 16u);
				}
			}
			if (MFMA) {
				#pragma unroll
				for (int m = 0; m < 64; m++) {
					acc[m & 15] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[m & 15], 0, 0, 0);
				}
			}
			stage ^= 1u;
			if (SLACK != 0) {
				if (LOAD && loader) {
					if (SLACK == 1) {
						WAIT_VMCNT(0);
					} else {
						WAIT_VMCNT(16);
					}
				}
				__syncthreads();
			}
		}
	}
	WAIT_VMCNT(0);
	float s = 0.0f;
	#pragma unroll
	for (int i = 0; i < 16; i++) {
		s += acc[i][0];
	}
	if (s != 0.0f) {                                   /* keeps the multiplies alive; never true (the operands are zero) */
		out[0] = s;
	}
}

extern "C" int amd_matmul_stream_probe(Dataflow_Handle * dataflow_handle, int stream_id, const void * src, uint64_t src_bytes,
									   int share, int slack, int flags, int passes, void * device_word) {
	hipStream_t stream;
	const bool share_ok = share == 0 || share == 1 || share == 2 || share == 4 || share == 8 || share == 16 || share == 32;
	const bool touch = (flags & AMD_STREAM_PROBE_TOUCH) != 0, no_loads = (flags & AMD_STREAM_PROBE_NO_LOADS) != 0, no_mfmas = (flags & AMD_STREAM_PROBE_NO_MFMAS) != 0;
	const bool via_regs = (flags & AMD_STREAM_PROBE_VIA_REGISTERS) != 0;
	if (!dataflow_handle || !src || !device_word || src_bytes < (4u << 20) || !share_ok || slack < 0 || slack > 2 || flags < 0 || flags > 15
			|| passes < 1 || (touch && (no_loads || slack != 1)) || (via_regs && (no_loads || touch || slack != 2))
			|| resolve_stream(dataflow_handle, stream_id, &stream)) {
		fprintf(stderr, "Error: bad arguments to the stream probe...\n");
		return -1;
	}
	if (hipSetDevice(dataflow_handle->device_id) != hipSuccess) {
		return -1;
	}
	Hip_Device_Info * info = (Hip_Device_Info *) dataflow_handle->device_info;
	const unsigned int grid = (unsigned int) ((info ? info->cu_count : 256) & ~7);
	const uint64_t regions64 = src_bytes / (4u << 20);
	const unsigned int regions = regions64 > 0x7fffffffull ? 0x7fffffffu : (unsigned int) regions64;
#define PROBE(SLACK_, LOAD_, MFMA_, TOUCH_) \
	hipLaunchKernelGGL((stream_probe_kernel<SLACK_, LOAD_, MFMA_, TOUCH_>), dim3(grid), dim3(512), 0, stream, (const char *) src, regions, share, passes, (float *) device_word)
#define PROBE_SLACK(SLACK_) do { \
		if (touch) { if (no_mfmas) { PROBE(1, true, false, true); } else { PROBE(1, true, true, true); } } \
		else if (no_loads) { PROBE(SLACK_, false, true, false); } \
		else if (no_mfmas) { PROBE(SLACK_, true, false, false); } \
		else { PROBE(SLACK_, true, true, false); } \
	} while (0)
	if (no_loads && no_mfmas) {
		fprintf(stderr, "Error: the stream probe needs loads or multiplies...\n");
		return -1;
	}
	if (via_regs) {
		if (no_mfmas) {
			hipLaunchKernelGGL((stream_probe_kernel<2, true, false, false, true>), dim3(grid), dim3(512), 0, stream, (const char *) src, regions, share, passes, (float *) device_word);
		} else {
			hipLaunchKernelGGL((stream_probe_kernel<2, true, true, false, true>), dim3(grid), dim3(512), 0, stream, (const char *) src, regions, share, passes, (float *) device_word);
		}
	} else if (slack == 0) { PROBE_SLACK(0); } else if (slack == 1) { PROBE_SLACK(1); } else { PROBE_SLACK(2); }
#undef PROBE_SLACK
#undef PROBE
	return check_launch();
}
