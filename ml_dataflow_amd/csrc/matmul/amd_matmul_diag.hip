/*
 * amd_matmul_diag.hip -- diagnostic kernels of the gfx950 GEMM work, in a library of their own (libamd_matmul_diag.so):
 * nothing in the product path loads it.  bench.py's mfma_only_* and gemm_stream_probe workloads and one GPU test do.
 *
 *   amd_matmul_mfma_probe     nothing but matrix instructions out of registers: what the card sustains under its power limit
 *   amd_matmul_stream_probe   the streaming GEMM's skeleton (operand loads into LDS stages, multiplies, a barrier) over a
 *                             table of data temperatures, sharing degrees and waits: what a k-tile step costs
 * Declared in include/amd_matmul_diag.h.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "dataflow_amd.h"
#include "amd_matmul_diag.h"
#include "gemm_kernel.h"

static int check_launch(void) {
	hipError_t e = hipGetLastError();
	if (e != hipSuccess) {
		fprintf(stderr, "Error: probe kernel launch failed: %s...\n", hipGetErrorString(e));
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
		fprintf(stderr, "Error: trying to launch a probe on stream id %d, but only have %d streams...\n", stream_id, handle->num_streams);
		return -1;
	}
	*stream = ((hipStream_t *) handle->streams)[stream_id];
	return 0;
}

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
__global__ void __launch_bounds__(512) stream_probe_kernel(const char * src, unsigned int regions, int share, int passes, float * out, int rotate, int per_group_clocks, int all_waves_load) {
	const long long clock_start = wall_clock64();
	constexpr unsigned int REGION = 4u << 20;
	constexpr int STEPS = 64;
	__shared__ __attribute__((aligned(16))) char stages[2][65536];
	const uint32_t stages_addr = (uint32_t) (uintptr_t) LDS_PTR(stages);
	const unsigned int die = blockIdx.x & 7, idx = blockIdx.x >> 3;
	const unsigned int groups = share == 0 ? 1 : (gridDim.x >> 3) / share * 8;       /* regions read at a time */
	const unsigned int group = share == 0 ? 0 : (idx / share) * 8 + die;
	const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
	const int tid = threadIdx.x & 255;
	const bool loader = wave < 4 || all_waves_load;  /* all_waves_load: eight loads per lane and step in every wave instead of sixteen in four */
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
	/* rotate: sharer i of a region takes its steps in the order i * rotate, i * rotate + 1, ... (wrapping), so that the
	 * work-groups that share a region do not ask for the same lines at the same time */
	const int first_step = (share > 1 ? (int) (idx % (unsigned int) share) * rotate : 0) % STEPS;
	for (int p = 0; p < passes; p++) {
		const i32x4 rsrc = make_raw_rsrc(src + (size_t) ((group + (unsigned int) p * groups) % regions) * REGION, REGION);
		for (int step = 0; step < STEPS; step++) {
			const int st = (step + first_step) & (STEPS - 1);
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
			if (LOAD && loader && !all_waves_load) {
				#pragma unroll
				for (int i = 0; i < 16; i++) {
					const uint32_t voff = (uint32_t) ((i * 32 + (tid >> 3)) * 8192 + st * 128 + (tid & 7) * 16);
					dma_load16(voff, rsrc, stages_addr + stage * 65536u + (uint32_t) (i * 256 + wave * 64) * 16u);
				}
			}
			if (LOAD && all_waves_load) {
				#pragma unroll
				for (int i = 0; i < 8; i++) {
					const uint32_t voff = (uint32_t) ((i * 64 + (threadIdx.x >> 3)) * 8192 + st * 128 + (threadIdx.x & 7) * 16);
					dma_load16(voff, rsrc, stages_addr + stage * 65536u + (uint32_t) (i * 512 + wave * 64) * 16u);
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
	if (per_group_clocks && threadIdx.x == 0) {       /* ticks of the 100 MHz wall clock this work-group ran */
		out[1 + blockIdx.x] = (float) (wall_clock64() - clock_start);
	}
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
	const int known_flags = 15 | (63 << AMD_STREAM_PROBE_ROTATE_SHIFT) | AMD_STREAM_PROBE_PER_GROUP_CLOCKS | AMD_STREAM_PROBE_ALL_WAVES_LOAD;
	if (flags < 0 || (flags & ~known_flags)) {
		fprintf(stderr, "Error: unknown flags for the stream probe...\n");
		return -1;
	}
	const int rotate = (flags >> AMD_STREAM_PROBE_ROTATE_SHIFT) & 63;
	const int per_group_clocks = (flags & AMD_STREAM_PROBE_PER_GROUP_CLOCKS) != 0;
	const int all_waves_load = (flags & AMD_STREAM_PROBE_ALL_WAVES_LOAD) != 0;
	flags &= (1 << AMD_STREAM_PROBE_ROTATE_SHIFT) - 1;
	if (!dataflow_handle || !src || !device_word || src_bytes < (4u << 20) || !share_ok || slack < 0 || slack > 2 || flags < 0 || flags > 15
			|| ((rotate || all_waves_load || per_group_clocks) && via_regs) || ((rotate || all_waves_load) && touch) || (all_waves_load && slack == 2)
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
	hipLaunchKernelGGL((stream_probe_kernel<SLACK_, LOAD_, MFMA_, TOUCH_>), dim3(grid), dim3(512), 0, stream, (const char *) src, regions, share, passes, (float *) device_word, rotate, per_group_clocks, all_waves_load)
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
			hipLaunchKernelGGL((stream_probe_kernel<2, true, false, false, true>), dim3(grid), dim3(512), 0, stream, (const char *) src, regions, share, passes, (float *) device_word, 0, 0, 0);
		} else {
			hipLaunchKernelGGL((stream_probe_kernel<2, true, true, false, true>), dim3(grid), dim3(512), 0, stream, (const char *) src, regions, share, passes, (float *) device_word, 0, 0, 0);
		}
	} else if (slack == 0) { PROBE_SLACK(0); } else if (slack == 1) { PROBE_SLACK(1); } else { PROBE_SLACK(2); }
#undef PROBE_SLACK
#undef PROBE
	return check_launch();
}
