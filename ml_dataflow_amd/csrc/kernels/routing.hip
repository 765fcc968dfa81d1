/*
 * routing.hip -- top-k expert selection and the dispatch permutation, for gfx950 (wave64).
 *
 * default_select_experts_bf16_kernel   replaces backends/nvidia/src/ops/src/native/src/moe/select_experts.cu:302-594
 * default_build_expert_mapping_kernel  replaces .../moe/build_expert_mapping.cu:18-103
 * default_router_gate_bwd_x_bf16_bf16_kernel replaces .../moe/router_gate_bwd_x.cu:7-57
 *
 * Both routing kernels move at most a few MB and are latency-bound; the design goal is exact integer
 * results with every lane busy, not bandwidth.
 */
#include "moe_common.h"

#define SELECT_TOKENS_PER_BLOCK 64          /* one wave, one token per lane */
#define SELECT_EXPERT_CHUNK 128             /* experts staged in LDS per pass */
#define SELECT_ROW_DWORDS (SELECT_EXPERT_CHUNK / 2 + 1)   /* odd stride: lanes walk their rows conflict-free */
#define SELECT_MAX_DYNAMIC_K 32

/* The reference keeps K (value, expert) slots per token and walks the experts in ascending order
 * (select_experts.cu:417-468): an expert enters only if its logit is STRICTLY greater than the current
 * minimum slot, it takes that slot's place, and the new minimum is the smallest value with ties going to
 * the slot that holds the LARGER expert id.  The slot order is part of the result.  Here one lane replays
 * exactly that walk for one token with the slots in registers (K known at compile time). */
template <int K>
struct TopKSlots {
	float val[K];
	int idx[K];
	float min_val;
	float max_val;
	int min_slot;

	__device__ __forceinline__ void reset() {
		#pragma unroll
		for (int k = 0; k < K; k++) {
			val[k] = -INFINITY;
			idx[k] = 0xFFFF;
		}
		min_val = -INFINITY;
		max_val = -INFINITY;
		min_slot = 0;
	}

	__device__ __forceinline__ void offer(float v, int e) {
		if (v > min_val) {
			max_val = fmaxf(max_val, v);
			#pragma unroll
			for (int k = 0; k < K; k++) {
				if (k == min_slot) {
					val[k] = v;
					idx[k] = e;
				}
			}
			float mv = INFINITY;
			int ms = 0;
			int me = 0xFFFF;
			#pragma unroll
			for (int k = 0; k < K; k++) {
				if ((val[k] < mv) || (val[k] == mv && idx[k] > me)) {
					mv = val[k];
					ms = k;
					me = idx[k];
				}
			}
			min_val = mv;
			min_slot = ms;
		}
	}
};

/* stage logits [tokens t0..t0+64) x experts [c0..c0+SELECT_EXPERT_CHUNK) into LDS, -inf beyond the matrix */
__device__ __forceinline__ void select_stage_tile(const bf16_t * __restrict__ logits, uint32_t * tile,
												  int t0, int c0, int total_tokens, int n_experts) {
	const int vec_per_row = SELECT_EXPERT_CHUNK / 8;
	const bool rows_vectorizable = ((n_experts & 7) == 0) && ((((uintptr_t) logits) & 15) == 0);
	const uint32_t ninf2 = 0xFF80FF80u;
	for (int i = threadIdx.x; i < SELECT_TOKENS_PER_BLOCK * vec_per_row; i += blockDim.x) {
		int r = i / vec_per_row;
		int v = i - r * vec_per_row;
		int t = t0 + r;
		int e0 = c0 + v * 8;
		uint32_t * dst = tile + r * SELECT_ROW_DWORDS + v * 4;
		if (t < total_tokens && rows_vectorizable && e0 + 8 <= n_experts) {
			u32x4 q = *((const u32x4 *) (logits + (size_t) t * n_experts + e0));
			dst[0] = q.x; dst[1] = q.y; dst[2] = q.z; dst[3] = q.w;
		} else {
			for (int j = 0; j < 4; j++) {
				uint32_t pair = ninf2;
				if (t < total_tokens) {
					int ea = e0 + 2 * j;
					uint32_t lo = (ea < n_experts) ? logits[(size_t) t * n_experts + ea] : 0xFF80u;
					uint32_t hi = (ea + 1 < n_experts) ? logits[(size_t) t * n_experts + ea + 1] : 0xFF80u;
					pair = lo | (hi << 16);
				}
				dst[j] = pair;
			}
		}
	}
}

template <int K>
__device__ __forceinline__ void select_tokens_static(int total_tokens, int n_experts, const bf16_t * __restrict__ logits,
													 float * __restrict__ weights, uint16_t * __restrict__ chosen,
													 uint32_t * tile, int * hist) {
	const int t0 = blockIdx.x * SELECT_TOKENS_PER_BLOCK;
	const int t = t0 + threadIdx.x;
	TopKSlots<K> s;
	s.reset();
	for (int c0 = 0; c0 < n_experts; c0 += SELECT_EXPERT_CHUNK) {
		__syncthreads();
		select_stage_tile(logits, tile, t0, c0, total_tokens, n_experts);
		__syncthreads();
		const uint32_t * row = tile + threadIdx.x * SELECT_ROW_DWORDS;
		int lim = min(SELECT_EXPERT_CHUNK, n_experts - c0);
		for (int j = 0; j < lim; j += 2) {
			uint32_t pair = row[j >> 1];
			s.offer(lo_f32(pair), c0 + j);
			if (j + 1 < lim) {
				s.offer(hi_f32(pair), c0 + j + 1);
			}
		}
	}
	if (t < total_tokens) {
		/* softmax over the K slots; the reference subtracts the max in bf16 before expf (select_experts.cu:480,488) */
		float ex[K];
		float sum = 0.0f;
		#pragma unroll
		for (int k = 0; k < K; k++) {
			ex[k] = expf(bf16_to_f32(f32_to_bf16(s.val[k] - s.max_val)));
			sum += ex[k];
		}
		#pragma unroll
		for (int k = 0; k < K; k++) {
			weights[(size_t) t * K + k] = ex[k] / sum;
			chosen[(size_t) t * K + k] = (uint16_t) s.idx[k];
			if (s.idx[k] < n_experts) {
				atomicAdd(&hist[s.idx[k]], 1);
			}
		}
	}
}

/* any K up to SELECT_MAX_DYNAMIC_K: same walk with the slots in LDS (one column per lane) */
__device__ void select_tokens_dynamic(int total_tokens, int n_experts, int K, const bf16_t * __restrict__ logits,
									  float * __restrict__ weights, uint16_t * __restrict__ chosen,
									  uint32_t * tile, int * hist, float * slot_val, int * slot_idx) {
	const int t0 = blockIdx.x * SELECT_TOKENS_PER_BLOCK;
	const int lane = threadIdx.x;
	const int t = t0 + lane;
	/* slot k of this lane lives at [k * 64 + lane] */
	for (int k = 0; k < K; k++) {
		slot_val[k * SELECT_TOKENS_PER_BLOCK + lane] = -INFINITY;
		slot_idx[k * SELECT_TOKENS_PER_BLOCK + lane] = 0xFFFF;
	}
	float min_val = -INFINITY, max_val = -INFINITY;
	int min_slot = 0;
	for (int c0 = 0; c0 < n_experts; c0 += SELECT_EXPERT_CHUNK) {
		__syncthreads();
		select_stage_tile(logits, tile, t0, c0, total_tokens, n_experts);
		__syncthreads();
		const uint32_t * row = tile + lane * SELECT_ROW_DWORDS;
		int lim = min(SELECT_EXPERT_CHUNK, n_experts - c0);
		for (int j = 0; j < lim; j++) {
			uint32_t pair = row[j >> 1];
			float v = (j & 1) ? hi_f32(pair) : lo_f32(pair);
			if (v > min_val) {
				max_val = fmaxf(max_val, v);
				slot_val[min_slot * SELECT_TOKENS_PER_BLOCK + lane] = v;
				slot_idx[min_slot * SELECT_TOKENS_PER_BLOCK + lane] = c0 + j;
				float mv = INFINITY;
				int ms = 0, me = 0xFFFF;
				for (int k = 0; k < K; k++) {
					float cv = slot_val[k * SELECT_TOKENS_PER_BLOCK + lane];
					int ce = slot_idx[k * SELECT_TOKENS_PER_BLOCK + lane];
					if ((cv < mv) || (cv == mv && ce > me)) {
						mv = cv; ms = k; me = ce;
					}
				}
				min_val = mv;
				min_slot = ms;
			}
		}
	}
	if (t < total_tokens) {
		float sum = 0.0f;
		for (int k = 0; k < K; k++) {
			sum += expf(bf16_to_f32(f32_to_bf16(slot_val[k * SELECT_TOKENS_PER_BLOCK + lane] - max_val)));
		}
		for (int k = 0; k < K; k++) {
			float ex = expf(bf16_to_f32(f32_to_bf16(slot_val[k * SELECT_TOKENS_PER_BLOCK + lane] - max_val)));
			int e = slot_idx[k * SELECT_TOKENS_PER_BLOCK + lane];
			weights[(size_t) t * K + k] = ex / sum;
			chosen[(size_t) t * K + k] = (uint16_t) e;
			if (e < n_experts) {
				atomicAdd(&hist[e], 1);
			}
		}
	}
}

/* Launch: grid = ceil(T / 64), block = 64, dynamic LDS = n_experts ints (histogram).
 * expert_counts has n_experts + 1 entries, zeroed by the caller; the last one is the block ticket and ends
 * equal to gridDim.x.  The block that draws the last ticket scans the counts (exclusive) into
 * expert_counts_cumsum and copies them to host_expert_counts (device-visible host memory). */
extern "C" __global__ void __launch_bounds__(SELECT_TOKENS_PER_BLOCK)
default_select_experts_bf16_kernel(int total_tokens, int n_experts, int top_k_experts, const bf16_t * X_routed,
								   float * token_expert_weights, uint16_t * chosen_experts, int * expert_counts,
								   int * expert_counts_cumsum, int * host_expert_counts) {
	__shared__ uint32_t tile[SELECT_TOKENS_PER_BLOCK * SELECT_ROW_DWORDS];
	__shared__ int ticket;
	extern __shared__ int hist[];

	for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
		hist[e] = 0;
	}
	/* the first __syncthreads inside the walk orders the clear before any atomicAdd */

	switch (top_k_experts) {
		case 1: select_tokens_static<1>(total_tokens, n_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 2: select_tokens_static<2>(total_tokens, n_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 4: select_tokens_static<4>(total_tokens, n_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 6: select_tokens_static<6>(total_tokens, n_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 8: select_tokens_static<8>(total_tokens, n_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		default: {
			/* the launch configuration reserves 64 * K * 8 bytes after the histogram for the slots */
			float * slot_val = (float *) (hist + n_experts);
			int * slot_idx = (int *) (slot_val + top_k_experts * SELECT_TOKENS_PER_BLOCK);
			select_tokens_dynamic(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts,
								  tile, hist, slot_val, slot_idx);
		}
	}

	__syncthreads();
	for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
		int c = hist[e];
		if (c) {
			atomicAdd(&expert_counts[e], c);
		}
	}
	__threadfence();
	__syncthreads();
	if (threadIdx.x == 0) {
		ticket = atomicAdd(&expert_counts[n_experts], 1);
	}
	__syncthreads();
	if (ticket != (int) gridDim.x - 1) {
		return;
	}
	__threadfence();

	/* last block: wave-wide exclusive scan, 64 experts per step */
	const int lane = threadIdx.x;
	int carry = 0;
	for (int base = 0; base < n_experts; base += WAVE) {
		int e = base + lane;
		int c = (e < n_experts) ? __hip_atomic_load(&expert_counts[e], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : 0;
		int incl = c;
		#pragma unroll
		for (int off = 1; off < WAVE; off <<= 1) {
			int up = __shfl_up(incl, off, WAVE);
			if (lane >= off) {
				incl += up;
			}
		}
		if (e < n_experts) {
			expert_counts_cumsum[e] = carry + incl - c;
			host_expert_counts[e] = c;
		}
		carry += __shfl(incl, WAVE - 1, WAVE);
	}
	__threadfence_system();
}

/* ------------------------------------------------------------------ build_expert_mapping */

#define BUILD_THREADS 256
#define BUILD_WAVES (BUILD_THREADS / WAVE)

/* Stable counting sort of the R = num_tokens * K routed entries by expert id, with no cross-block
 * communication: block b owns entries [b*tile, (b+1)*tile); it counts the whole id array once (total
 * per expert, and how many precede its tile), scans the totals itself, then its four waves rank their
 * own quarter of the tile in entry order with ballots.  Positions therefore ascend with the token id
 * inside every expert, which is one of the orders the reference's atomics can produce
 * (build_expert_mapping.cu:47-51, 90-100) made deterministic.
 *
 * expert_counts_cumsum is taken to be the exclusive scan of the per-expert totals (what select_experts
 * leaves, select_experts.cu:573-575); it is rebuilt from the ids rather than read, and block 0 stores the
 * inclusive scan over it, the state the reference's atomicAdd leaves behind (build_expert_mapping.cu:66).
 *
 * Launch: grid = ceil(R / tile) with tile = entries_per_block (a multiple of 256, passed through the
 * launch configuration as gridDim -> tile = ceil(R / gridDim) rounded up to 256), block = 256,
 * dynamic LDS = 6 * num_routed_experts ints. */
extern "C" __global__ void __launch_bounds__(BUILD_THREADS)
default_build_expert_mapping_kernel(int num_tokens, int num_routed_experts, int num_selected_experts,
									const uint16_t * chosen_experts, int * expert_counts_cumsum,
									int * expert_mapping, int * token_mapping) {
	extern __shared__ int lds[];
	const int E = num_routed_experts;
	int * tot = lds;                    /* [E] entries per expert in the whole array */
	int * pre = lds + E;                /* [E] entries per expert before this block's tile */
	int * run = lds + 2 * E;            /* [BUILD_WAVES][E] per-wave counts, then per-wave running positions */

	const long R = (long) num_tokens * (long) num_selected_experts;
	long tile = (R + gridDim.x - 1) / gridDim.x;
	tile = (tile + BUILD_THREADS - 1) / BUILD_THREADS * BUILD_THREADS;
	const long sub = tile / BUILD_WAVES;               /* multiple of 64 */
	const long tile_lo = (long) blockIdx.x * tile;
	const long tile_hi = min(tile_lo + tile, R);

	for (int i = threadIdx.x; i < 6 * E; i += BUILD_THREADS) {
		lds[i] = 0;
	}
	__syncthreads();

	/* pass 1: histogram of everything, 8 ids per 16-byte load */
	const long nvec = R / 8;
	const bool aligned = ((((uintptr_t) chosen_experts) & 15) == 0);
	if (aligned) {
		const u32x4 * ids = (const u32x4 *) chosen_experts;
		for (long v = threadIdx.x; v < nvec; v += BUILD_THREADS) {
			u32x4 q = ids[v];
			uint32_t w[4] = {q.x, q.y, q.z, q.w};
			long i0 = v * 8;
			#pragma unroll
			for (int j = 0; j < 8; j++) {
				int e = (int) ((w[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu);
				long i = i0 + j;
				if (e < E) {
					atomicAdd(&tot[e], 1);
					if (i < tile_lo) {
						atomicAdd(&pre[e], 1);
					} else if (i < tile_hi) {
						atomicAdd(&run[(int) ((i - tile_lo) / sub) * E + e], 1);
					}
				}
			}
		}
	}
	for (long i = (aligned ? nvec * 8 : 0) + threadIdx.x; i < R; i += BUILD_THREADS) {
		int e = chosen_experts[i];
		if (e < E) {
			atomicAdd(&tot[e], 1);
			if (i < tile_lo) {
				atomicAdd(&pre[e], 1);
			} else if (i < tile_hi) {
				atomicAdd(&run[(int) ((i - tile_lo) / sub) * E + e], 1);
			}
		}
	}
	__syncthreads();

	/* exclusive scan of tot by wave 0; pre[e] becomes the first position of this block's entries of expert e */
	const int lane = threadIdx.x & (WAVE - 1);
	const int wave = threadIdx.x / WAVE;
	if (wave == 0) {
		int carry = 0;
		for (int base = 0; base < E; base += WAVE) {
			int e = base + lane;
			int c = (e < E) ? tot[e] : 0;
			int incl = c;
			#pragma unroll
			for (int off = 1; off < WAVE; off <<= 1) {
				int up = __shfl_up(incl, off, WAVE);
				if (lane >= off) {
					incl += up;
				}
			}
			if (e < E) {
				int excl = carry + incl - c;
				pre[e] += excl;
				if (blockIdx.x == 0) {
					expert_counts_cumsum[e] = excl + c;
				}
			}
			carry += __shfl(incl, WAVE - 1, WAVE);
		}
	}
	__syncthreads();
	/* per-wave counts -> per-wave starting positions */
	for (int e = threadIdx.x; e < E; e += BUILD_THREADS) {
		int pos = pre[e];
		#pragma unroll
		for (int w = 0; w < BUILD_WAVES; w++) {
			int c = run[w * E + e];
			run[w * E + e] = pos;
			pos += c;
		}
	}
	__syncthreads();

	/* pass 2: each wave walks its quarter of the tile 64 entries at a time */
	int * my_run = run + wave * E;
	const long lo = tile_lo + (long) wave * sub;
	const long hi = min(lo + sub, tile_hi);
	for (long i0 = lo; i0 < hi; i0 += WAVE) {
		long i = i0 + lane;
		bool valid = i < hi;
		int e = valid ? (int) chosen_experts[i] : -1;
		valid = valid && (e < E);
		int slot = -1;
		uint64_t pending = __ballot(valid);
		while (pending) {
			int leader = __ffsll((long long) pending) - 1;
			int le = __shfl(e, leader, WAVE);
			bool mine = valid && (e == le);
			uint64_t m = __ballot(mine);
			int start = my_run[le];
			if (mine) {
				slot = start + __popcll(m & lanemask_lt());
			}
			if (lane == leader) {
				my_run[le] = start + __popcll(m);
			}
			pending &= ~m;
		}
		if (valid) {
			expert_mapping[slot] = (int) (i / num_selected_experts);
			token_mapping[i] = slot;
		}
	}
}

/* ------------------------------------------------------------------ router_gate_bwd_x */

/* Softmax-over-selected backward, in place on the K chosen columns of dX_routed [T, E]
 * (router_gate_bwd_x.cu:7-57): g_k = p_k * (d_k - sum_j d_j p_j).  One lane per token.
 * Launch: grid = ceil(T / 256), block = 256. */
extern "C" __global__ void __launch_bounds__(256)
default_router_gate_bwd_x_bf16_bf16_kernel(int num_tokens, int num_routed_experts, int top_k_active,
										   const uint16_t * chosen_experts, const float * token_expert_weights,
										   bf16_t * dX_routed) {
	int t = blockIdx.x * blockDim.x + threadIdx.x;
	if (t >= num_tokens) {
		return;
	}
	const uint16_t * c = chosen_experts + (size_t) t * top_k_active;
	const float * p = token_expert_weights + (size_t) t * top_k_active;
	bf16_t * d = dX_routed + (size_t) t * num_routed_experts;
	float m = 0.0f;
	for (int k = 0; k < top_k_active; k++) {
		m += bf16_to_f32(d[c[k]]) * p[k];
	}
	for (int k = 0; k < top_k_active; k++) {
		d[c[k]] = f32_to_bf16(p[k] * (bf16_to_f32(d[c[k]]) - m));
	}
}
