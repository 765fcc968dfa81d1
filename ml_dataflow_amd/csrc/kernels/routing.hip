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

#define SELECT_TOKENS_PER_BLOCK 32          /* a group of LANES lanes per token, LANES = the power of two >= K */
#define SELECT_EXPERT_CHUNK 128             /* experts staged in LDS per pass */
#define SELECT_ROW_DWORDS (SELECT_EXPERT_CHUNK / 2 + 1)   /* odd stride: the groups of a wave read their rows conflict-free */
#define SELECT_MAX_K 32

/* The reference keeps K (value, expert) slots per token and walks the experts in ascending order
 * (select_experts.cu:417-468): an expert enters only if its logit is STRICTLY greater than the current
 * minimum slot, it takes that slot's place, and the new minimum is the smallest value with ties going to
 * the slot that holds the LARGER expert id (among never-filled slots, which all hold -inf / 0xFFFF, the
 * lowest slot).  The slot order is part of the result.
 *
 * Here a group of LANES lanes replays exactly that walk for one token with ONE SLOT PER LANE: every lane sees
 * the same logit, the lane whose slot is the current minimum takes it, and the new minimum is found with
 * log2(LANES) cross-lane steps instead of a serial pass over K slots.  The walk itself stays sequential in
 * the experts, as the result depends on their order.  Lanes beyond K hold +inf and never win. */

/* lane i <-> lane i ^ 1, i ^ 2 (inside quads), 7 - i (inside 8), 15 - i (inside 16): after the steps before it each
 * mirror pairs a lane with one from the other half, which is all a reduction needs */
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
	return (uint32_t) __builtin_amdgcn_update_dpp((int) v, (int) v, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
__device__ __forceinline__ void slot_min_step(float & val, uint32_t & key) {
	const float oval = __uint_as_float(dpp_u32<CTRL>(__float_as_uint(val)));
	const uint32_t okey = dpp_u32<CTRL>(key);
	const bool take = (oval < val) || (oval == val && okey > key);
	val = take ? oval : val;
	key = take ? okey : key;
}
__device__ __forceinline__ void slot_min_step_32(float & val, uint32_t & key) {
	const float oval = __shfl_xor(val, 16, WAVE);
	const uint32_t okey = (uint32_t) __shfl_xor((int) key, 16, WAVE);
	const bool take = (oval < val) || (oval == val && okey > key);
	val = take ? oval : val;
	key = take ? okey : key;
}

/* stage logits [tokens t0..t0+SELECT_TOKENS_PER_BLOCK) x experts [c0..c0+SELECT_EXPERT_CHUNK) into LDS, -inf beyond the matrix */
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

template <int LANES>
__device__ __forceinline__ void select_tokens(int total_tokens, int n_experts, int K, const bf16_t * __restrict__ logits,
											  float * __restrict__ weights, uint16_t * __restrict__ chosen,
											  uint32_t * tile, int * hist) {
	const int t0 = blockIdx.x * SELECT_TOKENS_PER_BLOCK;
	const int group = threadIdx.x / LANES;                 /* token of the block */
	const int slot = threadIdx.x % LANES;
	const int t = t0 + group;
	const bool live = slot < K;
	float val = live ? -INFINITY : INFINITY;
	int idx = 0xFFFF;
	float min_val = -INFINITY;
	float max_val = -INFINITY;
	int min_slot = 0;

	for (int c0 = 0; c0 < n_experts; c0 += SELECT_EXPERT_CHUNK) {
		__syncthreads();
		select_stage_tile(logits, tile, t0, c0, total_tokens, n_experts);
		__syncthreads();
		const uint32_t * row = tile + group * SELECT_ROW_DWORDS;
		const int lim = min(SELECT_EXPERT_CHUNK, n_experts - c0);
		for (int j = 0; j < lim; j++) {
			const uint32_t pair = row[j >> 1];
			const float v = (j & 1) ? hi_f32(pair) : lo_f32(pair);
			const bool enters = v > min_val;                /* the same in every lane of the group */
			max_val = enters ? fmaxf(max_val, v) : max_val;
			if (enters && slot == min_slot) {
				val = v;
				idx = c0 + j;
			}
			if (LANES > 1) {
				/* smallest value; ties: larger expert id, then lower slot.  key = id * 64 + (63 - slot), larger wins */
				float mv = val;
				uint32_t mk = ((uint32_t) idx << 6) | (uint32_t) (63 - slot);
				slot_min_step<0xB1>(mv, mk);
				if (LANES > 2) { slot_min_step<0x4E>(mv, mk); }
				if (LANES > 4) { slot_min_step<0x141>(mv, mk); }
				if (LANES > 8) { slot_min_step<0x140>(mv, mk); }
				if (LANES > 16) { slot_min_step_32(mv, mk); }
				min_val = mv;
				min_slot = 63 - (int) (mk & 63u);
			} else {
				min_val = val;
			}
		}
	}
	if (t < total_tokens) {
		/* softmax over the K slots, summed in slot order; the reference subtracts the max in bf16 before expf
		 * (select_experts.cu:480,488) */
		const float ex = live ? expf(bf16_to_f32(f32_to_bf16(val - max_val))) : 0.0f;
		float sum = 0.0f;
		const int base = (threadIdx.x & (WAVE - 1)) - slot;
		for (int k = 0; k < K; k++) {
			sum += __shfl(ex, base + k, WAVE);
		}
		if (live) {
			weights[(size_t) t * K + slot] = ex / sum;
			chosen[(size_t) t * K + slot] = (uint16_t) idx;
			if (idx < n_experts) {
				atomicAdd(&hist[idx], 1);
			}
		}
	}
}

/* Launch: grid = ceil(T / 32), block = 32 * LANES with LANES the power of two >= top_k (1..32), dynamic LDS =
 * n_experts ints (histogram).
 * expert_counts has n_experts + 1 entries, zeroed by the caller; the last one is the block ticket and ends
 * equal to gridDim.x.  The block that draws the last ticket scans the counts (exclusive) into
 * expert_counts_cumsum and copies them to host_expert_counts (device-visible host memory). */
extern "C" __global__ void __launch_bounds__(SELECT_TOKENS_PER_BLOCK * SELECT_MAX_K)
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

	switch (blockDim.x / SELECT_TOKENS_PER_BLOCK) {
		case 1: select_tokens<1>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 2: select_tokens<2>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 4: select_tokens<4>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 8: select_tokens<8>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 16: select_tokens<16>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		default: select_tokens<32>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
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
	if (ticket != (int) gridDim.x - 1 || threadIdx.x >= WAVE) {
		return;
	}
	__threadfence();

	/* last block, first wave: wave-wide exclusive scan, 64 experts per step (a block of 32 threads is half a wave:
	 * its missing lanes read as zero in the shuffles below because they never pass e < n_experts) */
	const int lane = threadIdx.x;
	int carry = 0;
	for (int base = 0; base < n_experts; base += (int) min(blockDim.x, (unsigned int) WAVE)) {
		const int width = (int) min(blockDim.x, (unsigned int) WAVE);
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
		carry += __shfl(incl, width - 1, WAVE);
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
