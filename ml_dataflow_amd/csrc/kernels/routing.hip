/*
 * routing.hip -- top-k expert selection and the dispatch permutation, for gfx950 (wave64).
 *
 * default_select_experts_bf16_kernel   replaces backends/nvidia/src/ops/src/native/src/moe/select_experts.cu:302-594
 * default_select_experts_fp32_kernel   replaces .../moe/select_experts.cu:3-295 (the reference's fp16 and fp8 kernels
 *                                      of this op are empty, :298-300, :883-890, and have no counterpart here)
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
 * the experts, as the result depends on their order: its length is 64 dependent steps for 64 experts whatever the
 * token count, so a step is kept to a handful of instructions.  Lanes beyond K hold the largest key and never win. */

/* The walk compares and moves one 32-bit key per slot instead of a (value, expert) pair:
 *   high half: the logit's bf16 bits made monotonic (sort_key16: a larger value is a larger number; -0 counts as +0, as
 *              it does in a float comparison; a NaN becomes 0, below -inf, so it never enters, as no float comparison
 *              with a NaN holds)
 *   low half:  0xFFFF - expert id, so that among equal values the larger id is the smaller key; a never-filled slot
 *              holds (-inf, slot number): the lowest such slot is the minimum, and nothing displaces it but a real
 *              entry, since a logit of -inf is not strictly greater than -inf and never enters.
 * The minimum slot of the reference's rule is then the smallest key, one v_min_u32 per cross-lane step. */
#define KEY16_NEG_INF 0x007Fu
__device__ __forceinline__ uint32_t sort_key16(uint32_t bits) {
	const uint32_t mag = bits & 0x7FFFu;
	if (mag > 0x7F80u) {
		return 0u;
	}
	if (mag == 0u) {
		return 0x8000u;
	}
	return (bits & 0x8000u) ? (bits ^ 0xFFFFu) : (bits | 0x8000u);
}
__device__ __forceinline__ float sort_key16_value(uint32_t key) {
	const uint32_t bits = (key & 0x8000u) ? (key & 0x7FFFu) : (key ^ 0xFFFFu);
	return __uint_as_float(bits << 16);
}

/* lane i <-> lane i ^ 1, i ^ 2 (inside quads), 7 - i (inside 8), 15 - i (inside 16): after the steps before it each
 * mirror pairs a lane with one from the other half, which is all a reduction needs */
template <int CTRL>
__device__ __forceinline__ uint32_t key_min_step(uint32_t key) {
	const uint32_t other = (uint32_t) __builtin_amdgcn_update_dpp((int) key, (int) key, CTRL, 0xF, 0xF, false);
	return min(key, other);
}

/* stage logits [tokens t0..t0+SELECT_TOKENS_PER_BLOCK) x experts [c0..c0+SELECT_EXPERT_CHUNK) into LDS as 16-bit sort
 * keys, two per dword, -inf beyond the matrix */
__device__ __forceinline__ uint32_t sort_key_pair(uint32_t pair) {
	return sort_key16(pair & 0xFFFFu) | (sort_key16(pair >> 16) << 16);
}
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
			dst[0] = sort_key_pair(q.x); dst[1] = sort_key_pair(q.y); dst[2] = sort_key_pair(q.z); dst[3] = sort_key_pair(q.w);
		} else {
			for (int j = 0; j < 4; j++) {
				uint32_t pair = ninf2;
				if (t < total_tokens) {
					int ea = e0 + 2 * j;
					uint32_t lo = (ea < n_experts) ? logits[(size_t) t * n_experts + ea] : 0xFF80u;
					uint32_t hi = (ea + 1 < n_experts) ? logits[(size_t) t * n_experts + ea + 1] : 0xFF80u;
					pair = lo | (hi << 16);
				}
				dst[j] = sort_key_pair(pair);
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
	uint32_t key = live ? ((KEY16_NEG_INF << 16) | (uint32_t) slot) : 0xFFFFFFFFu;   /* lanes beyond K are never the minimum */
	uint32_t min_key = (KEY16_NEG_INF << 16);              /* slot 0's key: the same in every lane of the group */
	uint32_t max_key16 = KEY16_NEG_INF;                    /* largest value that entered */

	for (int c0 = 0; c0 < n_experts; c0 += SELECT_EXPERT_CHUNK) {
		__syncthreads();
		select_stage_tile(logits, tile, t0, c0, total_tokens, n_experts);
		__syncthreads();
		const uint32_t * row = tile + group * SELECT_ROW_DWORDS;
		const int lim = min(SELECT_EXPERT_CHUNK, n_experts - c0);
		/* experts in pairs (one LDS dword); an odd count's last partner is staged as -inf and never enters */
		for (int j = 0; j < lim; j += 2) {
			const uint32_t pair = row[j >> 1];
			#pragma unroll
			for (int h = 0; h < 2; h++) {
				const uint32_t k16 = h ? (pair >> 16) : (pair & 0xFFFFu);
				const bool enters = k16 > (min_key >> 16);      /* the same in every lane of the group */
				max_key16 = enters ? max(max_key16, k16) : max_key16;
				if (enters && key == min_key) {
					key = (k16 << 16) | (0xFFFFu - (uint32_t) (c0 + j + h));
				}
				if (LANES > 1) {
					uint32_t m = key_min_step<0xB1>(key);
					if (LANES > 2) { m = key_min_step<0x4E>(m); }
					if (LANES > 4) { m = key_min_step<0x141>(m); }
					if (LANES > 8) { m = key_min_step<0x140>(m); }
					if (LANES > 16) { m = min(m, (uint32_t) __shfl_xor((int) m, 16, WAVE)); }
					min_key = m;
				} else {
					min_key = key;
				}
			}
		}
	}
	if (t < total_tokens) {
		/* softmax over the K slots, summed in slot order; the reference subtracts the max in bf16 before expf
		 * (select_experts.cu:480,488) */
		const bool filled = live && (key >> 16) != KEY16_NEG_INF;
		const float val = filled ? sort_key16_value(key >> 16) : -INFINITY;
		const int idx = filled ? (int) (0xFFFFu - (key & 0xFFFFu)) : 0xFFFF;
		const float max_val = sort_key16_value(max_key16);
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

/* What follows the walk in every element type's kernel: the work-group's histogram goes to the device-wide counters,
 * and the work-group that draws the last ticket scans them.  `ticket`: one int of LDS. */
__device__ __forceinline__ void select_finish(int n_experts, const int * hist, int * ticket_lds, int * expert_counts,
											  int * expert_counts_cumsum, int * host_expert_counts) {
#define ticket (*ticket_lds)
	__syncthreads();
	/* The work-group's counts go to the device-wide counters with returning atomics, and the ticket is drawn once every
	 * lane holds its returned values: an atomic that has returned has been performed where all dies see it, so whoever
	 * draws the last ticket finds every work-group's counts there.  No fence: a release fence per work-group would write
	 * back the die's whole L2 each time, which made this kernel several times longer than its work. */
	for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
		int c = hist[e];
		if (c) {
			int before = __hip_atomic_fetch_add(&expert_counts[e], c, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
			asm volatile("" :: "v"(before));              /* the value has to arrive: the wait for it is what orders the ticket behind it */
		}
	}
	__syncthreads();
	if (threadIdx.x == 0) {
		ticket = __hip_atomic_fetch_add(&expert_counts[n_experts], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
	}
	__syncthreads();
	if (ticket != (int) gridDim.x - 1 || threadIdx.x >= WAVE) {
		return;
	}

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
#undef ticket
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

	select_finish(n_experts, hist, &ticket, expert_counts, expert_counts_cumsum, host_expert_counts);
}

/* ---- fp32 logits (select_experts.cu:3-295): the same walk on float values; the softmax difference is not rounded ---- */

template <int CTRL>
__device__ __forceinline__ uint32_t dpp_u32(uint32_t v) {
	return (uint32_t) __builtin_amdgcn_update_dpp((int) v, (int) v, CTRL, 0xF, 0xF, false);
}
/* smallest value; ties: larger expert id, then lower slot.  key = id * 64 + (63 - slot), the larger key wins */
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

#define SELECT_F32_CHUNK 64                      /* experts staged per pass: 32 tokens x 65 floats of LDS */
#define SELECT_F32_ROW (SELECT_F32_CHUNK + 1)

template <int LANES>
__device__ __forceinline__ void select_tokens_f32(int total_tokens, int n_experts, int K, const float * __restrict__ logits,
												  float * __restrict__ weights, uint16_t * __restrict__ chosen,
												  float * tile, int * hist) {
	const int t0 = blockIdx.x * SELECT_TOKENS_PER_BLOCK;
	const int group = threadIdx.x / LANES;
	const int slot = threadIdx.x % LANES;
	const int t = t0 + group;
	const bool live = slot < K;
	float val = live ? -INFINITY : INFINITY;             /* lanes beyond K hold +inf and never are the minimum */
	int idx = 0xFFFF;
	float min_val = -INFINITY;
	float max_val = -INFINITY;
	int min_slot = 0;

	for (int c0 = 0; c0 < n_experts; c0 += SELECT_F32_CHUNK) {
		__syncthreads();
		for (int i = threadIdx.x; i < SELECT_TOKENS_PER_BLOCK * SELECT_F32_CHUNK; i += blockDim.x) {
			const int r = i / SELECT_F32_CHUNK, c = i % SELECT_F32_CHUNK;
			tile[r * SELECT_F32_ROW + c] = (t0 + r < total_tokens && c0 + c < n_experts) ? logits[(size_t) (t0 + r) * n_experts + c0 + c] : -INFINITY;
		}
		__syncthreads();
		const float * row = tile + group * SELECT_F32_ROW;
		const int lim = min(SELECT_F32_CHUNK, n_experts - c0);
		for (int j = 0; j < lim; j++) {
			const float v = row[j];
			const bool enters = v > min_val;                /* the same in every lane of the group */
			max_val = enters ? fmaxf(max_val, v) : max_val;
			if (enters && slot == min_slot) {
				val = v;
				idx = c0 + j;
			}
			if (LANES > 1) {
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
		const float ex = live ? expf(val - max_val) : 0.0f;      /* select_experts.cu:181, 189 */
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

/* Same launch and same contract as the bf16 kernel. */
extern "C" __global__ void __launch_bounds__(SELECT_TOKENS_PER_BLOCK * SELECT_MAX_K)
default_select_experts_fp32_kernel(int total_tokens, int n_experts, int top_k_experts, const float * X_routed,
								   float * token_expert_weights, uint16_t * chosen_experts, int * expert_counts,
								   int * expert_counts_cumsum, int * host_expert_counts) {
	__shared__ float tile[SELECT_TOKENS_PER_BLOCK * SELECT_F32_ROW];
	__shared__ int ticket;
	extern __shared__ int hist[];

	for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
		hist[e] = 0;
	}
	switch (blockDim.x / SELECT_TOKENS_PER_BLOCK) {
		case 1: select_tokens_f32<1>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 2: select_tokens_f32<2>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 4: select_tokens_f32<4>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 8: select_tokens_f32<8>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		case 16: select_tokens_f32<16>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
		default: select_tokens_f32<32>(total_tokens, n_experts, top_k_experts, X_routed, token_expert_weights, chosen_experts, tile, hist); break;
	}
	select_finish(n_experts, hist, &ticket, expert_counts, expert_counts_cumsum, host_expert_counts);
}

/* ------------------------------------------------------------------ build_expert_mapping */

#define BUILD_THREADS 256
#define BUILD_WAVES (BUILD_THREADS / WAVE)
#define BUILD_PRIVATE_INTS 2048             /* counters of one wave's private histogram (E * copies of them) */
#define BUILD_LOADS_AHEAD 8                 /* 16-byte loads of ids a lane keeps in flight while counting */

/* Counters per expert in a wave's private histogram: the largest power of two (at most 32) with E * copies <=
 * BUILD_PRIVATE_INTS; 1 = no private histograms.  The launch configuration sizes the LDS with the same rule. */
__host__ __device__ inline int build_private_copies(int E) {
	int copies = 32;
	while (copies > 1 && E * copies > BUILD_PRIVATE_INTS) {
		copies >>= 1;
	}
	return copies;
}

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
 * dynamic LDS = 6 * num_routed_experts ints, plus 4 * E * copies ints of private histograms where copies =
 * build_private_copies(E) is above 1. */
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

	const int lane = threadIdx.x & (WAVE - 1);
	const int wave = threadIdx.x / WAVE;
	const int copies = build_private_copies(E);
	for (int i = threadIdx.x; i < 6 * E + (copies > 1 ? BUILD_WAVES * E * copies : 0); i += BUILD_THREADS) {
		lds[i] = 0;
	}
	__syncthreads();

	const bool aligned = ((((uintptr_t) chosen_experts) & 15) == 0);
	if (copies > 1) {
		/* pass 1, E up to 1024: every id is counted once, into a histogram private to the wave with `copies` counters per
		 * expert (lane l adds to copy l % copies), so that lanes with the same id rarely meet at one address.  First the
		 * ids in front of the tile (their sums are pre), then the rest on top of them (the sums are tot). */
		int * priv = lds + 6 * E + wave * E * copies;
		const int copy = lane & (copies - 1);
		const long bounds[3] = {0, min(tile_lo, R), R};
		for (int phase = 0; phase < 2; phase++) {
			const long lo_ = bounds[phase], hi_ = bounds[phase + 1];          /* lo_ is 0 or a multiple of 256 */
			const long vec_hi = aligned ? max(lo_, hi_ & ~7L) : lo_;      /* 8 ids per 16-byte load up to here, one by one behind */
			const u32x4 * ids = (const u32x4 *) chosen_experts;
			/* BUILD_LOADS_AHEAD loads of a lane are in flight together: one after the other, each waiting for its ids, the
			 * latency of a load (the same 16 bytes for every work-group, so an L2 hit) times the loads per lane is the
			 * length of this pass */
			for (long v0 = (lo_ >> 3) + threadIdx.x; v0 < (vec_hi >> 3); v0 += BUILD_LOADS_AHEAD * BUILD_THREADS) {
				u32x4 q[BUILD_LOADS_AHEAD];
				#pragma unroll
				for (int u = 0; u < BUILD_LOADS_AHEAD; u++) {
					const long v = v0 + (long) u * BUILD_THREADS;
					q[u] = v < (vec_hi >> 3) ? ids[v] : u32x4{0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu};   /* ids no expert has */
				}
				#pragma unroll
				for (int u = 0; u < BUILD_LOADS_AHEAD; u++) {
					const uint32_t w[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
					#pragma unroll
					for (int j = 0; j < 8; j++) {
						const int e = (int) ((w[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu);
						if (e < E) {
							atomicAdd(&priv[e * copies + copy], 1);
						}
					}
				}
			}
			for (long i = vec_hi + threadIdx.x; i < hi_; i += BUILD_THREADS) {
				const int e = chosen_experts[i];
				if (e < E) {
					atomicAdd(&priv[e * copies + copy], 1);
				}
			}
			__syncthreads();
			int * out = phase == 0 ? pre : tot;
			for (int idx = threadIdx.x; idx < E * copies; idx += BUILD_THREADS) {  /* E * copies is a multiple of 64 or below 64 */
				int sum = 0;
				#pragma unroll
				for (int w_ = 0; w_ < BUILD_WAVES; w_++) {
					sum += lds[6 * E + w_ * E * copies + idx];
				}
				for (int off = 1; off < copies; off <<= 1) {
					sum += __shfl_xor(sum, off, WAVE);
				}
				if ((idx & (copies - 1)) == 0) {
					out[idx / copies] = sum;
				}
			}
			__syncthreads();
		}
		/* the tile's own entries per wave quarter */
		const long qlo = tile_lo + (long) wave * sub;
		const long qhi = min(qlo + sub, tile_hi);
		for (long i = qlo + lane; i < qhi; i += WAVE) {
			const int e = chosen_experts[i];
			if (e < E) {
				atomicAdd(&run[wave * E + e], 1);
			}
		}
	} else {
	/* pass 1, more experts than private histograms have room for: histogram of everything, 8 ids per 16-byte load */
	const long nvec = R / 8;
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
	}
	__syncthreads();

	/* exclusive scan of tot by wave 0; pre[e] becomes the first position of this block's entries of expert e */
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

	/* pass 2: each wave walks its quarter of the tile 64 entries at a time.  A lane finds the lanes that hold its expert
	 * with one ballot per bit of the id (lanes that agree in every bit), its rank among them is its place behind the
	 * wave's running position of that expert, and the first of them moves the position on.  An invalid lane takes part
	 * as id E, which no valid lane holds, so it never shares a mask with one. */
	int * my_run = run + wave * E;
	const long lo = tile_lo + (long) wave * sub;
	const long hi = min(lo + sub, tile_hi);
	int id_bits = 1;
	while ((1 << id_bits) <= E) {
		id_bits++;
	}
	for (long i0 = lo; i0 < hi; i0 += WAVE) {
		long i = i0 + lane;
		bool valid = i < hi;
		int e = valid ? (int) chosen_experts[i] : E;
		valid = valid && (e < E);
		e = valid ? e : E;
		uint64_t same = ~0ULL;
		for (int bit = 0; bit < id_bits; bit++) {
			const bool set = (e >> bit) & 1;
			const uint64_t with_bit = __ballot(set);
			same &= set ? with_bit : ~with_bit;
		}
		int start = 0;
		if (valid) {
			start = my_run[e];
		}
		/* every lane has read the position before the first lane of each expert replaces it (a wave executes the read of all
		 * its lanes before the write below; the compiler keeps the order of the two LDS accesses to the same array) */
		const int rank = __popcll(same & lanemask_lt());
		if (valid && rank == 0) {
			my_run[e] = start + __popcll(same);
		}
		if (valid) {
			const int slot = start + rank;
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
