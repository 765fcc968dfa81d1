/*
 * amd_matmul.h -- entry points of libamd_matmul.so, the external-op library of the gfx950 backend (the counterpart of
 * the reference's libmatmulwrapper, backends/nvidia/src/ops/src/external/matmul_helper/include/matmul_helper.h:24-33).
 *
 * The handle loads the library in register_external_code and calls these through the op table; the signatures of the
 * first three are the external-op contract of libdataflow (dataflow_handle.h:161-166).  All return 0 on success and -1
 * on error with a message on stderr.  BF16 operands and result, fp32 accumulation; the single matmul (amd_matmul) also
 * takes the other combinations the reference's matmul accepts with the fp32 compute type (matmul_helper.c:168-296):
 * fp32 operands with an fp32 result, fp16 operands with an fp16 or fp32 result, bf16 operands with an fp32 result, C in
 * D's type, on a general kernel of their own (no split along K, workspace unused).
 */
#ifndef AMD_MATMUL_H
#define AMD_MATMUL_H

#include "dataflow_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

/* replaces cublas_matmul_init (matmul_helper.c:640): per-op state (compute-unit count of the handle's device) */
int amd_matmul_init(Dataflow_Handle * dataflow_handle, void * op_table_value);

/* replaces cublas_matmul (matmul_helper.c:774-946): the "default_matmul" op; arguments decoded from op->op_args as
 * libdataflowops/src/submit_ops/matmul_op.c:33-53 lays them out */
int amd_matmul(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra);

/* the "amd_grouped_matmul" op (an addition: one launch for all experts of a ragged group, see dataflow_amd_ops.h) */
int amd_grouped_matmul(Dataflow_Handle * dataflow_handle, int stream_id, Op * op, void * op_extra);

/* No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid it): D = alpha * op(A) op(B) + beta * C exactly as the matmul op computes
 * it (same kernels, same split along K, bit-identical results; to_trans_a / to_trans_b, M, K, N and the array layouts
 * as for dataflow_submit_matmul), with the fp32 partial sums of the split kept in a device array of the library itself
 * instead of a caller's workspace.  The call makes no allocation of any kind.  C is ignored when NULL or beta == 0.
 * Limit: a problem whose split needs more than 8 MiB of partial sums (splits * M * N * 4 bytes) is refused with -1.
 * Every call on a device shares that device's array: calls that overlap on one device (two streams, two host
 * threads) race on it.  Needs a handle on which dataflow_register_default_ops has run (that is where the array's
 * address on the handle's device is looked up). */
int amd_matmul_no_alloc(Dataflow_Handle * dataflow_handle, int stream_id, int to_trans_a, int to_trans_b,
						int M, int K, int N, float alpha, float beta, void * A, void * B, void * C, void * D);

/* No counterpart in the reference (cuBLASLt picks its kernels by heuristic, matmul_helper.c:527-600): which persistent
 * kernel large problems without a C operand run on.
 *   EIGHT_WAVES: two waves per SIMD, operands straight from global memory into one of two LDS stages, 256 x 256 tiles
 *     (256 x 288 over the token rows of a ragged-N launch).
 *   FOUR_WAVES_384: one wave per SIMD with the accumulators in the accumulation registers, 256 x 384 tiles (12 % fewer
 *     operand bytes per flop), every wave loading straight into the LDS and multiplying, its own token rows reloaded
 *     without the barrier.
 *   FOUR_WAVES: one loading wave (operands through its registers) and three multiplying waves, 256 x 288 tiles.
 *   AUTO (the default): ragged-N launches that both EIGHT_WAVES and FOUR_WAVES_384 can take are launched on both, and the
 *     work-groups decide from the group sizes on the device which of the two does the work (the other returns at once):
 *     the larger tile where the groups fill it and the rounds of tiles over the compute units come out no worse.
 *     For a single problem the same rule is evaluated on the host.  Everything else runs EIGHT_WAVES.
 * The four-wave kernels are taken only where their limits hold (no C operand, N-side operand k-contiguous, K a multiple
 * of 128 and at most 2^21, M a multiple of 8, 16-byte aligned D), the eight-wave kernel elsewhere.  Results are
 * bit-identical whichever kernel runs.  The choice is process-wide; the environment variable AMD_MATMUL_KERNEL ("auto",
 * "8", "384" or "4") sets it when the matmul op is registered. */
#define AMD_MATMUL_KERNEL_AUTO 0
#define AMD_MATMUL_KERNEL_EIGHT_WAVES 8
#define AMD_MATMUL_KERNEL_FOUR_WAVES 4
#define AMD_MATMUL_KERNEL_FOUR_WAVES_384 384
#define AMD_MATMUL_KERNEL_DEFAULT AMD_MATMUL_KERNEL_AUTO
int amd_matmul_select_kernel(int which);

#ifdef __cplusplus
}
#endif

#endif
