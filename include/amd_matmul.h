/*
 * amd_matmul.h -- entry points of libamd_matmul.so, the external-op library of the gfx950 backend (the counterpart of
 * the reference's libmatmulwrapper, backends/nvidia/src/ops/src/external/matmul_helper/include/matmul_helper.h:24-33).
 *
 * The handle loads the library in register_external_code and calls these through the op table; the signatures of the
 * first three are the external-op contract of libdataflow (dataflow_handle.h:161-166).  All return 0 on success and -1
 * on error with a message on stderr.  BF16 operands and result, fp32 accumulation.
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

/* No counterpart in the reference (cuBLASLt picks its kernels by heuristic, matmul_helper.c:527-600): which of the two
 * persistent kernels large problems without a C operand run on.  EIGHT_WAVES: two waves per SIMD, operands straight
 * from global memory into one of two LDS stages (a load has one k-tile of multiplies to arrive).  FOUR_WAVES: one wave
 * per SIMD with the accumulators in the accumulation registers, operands through registers into the LDS (two k-tiles to
 * arrive); taken only where its limits hold (no C operand, N-side operand k-contiguous, K a multiple of 128 and at most
 * 2^21, M a multiple of 8, 16-byte aligned D), the eight-wave kernel elsewhere.  Results are bit-identical.  The choice
 * is process-wide; the environment variable AMD_MATMUL_KERNEL ("8" or "4") sets it when the matmul op is registered. */
#define AMD_MATMUL_KERNEL_EIGHT_WAVES 8
#define AMD_MATMUL_KERNEL_FOUR_WAVES 4
#define AMD_MATMUL_KERNEL_DEFAULT AMD_MATMUL_KERNEL_EIGHT_WAVES
int amd_matmul_select_kernel(int which);

/* Diagnostic, no counterpart in the reference: one launch of a kernel that issues nothing but bf16 MFMAs out of
 * registers (one 512-thread work-group per compute unit, `iters` rounds per wave of eight independent 32x32x16
 * instructions, or of sixteen 16x16x32 ones: 262144 flops per round either way); *flops receives the floating-point
 * operations of the launch.  What it sustains is the ceiling of any GEMM on the card under its power limit, which
 * depends on the operands and on the instruction, hence `mode`, any sum of:
 *   AMD_MFMA_PROBE_RANDOM    pseudo-random operands of full mantissa width (what a GEMM of real activations
 *                            multiplies); without it small integers scaled by a power of two (few bits toggle);
 *   AMD_MFMA_PROBE_SHAPE_16  v_mfma_f32_16x16x32_bf16 instead of v_mfma_f32_32x32x16_bf16;
 *   AMD_MFMA_PROBE_VARYING   consecutive instructions take different operand registers, as in a GEMM's k-step.
 * device_word: 4 bytes of device memory (never written in practice). */
#define AMD_MFMA_PROBE_RANDOM 1
#define AMD_MFMA_PROBE_SHAPE_16 2
#define AMD_MFMA_PROBE_VARYING 4
int amd_matmul_mfma_probe(Dataflow_Handle * dataflow_handle, int stream_id, int iters, int mode, void * device_word,
						  uint64_t * flops);

/* Diagnostic, no counterpart in the reference: one launch of the streaming GEMM's skeleton - per step and compute
 * unit 64 KiB of operand loads straight into one of two LDS stages (512 rows x 128 bytes at a row stride of 8 KiB,
 * issued by four of the eight waves), 64 v_mfma_f32_16x16x32_bf16 per wave on constant registers, a wait for loads
 * and a barrier - to tell what a k-tile step costs for a given temperature and sharing of the data, apart from
 * everything else a GEMM does.  src: src_bytes of device memory (a multiple of 4 MiB is used), read only; a region is
 * 4 MiB = 64 steps, `share` work-groups of a die (1, 2, 4, 8, 16, 32; 0: all work-groups of the card) read the same
 * region in step, and each of the `passes` passes takes regions not read before (modulo the source), so with a source
 * beyond the caches' size every line comes from HBM once per group of sharers.  The launch does 64 * passes steps.
 * slack: 1 = a step's loads are waited for at the end of that step (what two stages allow a GEMM), 2 = at the end of
 * the next step (three stages), 0 = never, and no barrier.  flags, any sum of:
 *   AMD_STREAM_PROBE_NO_LOADS   no loads;
 *   AMD_STREAM_PROBE_NO_MFMAS   no multiplies;
 *   AMD_STREAM_PROBE_TOUCH      (slack 1, with loads) one wave reads four bytes of every line of the work-group's
 *                               1 / share of the lines two steps ahead, so that the loads proper hit the L2;
 *   AMD_STREAM_PROBE_VIA_REGISTERS  (slack 2, with loads) a third stage that exists: all eight waves load their share of a
 *                               step into one of two register sets (eight 16-byte loads per lane) and write the set
 *                               requested a step earlier to an LDS stage with ds_write_b128 in front of the barrier.
 * device_word: 4 bytes of device memory (never written in practice). */
#define AMD_STREAM_PROBE_NO_LOADS 1
#define AMD_STREAM_PROBE_NO_MFMAS 2
#define AMD_STREAM_PROBE_TOUCH 4
#define AMD_STREAM_PROBE_VIA_REGISTERS 8
int amd_matmul_stream_probe(Dataflow_Handle * dataflow_handle, int stream_id, const void * src, uint64_t src_bytes,
							int share, int slack, int flags, int passes, void * device_word);

#ifdef __cplusplus
}
#endif

#endif
