/*
 * amd_matmul_diag.h -- entry points of libamd_matmul_diag.so: diagnostic kernels that measure what the card gives a bf16
 * GEMM (the rate of the matrix instructions alone, the cost of a k-tile step's loads).  No counterpart in the reference and
 * no part of the drop-in: nothing in libdataflow_amd.so or libamd_matmul.so loads this library; bench.py's diagnostic
 * workloads and a GPU test do.  Both functions take a handle made by dataflow_init_handle for its device and streams,
 * return 0 on success and -1 on error with a message on stderr.
 */
#ifndef AMD_MATMUL_DIAG_H
#define AMD_MATMUL_DIAG_H

#include "dataflow_amd.h"

#ifdef __cplusplus
extern "C" {
#endif

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
/* bits 4-9 of flags: sharer i of a region takes its steps in the order i * n, i * n + 1, ... (wrapping), n = 0..63 */
#define AMD_STREAM_PROBE_ROTATE_SHIFT 4
/* device_word then has room for 1 + (number of work-groups) floats: entry 1 + i receives the ticks of the 100 MHz wall
 * clock that work-group i ran (not with AMD_STREAM_PROBE_VIA_REGISTERS) */
#define AMD_STREAM_PROBE_PER_GROUP_CLOCKS 1024
/* every wave issues eight loads per lane and step instead of waves 0-3 sixteen each */
#define AMD_STREAM_PROBE_ALL_WAVES_LOAD 2048
int amd_matmul_stream_probe(Dataflow_Handle * dataflow_handle, int stream_id, const void * src, uint64_t src_bytes,
							int share, int slack, int flags, int passes, void * device_word);

#ifdef __cplusplus
}
#endif

#endif
