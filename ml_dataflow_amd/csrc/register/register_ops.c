/*
 * register_ops.c -- dataflow_register_default_ops for the gfx950 MoE backend.
 *
 * Counterpart of backends/nvidia/src/ops/src/register_ops/register_ops.c:412-421, restricted to the ops
 * of the MoE layer: the ten native kernels the reference registers for that path (bf16 variants), the RMS norm,
 * AdamW and cast ops next to it, its external matmul, and this backend's grouped additions.  Each op is keyed by the fingerprint of the same
 * skeleton the submit wrappers build, so callers find it without knowing which backend answered.
 *
 * Native kernel symbols follow the reference's naming, "<op>_<dtypes lower case>_kernel"
 * (register_ops.c:77-78, 223-224) and launch-configuration symbols "<op>_set_launch_config".
 */
#define _GNU_SOURCE
#include "dataflow_amd.h"
#include "dataflow_amd_ops.h"

#include <dlfcn.h>
#include <limits.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#define NATIVE_CODE_FILE "hip_kernels_gfx950.hsaco"
#define NATIVE_CONFIG_LIB "libhip_kernels_config.so"
#define MATMUL_LIB "libamd_matmul.so"

/* directory that holds the code objects: $DATAFLOW_AMD_LIB_DIR, else the directory of this library */
static int find_lib_dir(char * out, size_t out_len) {
	const char * env = getenv("DATAFLOW_AMD_LIB_DIR");
	if (env && env[0]) {
		snprintf(out, out_len, "%s", env);
		return 0;
	}
	Dl_info info;
	if (!dladdr((void *) &find_lib_dir, &info) || !info.dli_fname) {
		fprintf(stderr, "Error: cannot locate the backend library on disk; set DATAFLOW_AMD_LIB_DIR...\n");
		return -1;
	}
	snprintf(out, out_len, "%s", info.dli_fname);
	char * slash = strrchr(out, '/');
	if (slash) {
		*slash = '\0';
	} else {
		snprintf(out, out_len, ".");
	}
	return 0;
}

static int register_native(Dataflow_Handle * handle, const char * dir) {
	enum { N = 28 };
	Op_Skeleton skeletons[N];
	char * symbols[N];
	char * launch_symbols[N];
	char * init_symbols[N];
	const DataflowDatatype dt = DATAFLOW_BF16;
	int n = 0;

	dataflow_set_default_select_experts_skeleton(&skeletons[n], dt);
	symbols[n] = "default_select_experts_bf16_kernel"; launch_symbols[n] = "default_select_experts_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_build_expert_mapping_skeleton(&skeletons[n]);
	symbols[n] = "default_build_expert_mapping_kernel"; launch_symbols[n] = "default_build_expert_mapping_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_prepare_experts_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_prepare_experts_bf16_bf16_kernel"; launch_symbols[n] = "default_prepare_experts_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_prepare_expert_zone_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_prepare_expert_zone_bf16_bf16_kernel"; launch_symbols[n] = "default_prepare_expert_zone_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_merge_experts_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_merge_experts_bf16_bf16_kernel"; launch_symbols[n] = "default_merge_experts_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_merge_expert_result_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_merge_expert_result_bf16_bf16_kernel"; launch_symbols[n] = "default_merge_expert_result_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_router_bwd_x_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_router_bwd_x_bf16_bf16_kernel"; launch_symbols[n] = "default_router_bwd_x_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_router_gate_bwd_x_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_router_gate_bwd_x_bf16_bf16_kernel"; launch_symbols[n] = "default_router_gate_bwd_x_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_swiglu_skeleton(&skeletons[n], dt);
	symbols[n] = "default_swiglu_bf16_kernel"; launch_symbols[n] = "default_swiglu_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_swiglu_bwd_x_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_swiglu_bwd_x_bf16_bf16_kernel"; launch_symbols[n] = "default_swiglu_bwd_x_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_rms_norm_skeleton(&skeletons[n], dt);
	symbols[n] = "default_rms_norm_bf16_kernel"; launch_symbols[n] = "default_rms_norm_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_rms_norm_recompute_skeleton(&skeletons[n], dt);
	symbols[n] = "default_rms_norm_recompute_bf16_kernel"; launch_symbols[n] = "default_rms_norm_recompute_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_rms_norm_bwd_x_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_rms_norm_bwd_x_bf16_bf16_kernel"; launch_symbols[n] = "default_rms_norm_bwd_x_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_rms_norm_bwd_w_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "default_rms_norm_bwd_w_bf16_bf16_kernel"; launch_symbols[n] = "default_rms_norm_bwd_w_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_rms_norm_bwd_w_combine_skeleton(&skeletons[n], dt);
	symbols[n] = "default_rms_norm_bwd_w_combine_bf16_kernel"; launch_symbols[n] = "default_rms_norm_bwd_w_combine_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_adamw_step_skeleton(&skeletons[n], dt, dt, dt, dt);
	symbols[n] = "default_adamw_step_bf16_bf16_bf16_bf16_kernel"; launch_symbols[n] = "default_adamw_step_set_launch_config"; init_symbols[n++] = NULL;
	/* the two casts the reference registers (register_ops.c:168-177): bf16 -> fp32, and fp32 folded into bf16 */
	dataflow_set_default_cast_skeleton(&skeletons[n], dt, DATAFLOW_FP32, DATAFLOW_NONE);
	symbols[n] = "default_cast_bf16_fp32_kernel"; launch_symbols[n] = "default_cast_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_cast_and_add_skeleton(&skeletons[n], DATAFLOW_FP32, dt, dt);
	symbols[n] = "default_cast_and_add_fp32_bf16_bf16_kernel"; launch_symbols[n] = "default_cast_and_add_set_launch_config"; init_symbols[n++] = NULL;
	/* the element types beside bf16 for which the reference has real kernels of this path's ops (register_ops.c:87-103:
	 * one kernel symbol per type, one launch configuration per op): select_experts on fp32 logits (its fp16 and fp8
	 * kernels are empty), swiglu and swiglu_bwd_x on fp32 and fp16 */
	dataflow_set_default_select_experts_skeleton(&skeletons[n], DATAFLOW_FP32);
	symbols[n] = "default_select_experts_fp32_kernel"; launch_symbols[n] = "default_select_experts_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_swiglu_skeleton(&skeletons[n], DATAFLOW_FP32);
	symbols[n] = "default_swiglu_fp32_kernel"; launch_symbols[n] = "default_swiglu_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_swiglu_skeleton(&skeletons[n], DATAFLOW_FP16);
	symbols[n] = "default_swiglu_fp16_kernel"; launch_symbols[n] = "default_swiglu_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_swiglu_bwd_x_skeleton(&skeletons[n], DATAFLOW_FP32, DATAFLOW_FP32);
	symbols[n] = "default_swiglu_bwd_x_fp32_fp32_kernel"; launch_symbols[n] = "default_swiglu_bwd_x_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_default_swiglu_bwd_x_skeleton(&skeletons[n], DATAFLOW_FP16, DATAFLOW_FP16);
	symbols[n] = "default_swiglu_bwd_x_fp16_fp16_kernel"; launch_symbols[n] = "default_swiglu_bwd_x_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_amd_router_bwd_x_all_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "amd_router_bwd_x_all_bf16_bf16_kernel"; launch_symbols[n] = "amd_router_bwd_x_all_set_launch_config"; init_symbols[n++] = NULL;

	dataflow_set_amd_prepare_experts_scaled_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "amd_prepare_experts_scaled_bf16_bf16_kernel"; launch_symbols[n] = "amd_prepare_experts_scaled_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_amd_swiglu_strided_skeleton(&skeletons[n], dt);
	symbols[n] = "amd_swiglu_strided_bf16_kernel"; launch_symbols[n] = "amd_swiglu_strided_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_amd_swiglu_bwd_x_routed_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "amd_swiglu_bwd_x_routed_bf16_bf16_kernel"; launch_symbols[n] = "amd_swiglu_bwd_x_routed_set_launch_config"; init_symbols[n++] = NULL;
	dataflow_set_amd_merge_experts_fresh_skeleton(&skeletons[n], dt, dt);
	symbols[n] = "amd_merge_experts_fresh_bf16_bf16_kernel"; launch_symbols[n] = "default_merge_experts_set_launch_config"; init_symbols[n++] = NULL;

	char code_file[PATH_MAX];
	char config_lib[PATH_MAX];
	snprintf(code_file, sizeof(code_file), "%s/%s", dir, NATIVE_CODE_FILE);
	snprintf(config_lib, sizeof(config_lib), "%s/%s", dir, NATIVE_CONFIG_LIB);

	int added = (handle->register_native_code)(handle, code_file, config_lib, n, skeletons, symbols, launch_symbols, init_symbols);
	if (added != n) {
		fprintf(stderr, "Error: failed to register native ops, expected %d functions, got %d...\n", n, added);
		return -1;
	}
	return added;
}

static int register_external(Dataflow_Handle * handle, const char * dir) {
	enum { N = 3 };
	Op_Skeleton skeletons[N];
	dataflow_set_matmul_skeleton(&skeletons[0]);
	dataflow_set_amd_grouped_matmul_skeleton(&skeletons[1]);
	dataflow_set_amd_grouped_matmul_gathered_skeleton(&skeletons[2]);      /* same entry point: it tells the two by the argument count */
	char * symbols[N] = {"amd_matmul", "amd_grouped_matmul", "amd_grouped_matmul"};
	char * init_symbols[N] = {"amd_matmul_init", "amd_matmul_init", "amd_matmul_init"};

	char lib[PATH_MAX];
	snprintf(lib, sizeof(lib), "%s/%s", dir, MATMUL_LIB);
	int added = (handle->register_external_code)(handle, lib, N, skeletons, symbols, init_symbols);
	if (added != N) {
		fprintf(stderr, "Error: failed to register matmul ops, expected %d functions, got %d...\n", N, added);
		return -1;
	}
	return added;
}

int dataflow_register_default_ops(Dataflow_Handle * dataflow_handle) {
	if (!dataflow_handle || !dataflow_handle->register_native_code || !dataflow_handle->register_external_code) {
		fprintf(stderr, "Error: cannot register ops on an uninitialised handle...\n");
		return -1;
	}
	char dir[PATH_MAX];
	if (find_lib_dir(dir, sizeof(dir))) {
		return -1;
	}
	int external = register_external(dataflow_handle, dir);
	if (external < 0) {
		return -1;
	}
	int native = register_native(dataflow_handle, dir);
	if (native < 0) {
		return -1;
	}
	return external + native;
}
