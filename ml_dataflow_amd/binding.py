"""ctypes view of the C boundary declared in include/dataflow_amd.h, dataflow_amd_ops.h and moe_layer.h.

This module is plumbing: it mirrors the C structs byte for byte and declares the argument types of the
exported entry points so Python callers (tests, bench.py) go through exactly the C ABI a C program would.
Nothing is computed here, and there is no fallback: if the shared libraries are missing or were built
without the HIP kernels, loading fails loudly.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(HERE, "lib")
LIB_NAME = "libdataflow_amd.so"
ARTIFACTS = (LIB_NAME, "hip_kernels_gfx950.hsaco", "libhip_kernels_config.so", "libamd_matmul.so")

# ---- enums (include/dataflow_amd.h) ----
(DATAFLOW_NONE, DATAFLOW_VOID, DATAFLOW_FP64, DATAFLOW_FP32, DATAFLOW_FP16, DATAFLOW_BF16, DATAFLOW_FP8E4M3,
 DATAFLOW_FP8E5M2, DATAFLOW_UINT64, DATAFLOW_UINT32, DATAFLOW_UINT16, DATAFLOW_UINT8, DATAFLOW_LONG, DATAFLOW_INT,
 DATAFLOW_BOOL, DATAFLOW_FP64_SCALAR, DATAFLOW_FP32_SCALAR, DATAFLOW_FP16_SCALAR, DATAFLOW_BF16_SCALAR,
 DATAFLOW_FP8E4M3_SCALAR, DATAFLOW_FP8E5M2_SCALAR, DATAFLOW_UINT64_SCALAR, DATAFLOW_UINT32_SCALAR,
 DATAFLOW_UINT16_SCALAR, DATAFLOW_UINT8_SCALAR, DATAFLOW_LONG_SCALAR, DATAFLOW_INT_SCALAR,
 DATAFLOW_BOOL_SCALAR) = range(28)

COMPUTE_NONE, COMPUTE_CPU, COMPUTE_CUDA, COMPUTE_HSA, COMPUTE_LEVEL_ZERO = range(5)

MAX_OP_ARGS = 32
MAX_STREAMS = 256
MAX_NATIVE_FUNCTION_LIBS = 1024
AMD_GROUPED_RAGGED_N, AMD_GROUPED_RAGGED_K = 0, 1
AMD_MOE_PER_EXPERT, AMD_MOE_GROUPED, AMD_MOE_FUSED = 0, 1, 2
AMD_MOE_FIRST_MICRO_BATCH = 0x100        # added to the backward's schedule: weight gradients written, not accumulated


class OpSkeletonHeader(C.Structure):
    _fields_ = [("op_nickname", C.c_char * 256), ("num_args", C.c_int), ("arg_dtypes", C.c_int * MAX_OP_ARGS)]


class OpSkeleton(C.Structure):
    _fields_ = [("header", OpSkeletonHeader), ("fingerprint", C.c_uint8 * 32)]


class Op(C.Structure):
    _fields_ = [("op_skeleton", OpSkeleton), ("op_args", C.c_void_p * MAX_OP_ARGS)]


class TableConfig(C.Structure):
    _fields_ = [("min_size", C.c_uint64), ("max_size", C.c_uint64), ("load_factor", C.c_float),
                ("shrink_factor", C.c_float), ("hash_func", C.c_void_p), ("key_size_bytes", C.c_uint64),
                ("value_size_bytes", C.c_uint64)]


class DataflowTable(C.Structure):
    _fields_ = [("cnt", C.c_uint64), ("size", C.c_uint64), ("config", TableConfig),
                ("is_empty_bit_vector", C.c_void_p), ("items", C.c_void_p)]


class DataflowHandle(C.Structure):
    pass


_H = C.POINTER(DataflowHandle)
_fn = C.CFUNCTYPE

DataflowHandle._fields_ = [
    # Dataflow_Profiler
    ("profiler_start", _fn(C.c_int)),
    ("profiler_stop", _fn(C.c_int)),
    ("profiler_name_device", _fn(None, _H, C.c_char_p)),
    ("profiler_name_handle", _fn(None, _H, C.c_char_p)),
    ("profiler_name_stream", _fn(None, _H, C.c_int, C.c_char_p)),
    ("profiler_name_thread", _fn(None, _H, C.c_char_p)),
    ("profiler_range_push", _fn(C.c_int, C.c_char_p)),
    ("profiler_range_pop", _fn(C.c_int)),
    ("compute_type", C.c_int),
    ("device_id", C.c_int),
    ("device_handle", C.c_void_p),
    ("device_info", C.c_void_p),
    ("hardware_arch_type", C.c_int),
    ("pcie_link_width", C.c_uint),
    ("pcie_link_gen", C.c_uint),
    ("ctx_id", C.c_int),
    ("ctx", C.c_void_p),
    ("num_streams", C.c_int),
    ("streams", C.c_void_p),
    ("stream_prios", C.c_int * MAX_STREAMS),
    ("stream_names", C.c_char_p * MAX_STREAMS),
    ("stream_states", C.c_void_p),
    ("num_native_function_libs", C.c_int),
    ("native_function_libs", C.c_void_p * MAX_NATIVE_FUNCTION_LIBS),
    ("num_ops", C.c_int),
    ("op_table", DataflowTable),
    ("get_num_procs", _fn(C.c_int, _H)),
    ("register_native_code", _fn(C.c_int, _H, C.c_char_p, C.c_char_p, C.c_int, C.POINTER(OpSkeleton),
                                 C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.POINTER(C.c_char_p))),
    ("register_external_code", _fn(C.c_int, _H, C.c_char_p, C.c_int, C.POINTER(OpSkeleton),
                                   C.POINTER(C.c_char_p), C.POINTER(C.c_char_p))),
    ("submit_op", _fn(C.c_int, _H, C.POINTER(Op), C.c_int)),
    ("submit_host_op", _fn(C.c_int, _H, C.c_void_p, C.c_void_p, C.c_int)),
    ("get_stream_state", _fn(C.c_void_p, _H, C.c_int)),
    ("submit_dependency", _fn(C.c_int, _H, C.c_int, C.c_void_p)),
    ("sync_stream", _fn(C.c_int, _H, C.c_int)),
    ("sync_handle", _fn(C.c_int, _H)),
    ("alloc_mem", _fn(C.c_void_p, _H, C.c_uint64)),
    ("free_mem", _fn(None, _H, C.c_void_p)),
    ("set_mem", _fn(C.c_int, _H, C.c_int, C.c_void_p, C.c_uint8, C.c_uint64)),
    ("enable_access_to_host_mem", _fn(C.c_int, _H, C.c_void_p, C.c_uint64, C.c_uint)),
    ("disable_access_to_host_mem", _fn(C.c_int, _H, C.c_void_p)),
    ("enable_access_to_peer_mem", _fn(C.c_int, _H, _H)),
    ("disable_access_to_peer_mem", _fn(C.c_int, _H, _H)),
    ("submit_inbound_transfer", _fn(C.c_int, _H, C.c_int, C.c_void_p, C.c_void_p, C.c_uint64)),
    ("submit_outbound_transfer", _fn(C.c_int, _H, C.c_int, C.c_void_p, C.c_void_p, C.c_uint64)),
    ("submit_peer_transfer", _fn(C.c_int, _H, C.c_int, C.c_void_p, C.c_void_p, C.c_uint64)),
]


class HipDeviceInfo(C.Structure):
    _fields_ = [("total_mem", C.c_size_t), ("arch_num", C.c_int), ("cu_count", C.c_int), ("xcd_count", C.c_int),
                ("wavefront_size", C.c_int), ("max_threads_per_block", C.c_int), ("max_lds_per_block", C.c_int),
                ("optin_max_lds_per_block", C.c_int), ("clock_khz", C.c_int), ("host_numa_id", C.c_int),
                ("device_name", C.c_char * 256), ("arch_name", C.c_char * 64)]


class AmdMoeBlockOffsets(C.Structure):
    """include/moe_layer.h: Amd_Moe_Block_Offsets"""
    _fields_ = [(name, C.c_uint64) for name in ("w_attn_norm", "w_q", "w_k", "w_v", "w_o", "w_ffn_norm", "w_router", "w_1", "w_3", "w_2",
                                                "expert_stride", "raw_size", "aligned_size")]


class AmdMoeLayer(C.Structure):
    _fields_ = [
        ("max_tokens", C.c_int), ("model_dim", C.c_int), ("num_experts", C.c_int), ("top_k", C.c_int),
        ("expert_dim", C.c_int), ("dt", C.c_int),
        ("slab", C.c_void_p), ("slab_bytes", C.c_uint64),
        ("w_router", C.c_void_p), ("w1", C.c_void_p), ("w3", C.c_void_p), ("w2", C.c_void_p),
        ("expert_stride_bytes", C.c_uint64),
        ("dw_router", C.c_void_p), ("dw1", C.c_void_p), ("dw3", C.c_void_p), ("dw2", C.c_void_p),
        ("x_routed", C.c_void_p), ("token_expert_weights", C.c_void_p), ("chosen_experts", C.c_void_p),
        ("expert_counts", C.c_void_p), ("expert_counts_cumsum", C.c_void_p), ("expert_mapping", C.c_void_p),
        ("token_mapping", C.c_void_p), ("x1", C.c_void_p), ("x3", C.c_void_p), ("host_expert_counts", C.c_void_p),
        ("d_routed", C.c_void_p), ("dx1", C.c_void_p), ("dx3", C.c_void_p),
        ("expert_zones", C.c_void_p), ("kernel_workspace", C.c_void_p), ("kernel_workspace_bytes", C.c_uint64),
        ("last_forward_tokens", C.c_int), ("saved_side_by_side", C.c_int), ("host_counts_synced", C.c_int),
    ]


_P = C.c_void_p
_I = C.c_int
_DT = C.c_int

# name -> (restype, argtypes); every symbol declared in include/*.h appears here
SIGNATURES = {
    # dataflow_amd.h
    "dataflow_init_handle": (_I, [_H, _I, _I, _I, C.c_uint, _I, C.POINTER(_I), C.POINTER(C.c_char_p), C.c_float]),
    "dataflow_register_default_ops": (_I, [_H]),
    "dataflow_sizeof_element": (C.c_size_t, [_DT]),
    "dataflow_datatype_as_string": (C.c_char_p, [_DT]),
    "dataflow_do_fingerprinting": (_I, [_P, C.c_uint64, C.POINTER(C.c_uint8)]),
    "dataflow_init_table": (_I, [C.POINTER(DataflowTable), _P, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float, C.c_float]),
    "dataflow_destroy_table": (None, [C.POINTER(DataflowTable)]),
    "dataflow_insert_table": (_I, [C.POINTER(DataflowTable), _P, _P]),
    "dataflow_find_table": (C.c_long, [C.POINTER(DataflowTable), _P, C.c_bool, C.POINTER(_P)]),
    "dataflow_remove_table": (_I, [C.POINTER(DataflowTable), _P, _P]),
    "solo_bf16_to_fp32": (C.c_float, [C.c_uint16]),
    "solo_fp32_to_bf16": (C.c_uint16, [C.c_float]),
    "dataflow_amd_alloc_host_mem": (_P, [_H, C.c_uint64]),
    "dataflow_amd_free_host_mem": (None, [_H, _P]),
    "dataflow_amd_destroy_handle": (None, [_H]),
    "dataflow_amd_get_stream": (_P, [_H, _I]),
    # dataflow_amd_ops.h: skeleton setters
    "dataflow_set_matmul_skeleton": (None, [C.POINTER(OpSkeleton)]),
    "dataflow_set_default_rms_norm_skeleton": (None, [C.POINTER(OpSkeleton), _DT]),
    "dataflow_set_default_rms_norm_recompute_skeleton": (None, [C.POINTER(OpSkeleton), _DT]),
    "dataflow_set_default_rms_norm_bwd_x_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_rms_norm_bwd_w_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_rms_norm_bwd_w_combine_skeleton": (None, [C.POINTER(OpSkeleton), _DT]),
    "dataflow_set_default_adamw_step_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT, _DT, _DT]),
    "dataflow_set_amd_prepare_experts_scaled_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_amd_swiglu_strided_skeleton": (None, [C.POINTER(OpSkeleton), _DT]),
    "dataflow_set_amd_merge_experts_fresh_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_amd_swiglu_bwd_x_routed_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_cast_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT, _DT]),
    "dataflow_set_default_cast_and_add_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT, _DT]),
    "dataflow_set_default_swiglu_skeleton": (None, [C.POINTER(OpSkeleton), _DT]),
    "dataflow_set_default_swiglu_bwd_x_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_select_experts_skeleton": (None, [C.POINTER(OpSkeleton), _DT]),
    "dataflow_set_default_build_expert_mapping_skeleton": (None, [C.POINTER(OpSkeleton)]),
    "dataflow_set_default_prepare_expert_zone_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_prepare_experts_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_merge_expert_result_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_merge_experts_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_router_bwd_x_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_default_router_gate_bwd_x_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    "dataflow_set_amd_grouped_matmul_skeleton": (None, [C.POINTER(OpSkeleton)]),
    "dataflow_set_amd_grouped_matmul_gathered_skeleton": (None, [C.POINTER(OpSkeleton)]),
    "dataflow_set_amd_router_bwd_x_all_skeleton": (None, [C.POINTER(OpSkeleton), _DT, _DT]),
    # dataflow_amd_ops.h: submit wrappers
    "dataflow_submit_matmul": (_I, [_H, _I, _DT, _DT, _DT, _DT, _DT, _I, _I, _I, _I, _I, C.c_float, C.c_float, _P, _P, _P, _P, C.c_uint64, _P]),
    "dataflow_submit_default_rms_norm": (_I, [_H, _I, _DT, _I, _I, C.c_float, _P, _P, _P, _P]),
    "dataflow_submit_default_rms_norm_recompute": (_I, [_H, _I, _DT, _I, _I, _P, _P, _P, _P]),
    "dataflow_submit_default_rms_norm_bwd_x": (_I, [_H, _I, _DT, _DT, _I, _I, C.c_float, _P, _P, _P, _P, _P, _P]),
    "dataflow_submit_default_rms_norm_bwd_w": (_I, [_H, _I, _DT, _DT, _I, _I, C.c_float, _P, _P, _P, _P, C.c_uint64, _P]),
    "dataflow_submit_default_adamw_step": (_I, [_H, _I, _DT, _DT, _DT, _DT, C.c_uint64, _I, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float,
                                            _P, _P, _P, _P]),
    "dataflow_submit_amd_prepare_experts_scaled": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _P, _P, _P, _P]),
    "dataflow_submit_amd_swiglu_bwd_x_routed": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "dataflow_submit_amd_swiglu_strided": (_I, [_H, _I, _DT, _I, _I, _I, _P, _P, _P]),
    "dataflow_submit_amd_merge_experts_fresh": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _P, _P, _P, _P]),
    "dataflow_submit_cast": (_I, [_H, _I, _DT, _DT, C.c_uint64, _P, _P]),
    "dataflow_submit_cast_and_add": (_I, [_H, _I, _DT, _DT, _DT, C.c_uint64, C.c_float, _P, C.c_float, _P, _P]),
    "dataflow_submit_default_swiglu": (_I, [_H, _I, _DT, _I, _I, _P, _P, _P]),
    "dataflow_submit_default_swiglu_bwd_x": (_I, [_H, _I, _DT, _DT, _I, _I, _P, _P, _P, _P, _P]),
    "dataflow_submit_default_select_experts": (_I, [_H, _I, _DT, _I, _I, _I, _P, _P, _P, _P, _P, _P]),
    "dataflow_submit_default_build_expert_mapping": (_I, [_H, _I, _I, _I, _I, _P, _P, _P, _P]),
    "dataflow_submit_default_prepare_experts": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _P, _P, _P]),
    "dataflow_submit_default_prepare_expert_zone": (_I, [_H, _I, _DT, _DT, _I, _P, _I, _P, _P, _P, _P]),
    "dataflow_submit_default_merge_experts": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _P, _P, _P, _P]),
    "dataflow_submit_default_merge_expert_result": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _P, _I, _P, _P, _P, _P, _P]),
    "dataflow_submit_router_bwd_x": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P, _P]),
    "dataflow_submit_router_gate_bwd_x": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _P, _P, _P]),
    "dataflow_submit_amd_grouped_matmul": (_I, [_H, _I, _DT, _DT, _DT, _DT, _DT, _I, _I, _I, _I, _I, _I, _I, _P, C.c_float, C.c_float,
                                                _P, C.c_uint64, _P, _P, _P, C.c_uint64]),
    "dataflow_submit_amd_grouped_matmul_gathered": (_I, [_H, _I, _DT, _DT, _DT, _DT, _DT, _I, _I, _I, _I, _I, _I, _I, _P, C.c_float, C.c_float,
                                                         _P, C.c_uint64, _P, _P, _P, C.c_uint64, _P, _I]),
    "dataflow_submit_amd_router_bwd_x_all": (_I, [_H, _I, _DT, _DT, _I, _I, _I, _I, _P, _P, _P, _P, _P, _P, _P]),
    # moe_layer.h
    "amd_moe_layer_bytes": (C.c_uint64, [_I, _I, _I, _I, _I]),
    "amd_moe_layer_alloc": (_I, [_H, C.POINTER(AmdMoeLayer), _I, _I, _I, _I, _I]),
    "amd_moe_layer_free": (None, [_H, C.POINTER(AmdMoeLayer)]),
    "amd_moe_layer_forward": (_I, [_H, _I, _I, C.POINTER(AmdMoeLayer), _I, _P, _P, _P, _I]),
    "amd_moe_layer_backward": (_I, [_H, _I, _I, C.POINTER(AmdMoeLayer), _I, _P, _P, _P, _I]),
    "amd_moe_block_weight_offsets": (_I, [_I, _I, _I, _I, _I, _DT, _I, C.POINTER(AmdMoeBlockOffsets)]),
    "amd_moe_layer_load_block_file": (_I, [_H, _I, C.POINTER(AmdMoeLayer), C.c_char_p, _I, _I, _I, _P]),
    "amd_moe_saved_array_path": (_I, [C.c_char_p, C.c_size_t, C.c_char_p, _I, _I, _I, _I, C.c_char_p]),
    "amd_moe_save_array": (_I, [_H, _I, C.c_char_p, _I, _I, _I, _I, C.c_char_p, _P, _I, _I, _DT]),
}

_lib = None


def missing_artifacts():
    return [name for name in ARTIFACTS if not os.path.exists(os.path.join(LIB_DIR, name))]


def load_library():
    """Load libdataflow_amd.so (built in-tree by ml_dataflow_amd/csrc/Makefile) and type every entry point."""
    global _lib
    if _lib is not None:
        return _lib
    missing = missing_artifacts()
    if missing:
        raise RuntimeError(
            "ml_dataflow_amd: native artifacts missing from %s: %s. Build them with "
            "`make -C ml_dataflow_amd/csrc` (or __graft_entry__.build()); there is no fallback path." % (LIB_DIR, ", ".join(missing)))
    lib = C.CDLL(os.path.join(LIB_DIR, LIB_NAME), mode=C.RTLD_GLOBAL)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError here means the library does not export a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib
