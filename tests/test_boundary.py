"""The C boundary without a GPU: exported symbols, op identities, table, error paths.

Op identity is checked against a library compiled from the reference's OWN sources (oracle/_ref, built by
oracle/Makefile from libdataflowops/src/set_ops/set_op_skeletons.c + libdataflow's fingerprint/dtype files);
that check is skipped where the reference tree was not available to build it.
"""
import ctypes as C
import hashlib
import os
import re

import numpy as np
import pytest

from ml_dataflow_amd import binding as B

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF_LIB = os.path.join(ROOT, "oracle", "_ref", "libref_skeletons.so")


@pytest.fixture(scope="module")
def lib():
    return B.load_library()


def declared_functions(headers=("dataflow_amd.h", "dataflow_amd_ops.h", "moe_layer.h")):
    names = set()
    for header in headers:
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        # prototypes start at the beginning of a line; function-pointer members of structs are indented or parenthesised
        for m in re.finditer(r"^(?:int|void|void \*|size_t|char \*|long|float|uint16_t|uint64_t)\s+\*?\s*([a-z_0-9]+)\s*\(", text, flags=re.M):
            names.add(m.group(1))
    return names


def test_library_exports_every_declared_symbol(lib):
    declared = declared_functions()
    assert len(declared) >= 45
    for name in declared:
        assert hasattr(lib, name), "declared in include/ but not exported: " + name
    assert declared <= set(B.SIGNATURES), sorted(declared - set(B.SIGNATURES))


def test_matmul_library_exports_every_declared_symbol():
    declared = declared_functions(("amd_matmul.h",))
    assert declared == {"amd_matmul_init", "amd_matmul", "amd_grouped_matmul", "amd_matmul_no_alloc", "amd_matmul_select_kernel"}
    mm = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul.so"))
    for name in declared:
        assert hasattr(mm, name), "declared in include/amd_matmul.h but not exported: " + name
    # the drop-in for the reference's matmul wrapper exports product entry points only: the probes live in a library of their own
    assert not hasattr(mm, "amd_matmul_mfma_probe") and not hasattr(mm, "amd_matmul_stream_probe")
    diag_declared = declared_functions(("amd_matmul_diag.h",))
    assert diag_declared == {"amd_matmul_mfma_probe", "amd_matmul_stream_probe"}
    diag = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul_diag.so"))
    for name in diag_declared:
        assert hasattr(diag, name), "declared in include/amd_matmul_diag.h but not exported: " + name


def test_plugin_libraries_export_their_entry_points():
    cfg = C.CDLL(os.path.join(B.LIB_DIR, "libhip_kernels_config.so"))
    for op in ("default_select_experts", "default_build_expert_mapping", "default_prepare_experts", "default_prepare_expert_zone",
               "default_merge_experts", "default_merge_expert_result", "default_router_bwd_x", "default_router_gate_bwd_x",
               "default_swiglu", "default_swiglu_bwd_x", "amd_router_bwd_x_all", "default_rms_norm", "default_rms_norm_recompute",
               "default_rms_norm_bwd_x", "default_rms_norm_bwd_w", "default_rms_norm_bwd_w_combine", "default_adamw_step",
               "default_cast", "default_cast_and_add"):
        assert hasattr(cfg, op + "_set_launch_config")
    mm = C.CDLL(os.path.join(B.LIB_DIR, "libamd_matmul.so"))
    for sym in ("amd_matmul", "amd_matmul_init", "amd_grouped_matmul"):
        assert hasattr(mm, sym)
    blob = open(os.path.join(B.LIB_DIR, "hip_kernels_gfx950.hsaco"), "rb").read()
    for kernel in (b"default_select_experts_bf16_kernel", b"default_build_expert_mapping_kernel",
                   b"default_prepare_experts_bf16_bf16_kernel", b"default_merge_experts_bf16_bf16_kernel",
                   b"default_swiglu_bf16_kernel", b"default_swiglu_bwd_x_bf16_bf16_kernel",
                   b"default_router_bwd_x_bf16_bf16_kernel", b"default_router_gate_bwd_x_bf16_bf16_kernel",
                   b"default_rms_norm_bf16_kernel", b"default_rms_norm_recompute_bf16_kernel", b"default_rms_norm_bwd_x_bf16_bf16_kernel",
                   b"default_rms_norm_bwd_w_bf16_bf16_kernel", b"default_rms_norm_bwd_w_combine_bf16_kernel",
                   b"default_adamw_step_bf16_bf16_bf16_bf16_kernel", b"default_cast_bf16_fp32_kernel",
                   b"default_cast_and_add_fp32_bf16_bf16_kernel"):
        assert kernel in blob


def test_struct_sizes_match_the_c_layout(lib):
    assert C.sizeof(B.OpSkeletonHeader) == 388
    assert C.sizeof(B.OpSkeleton) == 420
    assert C.sizeof(B.Op) == 424 + 32 * 8


def test_sha256_matches_hashlib(lib):
    rng = np.random.default_rng(0)
    for n in (0, 1, 55, 56, 63, 64, 65, 119, 120, 388, 1000):
        data = rng.integers(0, 256, size=n, dtype=np.uint8).tobytes()
        buf = C.create_string_buffer(data, max(n, 1))
        out = (C.c_uint8 * 32)()
        assert lib.dataflow_do_fingerprinting(C.cast(buf, C.c_void_p), n, out) == 0
        assert bytes(out) == hashlib.sha256(data).digest()


SETTERS = [
    ("dataflow_set_matmul_skeleton", ()),
    ("dataflow_set_default_swiglu_skeleton", (B.DATAFLOW_BF16,)),
    ("dataflow_set_default_swiglu_bwd_x_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_select_experts_skeleton", (B.DATAFLOW_BF16,)),
    ("dataflow_set_default_build_expert_mapping_skeleton", ()),
    ("dataflow_set_default_prepare_expert_zone_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_prepare_experts_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_merge_expert_result_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_merge_experts_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_router_bwd_x_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_router_gate_bwd_x_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_rms_norm_skeleton", (B.DATAFLOW_BF16,)),
    ("dataflow_set_default_rms_norm_recompute_skeleton", (B.DATAFLOW_BF16,)),
    ("dataflow_set_default_rms_norm_bwd_x_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_rms_norm_bwd_w_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_rms_norm_bwd_w_combine_skeleton", (B.DATAFLOW_BF16,)),
    ("dataflow_set_default_adamw_step_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_BF16, B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_adamw_step_skeleton", (B.DATAFLOW_FP32, B.DATAFLOW_BF16, B.DATAFLOW_FP32, B.DATAFLOW_FP32)),
    ("dataflow_set_default_cast_skeleton", (B.DATAFLOW_BF16, B.DATAFLOW_FP32, B.DATAFLOW_NONE)),
    ("dataflow_set_default_cast_and_add_skeleton", (B.DATAFLOW_FP32, B.DATAFLOW_BF16, B.DATAFLOW_BF16)),
    ("dataflow_set_default_select_experts_skeleton", (B.DATAFLOW_FP32,)),
    ("dataflow_set_default_swiglu_skeleton", (B.DATAFLOW_FP32,)),
    ("dataflow_set_default_swiglu_skeleton", (B.DATAFLOW_FP16,)),
    ("dataflow_set_default_swiglu_bwd_x_skeleton", (B.DATAFLOW_FP32, B.DATAFLOW_FP32)),
    ("dataflow_set_default_swiglu_bwd_x_skeleton", (B.DATAFLOW_FP16, B.DATAFLOW_FP16)),
    ("dataflow_set_default_swiglu_bwd_x_skeleton", (B.DATAFLOW_FP8E4M3, B.DATAFLOW_BF16)),
]


def test_fingerprint_is_sha256_of_the_388_header_bytes(lib):
    for name, args in SETTERS:
        sk = B.OpSkeleton()
        getattr(lib, name)(C.byref(sk), *args)
        header = bytes(sk.header)
        assert len(header) == 388
        assert bytes(sk.fingerprint) == hashlib.sha256(header).digest()
        nick = sk.header.op_nickname
        assert header[len(nick):256] == b"\0" * (256 - len(nick))
        # the reference's bwd_w skeleton carries one tag (the workspace size) behind its argument count
        first_unused = sk.header.num_args + (1 if name == "dataflow_set_default_rms_norm_bwd_w_skeleton" else 0)
        assert all(sk.header.arg_dtypes[i] == B.DATAFLOW_NONE for i in range(first_unused, 32))


@pytest.mark.skipif(not os.path.exists(REF_LIB), reason="oracle/_ref not built (reference tree absent)")
def test_op_identities_equal_the_reference_build(lib):
    ref = C.CDLL(REF_LIB)
    for name, args in SETTERS:
        mine, theirs = B.OpSkeleton(), B.OpSkeleton()
        getattr(lib, name)(C.byref(mine), *args)
        fn = getattr(ref, name)
        fn.restype = None
        fn.argtypes = [C.POINTER(B.OpSkeleton)] + [C.c_int] * len(args)
        C.memset(C.byref(theirs), 0xAA, C.sizeof(theirs))
        fn(C.byref(theirs), *args)
        assert mine.header.op_nickname == theirs.header.op_nickname, name
        assert bytes(mine.header) == bytes(theirs.header), name
        assert bytes(mine.fingerprint) == bytes(theirs.fingerprint), name


@pytest.mark.skipif(not os.path.exists(REF_LIB), reason="oracle/_ref not built (reference tree absent)")
def test_dtype_helpers_equal_the_reference_build(lib):
    ref = C.CDLL(REF_LIB)
    ref.dataflow_sizeof_element.restype = C.c_size_t
    ref.dataflow_datatype_as_string.restype = C.c_char_p
    for dt in range(28):
        assert lib.dataflow_sizeof_element(dt) == ref.dataflow_sizeof_element(dt)
        assert lib.dataflow_datatype_as_string(dt) == ref.dataflow_datatype_as_string(dt)


HASH = C.CFUNCTYPE(C.c_uint64, C.c_void_p, C.c_uint64)


def test_table_insert_find_remove_grow(lib):
    @HASH
    def hash_fn(key, size):
        return C.cast(key, C.POINTER(C.c_uint64))[0] % size      # forces collisions: keys k and k+size share a home

    t = B.DataflowTable()
    assert lib.dataflow_init_table(C.byref(t), C.cast(hash_fn, C.c_void_p), 8, 16, 8, 64, 0.5, 0.1) == 0
    vals = {}
    for k in [1, 9, 17, 2, 25, 8, 16, 3, 33, 41, 5]:
        key = C.c_uint64(k)
        val = (C.c_uint64 * 2)(k * 10, k * 100)
        assert lib.dataflow_insert_table(C.byref(t), C.byref(key), val) == 0
        vals[k] = (k * 10, k * 100)
    assert t.cnt == len(vals) and t.size > 8          # grew past the load factor
    assert lib.dataflow_insert_table(C.byref(t), C.byref(C.c_uint64(9)), (C.c_uint64 * 2)(0, 0)) == -1   # duplicate
    for k, v in vals.items():
        out = C.c_void_p()
        assert lib.dataflow_find_table(C.byref(t), C.byref(C.c_uint64(k)), False, C.byref(out)) >= 0
        got = C.cast(out, C.POINTER(C.c_uint64))
        assert (got[0], got[1]) == v
    out = C.c_void_p()
    assert lib.dataflow_find_table(C.byref(t), C.byref(C.c_uint64(77)), False, C.byref(out)) == -1 and not out.value
    removed = (C.c_uint64 * 2)()
    assert lib.dataflow_remove_table(C.byref(t), C.byref(C.c_uint64(9)), removed) == 0 and removed[0] == 90
    assert lib.dataflow_remove_table(C.byref(t), C.byref(C.c_uint64(9)), removed) == -1
    for k in vals:
        if k != 9:
            assert lib.dataflow_find_table(C.byref(t), C.byref(C.c_uint64(k)), False, None) >= 0
    lib.dataflow_destroy_table(C.byref(t))


def test_scalar_bf16_helpers(lib):
    assert lib.solo_fp32_to_bf16(1.0) == 0x3F80
    assert lib.solo_fp32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80          # tie to even
    assert lib.solo_fp32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82
    assert lib.solo_bf16_to_fp32(0xC000) == -2.0


def test_layer_sizing_needs_no_gpu(lib):
    small = lib.amd_moe_layer_bytes(256, 512, 8, 2, 1024)
    big = lib.amd_moe_layer_bytes(8192, 4096, 64, 8, 1024)
    assert small % 256 == 0 and big > small
    # weights + grads alone: 2 * E * 3 * D * H * 2 bytes
    assert big >= 2 * 64 * 3 * 4096 * 1024 * 2


def test_init_handle_rejects_bad_arguments_without_touching_a_gpu(lib):
    h = B.DataflowHandle()
    assert lib.dataflow_init_handle(C.byref(h), B.COMPUTE_CUDA, 0, 0, 0, 8, None, None, 1.0) == -1
    assert lib.dataflow_init_handle(C.byref(h), B.COMPUTE_HSA, 0, 0, 0, 0, None, None, 1.0) == -1
    assert lib.dataflow_init_handle(None, B.COMPUTE_HSA, 0, 0, 0, 8, None, None, 1.0) == -1
    assert lib.dataflow_register_default_ops(C.byref(B.DataflowHandle())) == -1


def test_missing_artifacts_fail_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(B, "LIB_DIR", str(tmp_path))
    monkeypatch.setattr(B, "_lib", None)
    with pytest.raises(RuntimeError, match="no fallback"):
        B.load_library()
