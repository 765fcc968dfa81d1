"""Drop-in check: the reference's OWN submit wrappers drive this backend.

oracle/_ref/libref_ops.so is compiled from the reference's libdataflowops sources (submit_ops/moe_ops.c, matmul_op.c,
mlp_misc_ops.c, norm_ops.c, optimizer_ops.c, cast_ops.c + set_op_skeletons.c + its fingerprint code), linked so that its
internal calls stay inside it.  Each wrapper builds an Op on its stack exactly as the reference's model code does
(nickname, dtypes, SHA-256 fingerprint, op_args = addresses of its arguments) and calls handle->submit_op on the
handle it is given: here, the handle filled by this repository's dataflow_init_handle.  The op parity tests of
test_gpu_ops.py / test_gpu_norm.py / test_adamw.py are then re-run with those wrappers in place of this
repository's, against the same CPU oracle and to the same bar.

The library is built in the container that holds the reference tree and travels with the repository; where it is
absent the module is skipped (the reference's sources are not part of this repository).
"""
import ctypes as C
import os

import pytest

from ml_dataflow_amd import binding as B
import test_adamw
import test_cast
import test_gpu_norm
import test_gpu_ops

pytestmark = pytest.mark.gpu

REF_OPS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle", "_ref", "libref_ops.so")


class ReferenceWrappers:
    """`lib` stand-in: a dataflow_submit_* symbol that the reference's library defines is taken from there (typed
    like this repository's declaration of the same name), everything else from this repository's library."""

    def __init__(self, own, ref):
        self._own = own
        self._ref = ref
        self.taken_from_reference = set()

    def __getattr__(self, name):
        # the reference's cast_and_add wrapper stores its pointer arguments themselves in the argument slots instead of
        # their addresses (cast_ops.c:39-42) and cannot drive any backend: this repository's wrapper stays in place
        if name.startswith("dataflow_submit_") and name in B.SIGNATURES and name != "dataflow_submit_cast_and_add":
            try:
                fn = getattr(self._ref, name)
            except AttributeError:
                return getattr(self._own, name)
            fn.restype, fn.argtypes = B.SIGNATURES[name]
            self.taken_from_reference.add(name)
            return fn
        return getattr(self._own, name)


class BackendThroughReference:
    def __init__(self, backend, lib):
        self._backend = backend
        self.lib = lib

    def __getattr__(self, name):
        return getattr(self._backend, name)


@pytest.fixture(scope="module")
def ref_backend(backend):
    if not os.path.exists(REF_OPS):
        pytest.skip("oracle/_ref/libref_ops.so not built (needs the reference tree: make -C oracle ref)")
    ref = C.CDLL(REF_OPS, mode=C.RTLD_LOCAL)
    return BackendThroughReference(backend, ReferenceWrappers(backend.lib, ref))


def test_routing_through_reference_wrappers(ref_backend, oracle):
    test_gpu_ops.test_select_experts_bit_exact(ref_backend, oracle, 1000, 32, 4, True)
    test_gpu_ops.test_select_experts_bit_exact(ref_backend, oracle, 8192, 64, 8, False)
    test_gpu_ops.test_build_expert_mapping_bit_exact(ref_backend, oracle, 3000, 300, 6)
    test_gpu_ops.test_router_gate_bwd_x(ref_backend, oracle)
    taken = ref_backend.lib.taken_from_reference
    assert {"dataflow_submit_default_select_experts", "dataflow_submit_default_build_expert_mapping", "dataflow_submit_router_gate_bwd_x"} <= taken


def test_movement_through_reference_wrappers(ref_backend, oracle):
    test_gpu_ops.test_dispatch_bit_exact(ref_backend, oracle, 1000, 512, 32, 4)
    test_gpu_ops.test_combine_bit_exact(ref_backend, oracle, 1000, 512, 32, 4, True)
    test_gpu_ops.test_combine_bit_exact(ref_backend, oracle, 1000, 512, 32, 4, False)
    test_gpu_ops.test_per_expert_combine(ref_backend, oracle)
    test_gpu_ops.test_swiglu_forward_and_backward(ref_backend, oracle, 1000, 1408)
    test_gpu_ops.test_router_bwd_x_per_expert_and_all(ref_backend, oracle, 512, 256, 8, 2)
    taken = ref_backend.lib.taken_from_reference
    assert {"dataflow_submit_default_prepare_experts", "dataflow_submit_default_prepare_expert_zone", "dataflow_submit_default_merge_experts",
            "dataflow_submit_default_merge_expert_result", "dataflow_submit_default_swiglu", "dataflow_submit_default_swiglu_bwd_x",
            "dataflow_submit_router_bwd_x"} <= taken


def test_matmul_through_reference_wrapper(ref_backend, oracle):
    for transa, transb in ((1, 0), (0, 0), (0, 1), (1, 1)):
        test_gpu_ops.test_matmul_layouts(ref_backend, oracle, transa, transb, 256, 512, 384)
    test_gpu_ops.test_matmul_unaligned_shapes_take_the_scalar_path(ref_backend, oracle, 100, 52, 36)
    assert "dataflow_submit_matmul" in ref_backend.lib.taken_from_reference


def test_norm_and_adamw_through_reference_wrappers(ref_backend, oracle):
    test_gpu_norm.test_rms_norm_forward_and_recompute(ref_backend, oracle, 1000, 2048)
    test_gpu_norm.test_rms_norm_bwd_x(ref_backend, oracle, 1000, 2048, True)
    test_gpu_norm.test_rms_norm_bwd_x(ref_backend, oracle, 1000, 2048, False)
    test_gpu_norm.test_rms_norm_bwd_w(ref_backend, oracle, 1000, 2048, 512)
    test_adamw.test_gpu_matches_oracle(ref_backend, oracle, 100003, 5, 0)
    taken = ref_backend.lib.taken_from_reference
    assert {"dataflow_submit_default_rms_norm", "dataflow_submit_default_rms_norm_recompute", "dataflow_submit_default_rms_norm_bwd_x",
            "dataflow_submit_default_rms_norm_bwd_w", "dataflow_submit_default_adamw_step"} <= taken


def test_cast_through_reference_wrapper(ref_backend, oracle):
    test_cast.test_gpu_cast_matches_oracle(ref_backend, oracle, 100003, 0)
    test_cast.test_gpu_cast_matches_oracle(ref_backend, oracle, 5000, 1)
    assert "dataflow_submit_cast" in ref_backend.lib.taken_from_reference
