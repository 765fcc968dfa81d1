"""The reference's own model code on this backend: dataflow_submit_transformer_moe_block_bwd_w
(libdataflowmodels/src/transformer/src/dataflow_transformer.c:3970-4247), compiled where it lies into
oracle/_ref/libref_models.so together with prep_seq_batch.c and the reference's submit wrappers, is handed the
Dataflow_Handle that this repository's dataflow_init_handle filled.  It re-dispatches the layer input, loops over the
experts on two streams for dW1 / dW3, accumulates the router's weight gradient and the four attention projection
weight gradients -- all through default_prepare_experts and default_matmul on this backend.

The structs it takes (Transformer_Block, Seq_Batch, Seq_Batch_Saved_Activations, Seq_Batch_Activation_Workspace:
transformer_structs.h, seq_batch_structs.h:206-281, 369-395) are filled by oracle/ref_bwd_w_driver.c, compiled against
the reference's headers, with the per-expert x_1 / x_3 pointers set by the reference's own
set_moe_working_activations_offsets (prep_seq_batch.c:370-397) from the host-side expert counts: so the buffer contract
this repository's layer keeps (expert-major rows of dx1 / dx3, token_mapping, host_expert_counts) is checked against
the real structs, not a restatement.

Skipped where oracle/_ref/libref_models.so is absent (it is built in the container that holds the reference tree)."""
import ctypes as C
import os

import numpy as np
import pytest

import oracle_lib as O
from ml_dataflow_amd import MoeLayer, binding as B
from util import normal_bf16, close

pytestmark = pytest.mark.gpu

REF_MODELS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle", "_ref", "libref_models.so")
_P, _I = C.c_void_p, C.c_int


class RefBwdWArgs(C.Structure):                      # oracle/ref_bwd_w_driver.c: Ref_Bwd_W_Args
    _fields_ = [("total_q", _I), ("model_dim", _I), ("attn_dim", _I), ("kv_dim", _I), ("ffn_dim", _I),
                ("num_routed_experts", _I), ("top_k_experts", _I), ("block_dt", _I), ("compute_dt", _I),
                ("host_expert_counts", _P), ("token_mapping", _P), ("x_attn_out", _P),
                ("recomputed_ffn_norm", _P), ("recomputed_attn_norm", _P), ("dx1_base", _P), ("dx3_base", _P), ("d_routed", _P),
                ("d_o", _P), ("d_q", _P), ("d_k_local", _P), ("d_v_local", _P),
                ("expert_zones", _P), ("kernel_workspace", _P), ("kernel_workspace_bytes", C.c_uint64),
                ("dw1_base", _P), ("dw3_base", _P), ("expert_stride_bytes", C.c_uint64),
                ("dw_router", _P), ("dw_o", _P), ("dw_q", _P), ("dw_k", _P), ("dw_v", _P)]


@pytest.mark.parametrize("T,D,E,K,H,attn_dim,kv_dim", [(512, 256, 8, 2, 128, 64, 32), (300, 512, 16, 4, 264, 128, 128)])
def test_reference_bwd_w_runs_on_this_backend(backend, oracle, T, D, E, K, H, attn_dim, kv_dim):
    if not os.path.exists(REF_MODELS):
        pytest.skip("oracle/_ref/libref_models.so not built (needs the reference tree: make -C oracle ref)")
    print("case reference bwd_w T=%d D=%d E=%d K=%d H=%d" % (T, D, E, K, H), flush=True)
    ref = C.CDLL(REF_MODELS, mode=C.RTLD_LOCAL)
    ref.ref_moe_block_bwd_w.restype = _I
    ref.ref_moe_block_bwd_w.argtypes = [C.POINTER(B.DataflowHandle), _I, _I, C.POINTER(RefBwdWArgs)]
    be = backend
    rng = np.random.default_rng(T + D + E)
    Wr, W1, W3, W2 = (normal_bf16(rng, s, 0.05) for s in ((E, D), (E, H, D), (E, H, D), (E, D, H)))
    X, resid, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    layer = MoeLayer(be, T, D, E, K, H)
    layer.load_weights(Wr, W1, W3, W2)
    d_X, d_out, d_dY, d_dX = be.upload(X), be.upload(resid), be.upload(dY), be.alloc(T * D * 2)
    # forward + backward by this repository's layer in the reference's own schedule: leaves dx1 / dx3 / d_routed /
    # token_mapping / host_expert_counts as the reference's bwd_x would, and its own dW1 / dW3 / dWr to compare with
    layer.forward(T, d_X.ptr, d_out.ptr, None, B.AMD_MOE_PER_EXPERT)
    layer.zero_grads()
    layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, B.AMD_MOE_PER_EXPERT)
    be.sync()
    own_dWr, own_dW1, own_dW3, _ = layer.read_grads()
    logits = be.read(layer.L.x_routed, (T, E), np.uint16)

    # attention-side operands of the same function: plain matmuls, random inputs
    attn_out, attn_norm = normal_bf16(rng, (T, attn_dim)), normal_bf16(rng, (T, D))
    g_o, g_q = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, attn_dim))
    g_k, g_v = normal_bf16(rng, (T, kv_dim)), normal_bf16(rng, (T, kv_dim))
    d_attn_out, d_attn_norm, d_go, d_gq, d_gk, d_gv = (be.upload(a) for a in (attn_out, attn_norm, g_o, g_q, g_k, g_v))
    dw_o, dw_q, dw_k, dw_v = be.alloc(D * attn_dim * 2), be.alloc(attn_dim * D * 2), be.alloc(kv_dim * D * 2), be.alloc(kv_dim * D * 2)
    for buf, n in ((dw_o, D * attn_dim), (dw_q, attn_dim * D), (dw_k, kv_dim * D), (dw_v, kv_dim * D)):
        be.zero(buf.ptr, n * 2)

    layer.zero_grads()
    L = layer.L
    args = RefBwdWArgs(total_q=T, model_dim=D, attn_dim=attn_dim, kv_dim=kv_dim, ffn_dim=H, num_routed_experts=E, top_k_experts=K,
                       block_dt=B.DATAFLOW_BF16, compute_dt=B.DATAFLOW_FP32, host_expert_counts=L.host_expert_counts,
                       token_mapping=L.token_mapping, x_attn_out=d_attn_out.ptr, recomputed_ffn_norm=d_X.ptr, recomputed_attn_norm=d_attn_norm.ptr,
                       dx1_base=L.dx1, dx3_base=L.dx3, d_routed=L.d_routed, d_o=d_go.ptr, d_q=d_gq.ptr, d_k_local=d_gk.ptr, d_v_local=d_gv.ptr,
                       expert_zones=L.expert_zones, kernel_workspace=L.kernel_workspace, kernel_workspace_bytes=L.kernel_workspace_bytes,
                       dw1_base=L.dw1, dw3_base=L.dw3, expert_stride_bytes=L.expert_stride_bytes, dw_router=L.dw_router,
                       dw_o=dw_o.ptr, dw_q=dw_q.ptr, dw_k=dw_k.ptr, dw_v=dw_v.ptr)
    assert ref.ref_moe_block_bwd_w(be.hp, 1, 2, C.byref(args)) == 0
    be.sync()
    dWr, dW1, dW3, _ = layer.read_grads()
    # the same ops in the same order as this repository's per-expert schedule: identical bits
    assert (dWr == own_dWr).all() and (dW1 == own_dW1).all() and (dW3 == own_dW3).all()
    # and the oracle's values
    ol = O.Layer(oracle, T, D, E, K, H, Wr, W1, W3, W2)
    ol.forward(X, resid, logits=logits)
    ol.backward(X, dY)
    close(dW1, ol.dW1, what="dW1")
    close(dW3, ol.dW3, what="dW3")
    close(dWr, ol.dWr, what="dWr")
    # attention projection weight gradients: dW[n, m] = sum_t B[t, n] * A[t, m]  (to_trans_a 0, to_trans_b 1)
    for name, buf, A, Bm, M, N in (("dw_o", dw_o, attn_out, g_o, attn_dim, D), ("dw_q", dw_q, attn_norm, g_q, D, attn_dim),
                                   ("dw_k", dw_k, attn_norm, g_k, D, kv_dim), ("dw_v", dw_v, attn_norm, g_v, D, kv_dim)):
        want = O.matmul(oracle, 0, 1, M, T, N, A, Bm, 1.0, 1.0, np.zeros((N, M), np.uint16))
        close(be.read(buf.ptr, (N, M), np.uint16), want, what=name)
    layer.free()
