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

The forward and bwd_x block functions of the reference (dataflow_submit_transformer_moe_block, dataflow_transformer.c:2197-2986,
and ..._bwd_x, :3326-3968) run here too, through oracle/ref_block_driver.c: the reference's host sync after routing, its
host_expert_counts and its per-expert loop over two streams drive this backend unmodified.  The four ops of the
attention half that those functions submit (rope, attention forward / backward, rope backward) are outside the MoE
path; the driver registers an op that does nothing for each through the handle's register_external_code, with the
reference's own skeletons, and the test puts known values where those ops would have written.

Skipped where oracle/_ref/libref_models.so is absent because the reference tree was not there at build time; where it
was (oracle/ref_built.marker, written by `make -C oracle ref`) a missing library is a failure."""
import ctypes as C
import os

import numpy as np
import pytest

import oracle_lib as O
from ml_dataflow_amd import MoeLayer, binding as B
from util import normal_bf16, close, f32_to_bf16

pytestmark = pytest.mark.gpu

REF_MODELS = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle", "_ref", "libref_models.so")
REF_MARKER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle", "ref_built.marker")
_P, _I = C.c_void_p, C.c_int


def reference_models_library():
    if not os.path.exists(REF_MODELS):
        assert not os.path.exists(REF_MARKER), "oracle/_ref/libref_models.so is missing although the reference tree was there at build time"
        pytest.skip("oracle/_ref/libref_models.so not built (needs the reference tree: make -C oracle ref)")
    return C.CDLL(REF_MODELS, mode=C.RTLD_LOCAL)


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
    ref = reference_models_library()
    print("case reference bwd_w T=%d D=%d E=%d K=%d H=%d" % (T, D, E, K, H), flush=True)
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


class RefBlockArgs(C.Structure):                     # oracle/ref_block_driver.c: Ref_Block_Args
    _fields_ = [(n, _I) for n in ("total_q", "model_dim", "attn_dim", "kv_dim", "ffn_dim", "num_routed_experts", "top_k_experts",
                                  "num_q_heads", "num_kv_heads", "head_dim", "block_dt", "compute_dt")] + [("eps", C.c_float)] + \
               [(n, _P) for n in ("host_expert_counts", "w_attn_norm", "w_q", "w_k", "w_v", "w_o", "w_ffn_norm", "w_router", "w1_base", "w3_base", "w2_base")] + \
               [("expert_stride_bytes", C.c_uint64)] + \
               [(n, _P) for n in ("x_inp", "attn_norm_rms_vals", "ffn_norm_rms_vals", "x_q", "x_k_local", "x_v_local", "x_attn_out", "softmax_lse", "x_o",
                                  "x_routed", "token_expert_weights", "chosen_experts", "expert_counts", "expert_counts_cumsum", "expert_mapping",
                                  "token_mapping", "x1_base", "x3_base", "ctx_k", "ctx_v", "x_temp", "x_temp_mlp", "expert_zones", "kernel_workspace")] + \
               [("kernel_workspace_bytes", C.c_uint64)] + \
               [(n, _P) for n in ("X_in", "X_out", "g_x_routed", "g_x_q", "g_x_k_local", "g_x_v_local", "g_x_o", "g_x1_base", "g_x3_base",
                                  "recomputed_ffn_norm", "recomputed_attn_norm", "g_ctx_k", "g_ctx_v", "dw2_base", "dw_ffn_norm", "dw_attn_norm")]


_noop_ops_registered = set()


@pytest.mark.parametrize("T,D,E,K,H,heads,kv_heads,head_dim", [(384, 256, 8, 2, 128, 4, 2, 16), (300, 512, 16, 4, 264, 8, 8, 16)])
def test_reference_forward_and_bwd_x_run_on_this_backend(backend, oracle, T, D, E, K, H, heads, kv_heads, head_dim):
    ref = reference_models_library()
    print("case reference forward + bwd_x T=%d D=%d E=%d K=%d H=%d" % (T, D, E, K, H), flush=True)
    be = backend
    BF = B.DATAFLOW_BF16
    EPS = 1e-5
    attn_dim, kv_dim, R = heads * head_dim, kv_heads * head_dim, T * K
    for fn in (ref.ref_moe_block_forward, ref.ref_moe_block_bwd_x):
        fn.restype = _I
        fn.argtypes = [C.POINTER(B.DataflowHandle), _I, _I, C.POINTER(RefBlockArgs)]
    ref.ref_register_noop_ops.restype = _I
    ref.ref_register_noop_ops.argtypes = [C.POINTER(B.DataflowHandle), C.c_char_p, _I]
    if id(be) not in _noop_ops_registered:             # once per handle: the op table keeps them
        assert ref.ref_register_noop_ops(be.hp, os.path.realpath(REF_MODELS).encode(), BF) == 4
        _noop_ops_registered.add(id(be))

    rng = np.random.default_rng(T + D + E + H)
    Wr, W1, W3, W2 = (normal_bf16(rng, s, 0.05) for s in ((E, D), (E, H, D), (E, H, D), (E, D, H)))
    Wq, Wk, Wv, Wo = (normal_bf16(rng, s, 0.05) for s in ((attn_dim, D), (kv_dim, D), (kv_dim, D), (D, attn_dim)))
    w_an = f32_to_bf16((1.0 + 0.1 * rng.standard_normal(D)).astype(np.float32))
    w_fn = f32_to_bf16((1.0 + 0.1 * rng.standard_normal(D)).astype(np.float32))
    X, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
    attn_out = normal_bf16(rng, (T, attn_dim))        # what the attention op would have written
    dQ, dK, dV = normal_bf16(rng, (T, attn_dim)), normal_bf16(rng, (T, kv_dim)), normal_bf16(rng, (T, kv_dim))   # and its backward

    up = be.upload
    d = {n: up(a) for n, a in dict(Wr=Wr, W1=W1, W3=W3, W2=W2, Wq=Wq, Wk=Wk, Wv=Wv, Wo=Wo, w_an=w_an, w_fn=w_fn, X=X, dY=dY, attn_out=attn_out,
                                   g_x_q=dQ, g_ctx_k=dK, g_ctx_v=dV).items()}
    sizes = dict(x_inp=T * D * 2, attn_rms=T * 4, ffn_rms=T * 4, x_q=T * attn_dim * 2, x_k=T * kv_dim * 2, x_v=T * kv_dim * 2, lse=T * heads * 4,
                 x_o=T * D * 2, logits=T * E * 2, tw=T * K * 4, chosen=T * K * 2, counts=(E + 1) * 4, cumsum=E * 4, emap=R * 4, tmap=R * 4,
                 x1=R * H * 2, x3=R * H * 2, ctx_k=T * kv_dim * 2, ctx_v=T * kv_dim * 2, x_temp=T * D * 2, x_temp_mlp=T * H * 2, zones=R * D * 2,
                 ws=16 << 20, out=T * D * 2, next_grad=T * D * 2, g_logits=T * E * 2, g_x_k=T * kv_dim * 2, g_x_v=T * kv_dim * 2, g_x_o=T * D * 2,
                 g_x1=R * H * 2, g_x3=R * H * 2, rec_ffn=T * D * 2, rec_attn=T * D * 2, dW2=E * D * H * 2, dw_fn=D * 2, dw_an=D * 2)
    for n, nbytes in sizes.items():
        d[n] = be.alloc(nbytes)
        be.zero(d[n].ptr, nbytes)
    host_counts = be.host_alloc(E * 4)
    p = lambda n: d[n].ptr
    args = RefBlockArgs(total_q=T, model_dim=D, attn_dim=attn_dim, kv_dim=kv_dim, ffn_dim=H, num_routed_experts=E, top_k_experts=K,
                        num_q_heads=heads, num_kv_heads=kv_heads, head_dim=head_dim, block_dt=BF, compute_dt=B.DATAFLOW_FP32, eps=EPS,
                        host_expert_counts=host_counts, w_attn_norm=p("w_an"), w_q=p("Wq"), w_k=p("Wk"), w_v=p("Wv"), w_o=p("Wo"),
                        w_ffn_norm=p("w_fn"), w_router=p("Wr"), w1_base=p("W1"), w3_base=p("W3"), w2_base=p("W2"), expert_stride_bytes=H * D * 2,
                        x_inp=p("x_inp"), attn_norm_rms_vals=p("attn_rms"), ffn_norm_rms_vals=p("ffn_rms"), x_q=p("x_q"), x_k_local=p("x_k"),
                        x_v_local=p("x_v"), x_attn_out=p("attn_out"), softmax_lse=p("lse"), x_o=p("x_o"), x_routed=p("logits"),
                        token_expert_weights=p("tw"), chosen_experts=p("chosen"), expert_counts=p("counts"), expert_counts_cumsum=p("cumsum"),
                        expert_mapping=p("emap"), token_mapping=p("tmap"), x1_base=p("x1"), x3_base=p("x3"), ctx_k=p("ctx_k"), ctx_v=p("ctx_v"),
                        x_temp=p("x_temp"), x_temp_mlp=p("x_temp_mlp"), expert_zones=p("zones"), kernel_workspace=p("ws"),
                        kernel_workspace_bytes=sizes["ws"], X_in=p("X"), X_out=p("out"), g_x_routed=p("g_logits"), g_x_q=p("g_x_q"),
                        g_x_k_local=p("g_x_k"), g_x_v_local=p("g_x_v"), g_x_o=p("g_x_o"), g_x1_base=p("g_x1"), g_x3_base=p("g_x3"),
                        recomputed_ffn_norm=p("rec_ffn"), recomputed_attn_norm=p("rec_attn"), g_ctx_k=p("g_ctx_k"), g_ctx_v=p("g_ctx_v"),
                        dw2_base=p("dW2"), dw_ffn_norm=p("dw_fn"), dw_attn_norm=p("dw_an"))

    # ---------------- forward: the reference's dataflow_submit_transformer_moe_block
    assert ref.ref_moe_block_forward(be.hp, 1, 2, C.byref(args)) == 0
    be.sync()
    rd = lambda n, shape, dt=np.uint16: be.read(d[n].ptr, shape, dt)
    assert (rd("x_inp", (T, D)) == X).all()                                         # the block input is saved
    attn_norm, attn_rms = np.zeros_like(X), np.zeros(T, dtype=np.float32)
    oracle.oracle_rms_norm(T, D, EPS, O.ptr(w_an), O.ptr(X), O.ptr(attn_norm), O.ptr(attn_rms))
    np.testing.assert_allclose(rd("attn_rms", (T,), np.float32), attn_rms, rtol=1e-5)
    close(rd("x_q", (T, attn_dim)), O.matmul(oracle, 1, 0, attn_dim, D, T, Wq, attn_norm), steps=3, what="x_q")
    close(rd("x_k", (T, kv_dim)), O.matmul(oracle, 1, 0, kv_dim, D, T, Wk, attn_norm), steps=3, what="x_k")
    assert (rd("ctx_k", (T, kv_dim)) == rd("x_k", (T, kv_dim))).all()               # keys and values reach the context
    assert (rd("ctx_v", (T, kv_dim)) == rd("x_v", (T, kv_dim))).all()
    x_o = rd("x_o", (T, D))
    close(x_o, O.matmul(oracle, 1, 0, D, attn_dim, T, Wo, attn_out, 1.0, 1.0, X), what="x_o")
    normed = rd("x_temp", (T, D))                                                   # the MoE layer's input: the FFN norm of x_o
    want_normed, ffn_rms = np.zeros_like(X), np.zeros(T, dtype=np.float32)
    oracle.oracle_rms_norm(T, D, EPS, O.ptr(w_fn), O.ptr(x_o), O.ptr(want_normed), O.ptr(ffn_rms))
    close(normed, want_normed, what="ffn norm")
    logits = rd("logits", (T, E))
    ol = O.Layer(oracle, T, D, E, K, H, Wr, W1, W3, W2)
    ol.forward(normed, x_o)
    close(logits, ol.logits, what="router logits")
    out_o = ol.forward(normed, x_o, logits=logits)                                  # routing replayed on the GPU's logits
    counts = np.ctypeslib.as_array(C.cast(host_counts, C.POINTER(C.c_int32)), (E,)).copy()
    assert (rd("chosen", (T, K)) == ol.chosen).all()
    assert (counts == ol.counts[:E]).all() and (rd("counts", (E + 1,), np.int32)[:E] == ol.counts[:E]).all()
    assert (rd("cumsum", (E,), np.int32) == ol.cumsum).all()
    assert (rd("emap", (R,), np.int32) == ol.expert_mapping).all() and (rd("tmap", (T, K), np.int32) == ol.token_mapping).all()
    np.testing.assert_allclose(rd("tw", (T, K), np.float32), ol.weights, rtol=2e-6, atol=1e-9)
    close(rd("x1", (R, H)), ol.x1, what="x1")                                        # expert-major rows, carved by the reference's own offsets
    close(rd("x3", (R, H)), ol.x3, what="x3")
    close(rd("out", (T, D)), out_o, what="block output")

    # ---------------- backward w.r.t. activations: the reference's dataflow_submit_transformer_moe_block_bwd_x
    args.X_in, args.X_out = p("dY"), p("next_grad")
    assert ref.ref_moe_block_bwd_x(be.hp, 1, 2, C.byref(args)) == 0
    be.sync()
    dX_moe = ol.backward(normed, dY)
    close(rd("g_logits", (T, E)), ol.dlogits, what="router-logit gradient")
    close(rd("g_x1", (R, H)), ol.dx1, what="dx1")
    close(rd("g_x3", (R, H)), ol.dx3, what="dx3")
    close(rd("dW2", (E, D, H)), ol.dW2, what="dW2")
    # through the FFN norm: the upstream gradient plus the norm's backward of the layer's dX (chained with the oracle's dX)
    want_gxo, rec = dY.copy(), np.zeros_like(X)
    oracle.oracle_rms_norm_bwd_x(T, D, EPS, O.ptr(ffn_rms), O.ptr(w_fn), O.ptr(x_o), O.ptr(dX_moe), O.ptr(want_gxo), O.ptr(rec))
    g_x_o = rd("g_x_o", (T, D))
    close(g_x_o, want_gxo, steps=4, what="gradient after the FFN norm")
    close(rd("rec_ffn", (T, D)), normed, what="recomputed FFN norm")
    want_dw_fn = np.zeros(D, dtype=np.uint16)
    oracle.oracle_rms_norm_bwd_w(T, D, EPS, O.ptr(ffn_rms), O.ptr(x_o), O.ptr(dX_moe), O.ptr(want_dw_fn))
    close(rd("dw_fn", (D,)), want_dw_fn, steps=4, what="FFN norm weight gradient")
    # the attention half with its backward ops doing nothing: dQ, dK, dV are the values put there
    assert (rd("g_x_k", (T, kv_dim)) == dK).all() and (rd("g_x_v", (T, kv_dim)) == dV).all()
    assert not rd("g_ctx_k", (T, kv_dim)).any() and not rd("g_ctx_v", (T, kv_dim)).any()      # the context gradients are cleared for the next layer
    U = O.matmul(oracle, 0, 0, D, attn_dim, T, Wq, dQ)
    U = O.matmul(oracle, 0, 0, D, kv_dim, T, Wk, dK, 1.0, 1.0, U)
    U = O.matmul(oracle, 0, 0, D, kv_dim, T, Wv, dV, 1.0, 1.0, U)
    want_next, rec = g_x_o.copy(), np.zeros_like(X)
    oracle.oracle_rms_norm_bwd_x(T, D, EPS, O.ptr(attn_rms), O.ptr(w_an), O.ptr(X), O.ptr(U), O.ptr(want_next), O.ptr(rec))
    close(rd("next_grad", (T, D)), want_next, steps=4, what="gradient leaving the block")
    close(rd("rec_attn", (T, D)), attn_norm, what="recomputed attention norm")
    want_dw_an = np.zeros(D, dtype=np.uint16)
    oracle.oracle_rms_norm_bwd_w(T, D, EPS, O.ptr(attn_rms), O.ptr(X), O.ptr(U), O.ptr(want_dw_an))
    close(rd("dw_an", (D,)), want_dw_an, steps=4, what="attention norm weight gradient")
    be.host_free(host_counts)
    for buf in d.values():
        buf.free()
