"""Golden fixtures of the MoE layer (tests/golden/*.npz, written by tests/golden/make_golden.py).

CPU: the oracle still reproduces them (integers exactly; values within one bf16 step, which allows for a
different libm build on another host).  GPU: the HIP path through the C ABI reproduces them (integers exactly,
values within 1e-2 of the tensor's scale, fp32 accumulation against the oracle's fp64)."""
import glob
import os

import numpy as np
import pytest

import oracle_lib as O
from util import bf16_to_f64, bf16_ulp_diff

FIXTURES = sorted(glob.glob(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "*.npz")))
INT_KEYS = ["chosen", "counts", "cumsum_inclusive", "expert_mapping", "token_mapping"]
VALUE_KEYS = ["logits", "x1", "x3", "out", "dX", "dx1", "dx3", "dlogits", "dWr", "dW1", "dW3", "dW2"]
TOL = 1e-2


def shape_of(fx):
    T, D = fx["X"].shape
    E, H, _ = fx["W1"].shape
    K = fx["chosen"].shape[1]
    return T, D, E, K, H


def test_fixtures_exist():
    assert len(FIXTURES) >= 2


@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_oracle_reproduces_fixture(oracle, path):
    fx = np.load(path)
    T, D, E, K, H = shape_of(fx)
    ol = O.Layer(oracle, T, D, E, K, H, fx["Wr"], fx["W1"], fx["W3"], fx["W2"])
    out = ol.forward(fx["X"], fx["residual"])
    dX = ol.backward(fx["X"], fx["dY"])
    got = dict(logits=ol.logits, weights=ol.weights, chosen=ol.chosen, counts=ol.counts[:E], cumsum_inclusive=ol.cumsum,
               expert_mapping=ol.expert_mapping, token_mapping=ol.token_mapping, x1=ol.x1, x3=ol.x3, out=out, dX=dX,
               dx1=ol.dx1, dx3=ol.dx3, dlogits=ol.dlogits, dWr=ol.dWr, dW1=ol.dW1, dW3=ol.dW3, dW2=ol.dW2)
    for k in INT_KEYS:
        assert (got[k] == fx[k]).all(), k
    np.testing.assert_allclose(got["weights"], fx["weights"], rtol=1e-6, atol=1e-9)
    for k in VALUE_KEYS:
        assert bf16_ulp_diff(got[k], fx[k]).max() <= 1, k


@pytest.mark.gpu
@pytest.mark.parametrize("schedule", [1, 0], ids=["grouped", "per_expert"])
@pytest.mark.parametrize("path", FIXTURES, ids=[os.path.basename(p) for p in FIXTURES])
def test_gpu_reproduces_fixture(backend, path, schedule):
    from ml_dataflow_amd import MoeLayer
    print("case golden %s schedule=%d" % (os.path.basename(path), schedule), flush=True)
    fx = np.load(path)
    T, D, E, K, H = shape_of(fx)
    R = T * K
    be = backend
    layer = MoeLayer(be, T, D, E, K, H)
    layer.load_weights(fx["Wr"], fx["W1"], fx["W3"], fx["W2"])
    d_X, d_out, d_dY, d_dX = be.upload(fx["X"]), be.upload(fx["residual"]), be.upload(fx["dY"]), be.alloc(T * D * 2)
    layer.forward(T, d_X.ptr, d_out.ptr, None, schedule)
    layer.zero_grads()
    layer.backward(T, d_X.ptr, d_dY.ptr, d_dX.ptr, schedule)
    be.sync()
    L = layer.L
    dWr, dW1, dW3, dW2 = layer.read_grads()
    got = dict(logits=be.read(L.x_routed, (T, E), np.uint16), weights=be.read(L.token_expert_weights, (T, K), np.float32),
               chosen=be.read(L.chosen_experts, (T, K), np.uint16), counts=be.read(L.expert_counts, (E,), np.int32),
               cumsum_inclusive=be.read(L.expert_counts_cumsum, (E,), np.int32), expert_mapping=be.read(L.expert_mapping, (R,), np.int32),
               token_mapping=be.read(L.token_mapping, (T, K), np.int32), x1=be.read(L.x1, (R, H), np.uint16),
               x3=be.read(L.x3, (R, H), np.uint16), out=be.read(d_out.ptr, (T, D), np.uint16), dX=be.read(d_dX.ptr, (T, D), np.uint16),
               dx1=be.read(L.dx1, (R, H), np.uint16), dx3=be.read(L.dx3, (R, H), np.uint16), dlogits=be.read(L.d_routed, (T, E), np.uint16),
               dWr=dWr, dW1=dW1, dW3=dW3, dW2=dW2)
    layer.free()
    assert bf16_ulp_diff(got["logits"], fx["logits"]).max() <= 1
    for k in INT_KEYS:                                              # the fixtures have a routing margin: exact
        assert (got[k] == fx[k]).all(), k
    np.testing.assert_allclose(got["weights"], fx["weights"], rtol=4e-2, atol=1e-6)   # a 1-step logit difference moves a weight by a few %
    for k in VALUE_KEYS[1:]:
        g, w = bf16_to_f64(got[k]), bf16_to_f64(fx[k])
        scale = max(float(np.abs(w).max()), 1e-30)
        assert float(np.abs(g - w).max()) <= TOL * scale, k
