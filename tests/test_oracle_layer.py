"""Pins the oracle's layer forward / backward (the op sequence of dataflow_transformer.c:2700-2986,
3386-3719, 4013-4185) against an independent fp64 numpy model of a top-k softmax-gated SwiGLU MoE and
central finite differences of L = <dY, MoE(X)> with the routing decision held fixed.
"""
import numpy as np
import pytest

import oracle_lib as O
from util import f32_to_bf16, bf16_to_f64, normal_bf16


def moe_f64(X, Wr, W1, W3, W2, chosen):
    """dense fp64 model: softmax over the selected logits, SwiGLU experts, weighted sum"""
    T, K = chosen.shape
    logits = X @ Wr.T
    sel = np.take_along_axis(logits, chosen, axis=1)
    p = np.exp(sel - sel.max(1, keepdims=True))
    p /= p.sum(1, keepdims=True)
    out = np.zeros_like(X)
    for t in range(T):
        for k in range(K):
            e = chosen[t, k]
            a = W1[e] @ X[t]
            b = W3[e] @ X[t]
            h = a / (1 + np.exp(-a)) * b
            out[t] += p[t, k] * (W2[e] @ h)
    return out


def setup(seed, T=24, D=32, E=4, K=2, H=48, wstd=0.25):
    rng = np.random.default_rng(seed)
    X = normal_bf16(rng, (T, D))
    Wr = normal_bf16(rng, (E, D), wstd)
    W1 = normal_bf16(rng, (E, H, D), wstd)
    W3 = normal_bf16(rng, (E, H, D), wstd)
    W2 = normal_bf16(rng, (E, D, H), wstd)
    dY = normal_bf16(rng, (T, D))
    return rng, (T, D, E, K, H), X, Wr, W1, W3, W2, dY


@pytest.mark.parametrize("seed", [0, 1])
def test_forward_matches_fp64_model(oracle, seed):
    rng, (T, D, E, K, H), X, Wr, W1, W3, W2, dY = setup(seed)
    L = O.Layer(oracle, T, D, E, K, H, Wr, W1, W3, W2)
    resid = normal_bf16(rng, (T, D))
    out = L.forward(X, resid)
    f = bf16_to_f64
    want = f(resid) + moe_f64(f(X), f(Wr), f(W1), f(W3), f(W2), L.chosen.astype(np.int64))
    scale = np.abs(want).max()
    assert np.abs(f(out) - want).max() <= 2e-2 * scale
    # bookkeeping invariants of the saved state
    assert L.counts[:E].sum() == T * K and L.counts[E] == 1
    assert (L.cumsum == np.cumsum(L.counts[:E])).all()
    assert (L.expert_mapping[L.token_mapping] == np.arange(T)[:, None]).all()


def test_forward_with_logit_bias_moves_routing(oracle):
    rng, (T, D, E, K, H), X, Wr, W1, W3, W2, dY = setup(2)
    L = O.Layer(oracle, T, D, E, K, H, Wr, W1, W3, W2)
    bias = np.zeros((T, E), dtype=np.float32)
    bias[:, 3] = 100.0
    L.forward(X, np.zeros((T, D), dtype=np.uint16), logit_bias=f32_to_bf16(bias))
    assert (L.chosen == 3).any(axis=1).all()
    assert L.counts[3] == T


@pytest.mark.parametrize("seed", [0, 3])
def test_backward_matches_finite_differences(oracle, seed):
    rng, (T, D, E, K, H), X, Wr, W1, W3, W2, dY = setup(seed)
    L = O.Layer(oracle, T, D, E, K, H, Wr, W1, W3, W2)
    L.forward(X, np.zeros((T, D), dtype=np.uint16))
    dX = L.backward(X, dY)
    chosen = L.chosen.astype(np.int64)
    f = bf16_to_f64
    params = {"X": f(X), "Wr": f(Wr), "W1": f(W1), "W3": f(W3), "W2": f(W2)}
    grads = {"X": f(dX), "Wr": f(L.dWr), "W1": f(L.dW1), "W3": f(L.dW3), "W2": f(L.dW2)}
    g = f(dY)

    def loss(p):
        return float((g * moe_f64(p["X"], p["Wr"], p["W1"], p["W3"], p["W2"], chosen)).sum())

    eps = 1e-5
    for name in params:
        for trial in range(3):
            V = rng.standard_normal(params[name].shape)
            plus = dict(params); plus[name] = params[name] + eps * V
            minus = dict(params); minus[name] = params[name] - eps * V
            fd = (loss(plus) - loss(minus)) / (2 * eps)
            got = float((grads[name] * V).sum())
            # bf16 rounding noise of the stored gradient projects to ~2^-9 * |grad| * |V| / sqrt(n)
            noise = 2.0 ** -8 * np.linalg.norm(grads[name]) * np.linalg.norm(V) / np.sqrt(V.size) * 4
            assert abs(got - fd) <= 3e-2 * abs(fd) + noise + 1e-6, (name, trial, got, fd)


def test_backward_accumulates_weight_gradients(oracle):
    rng, (T, D, E, K, H), X, Wr, W1, W3, W2, dY = setup(4)
    L = O.Layer(oracle, T, D, E, K, H, Wr, W1, W3, W2)
    L.forward(X, np.zeros((T, D), dtype=np.uint16))
    L.backward(X, dY)
    once = bf16_to_f64(L.dW2).copy()
    L.forward(X, np.zeros((T, D), dtype=np.uint16))
    L.backward(X, dY)
    twice = bf16_to_f64(L.dW2)
    assert np.abs(twice - 2 * once).max() <= 2.0 ** -6 * np.abs(once).max() + 1e-12


def test_unrouted_expert_leaves_its_gradients_untouched(oracle):
    rng, (T, D, E, K, H), X, Wr, W1, W3, W2, dY = setup(5, E=6)
    L = O.Layer(oracle, T, D, 6, K, H, Wr, W1, W3, W2)
    bias = np.zeros((T, 6), dtype=np.float32)
    bias[:, 5] = -1000.0           # expert 5 never selected
    L.dW1[5] = 0x3F80
    L.forward(X, np.zeros((T, D), dtype=np.uint16), logit_bias=f32_to_bf16(bias))
    L.backward(X, dY)
    assert L.counts[5] == 0
    assert (L.dW1[5] == 0x3F80).all() and (L.dW2[5] == 0).all()
