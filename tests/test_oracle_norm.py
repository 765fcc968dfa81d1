"""Pins the oracle's RMS norm functions (oracle/moe_oracle.c) against the mathematics: the fp64 closed form for
the forward pass and the saved statistic, central finite differences and an orthogonality identity for the
backward pass w.r.t. the input, numpy column sums for the backward pass w.r.t. the scale."""
import numpy as np
import pytest

from oracle_lib import ptr
from util import bf16_to_f64, bf16_to_f32, f32_to_bf16, normal_bf16, bf16_ulp_diff

EPS = 1e-5


def fwd64(x, w, eps=EPS):
    r = 1.0 / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps)
    return x * r * w, r[:, 0]


@pytest.mark.parametrize("rows,cols,seed", [(1, 8, 0), (7, 64, 1), (33, 1000, 2), (16, 4096, 3)])
def test_forward_is_the_closed_form(oracle, rows, cols, seed):
    rng = np.random.default_rng(seed)
    X, W = normal_bf16(rng, (rows, cols), 2.0), f32_to_bf16(1.0 + 0.1 * rng.standard_normal(cols).astype(np.float32))
    out, rms = np.zeros((rows, cols), np.uint16), np.zeros(rows, np.float32)
    oracle.oracle_rms_norm(rows, cols, EPS, ptr(W), ptr(X), ptr(out), ptr(rms))
    want, r = fwd64(bf16_to_f64(X), bf16_to_f64(W))
    np.testing.assert_allclose(rms, r, rtol=3e-7)
    assert bf16_ulp_diff(out, f32_to_bf16(want.astype(np.float32))).max() <= 1      # double rounding fp64 -> fp32 -> bf16 vs fp32 chain
    # the statistic is optional
    out2 = np.zeros_like(out)
    oracle.oracle_rms_norm(rows, cols, EPS, ptr(W), ptr(X), ptr(out2), None)
    assert (out2 == out).all()
    # the same output from the saved statistic
    out3 = np.zeros_like(out)
    oracle.oracle_rms_norm_recompute(rows, cols, ptr(W), ptr(rms), ptr(X), ptr(out3))
    assert (out3 == out).all()


def test_forward_special_cases(oracle):
    cols = 64
    W = f32_to_bf16(np.ones(cols, np.float32))
    # a constant row c normalises to sign(c) (eps is negligible), a zero row stays zero with r = 1/sqrt(eps)
    X = f32_to_bf16(np.stack([np.full(cols, 3.0, np.float32), np.full(cols, -0.5, np.float32), np.zeros(cols, np.float32)]))
    out, rms = np.zeros((3, cols), np.uint16), np.zeros(3, np.float32)
    oracle.oracle_rms_norm(3, cols, EPS, ptr(W), ptr(X), ptr(out), ptr(rms))
    o = bf16_to_f32(out)
    assert np.allclose(o[0], 1.0, atol=1e-2) and np.allclose(o[1], -1.0, atol=1e-2) and (o[2] == 0).all()
    np.testing.assert_allclose(rms, [1 / 3.0, 2.0, 1 / np.sqrt(EPS)], rtol=1e-4)


@pytest.mark.parametrize("rows,cols,seed", [(3, 16, 0), (5, 96, 1)])
def test_bwd_x_matches_finite_differences(oracle, rows, cols, seed):
    rng = np.random.default_rng(seed)
    X, G = normal_bf16(rng, (rows, cols)), normal_bf16(rng, (rows, cols))
    W = f32_to_bf16(1.0 + 0.2 * rng.standard_normal(cols).astype(np.float32))
    x, g, w = bf16_to_f64(X), bf16_to_f64(G), bf16_to_f64(W)
    _, r = fwd64(x, w)
    rms = r.astype(np.float32)
    dX, Xout = np.zeros((rows, cols), np.uint16), np.zeros((rows, cols), np.uint16)
    oracle.oracle_rms_norm_bwd_x(rows, cols, EPS, ptr(rms), ptr(W), ptr(X), ptr(G), ptr(dX), ptr(Xout))
    # numerical gradient of f(x) = <g, norm(x)> per row
    num = np.zeros_like(x)
    h = 1e-6
    for i in range(cols):
        xp, xm = x.copy(), x.copy()
        xp[:, i] += h
        xm[:, i] -= h
        num[:, i] = ((fwd64(xp, w)[0] * g).sum(axis=1) - (fwd64(xm, w)[0] * g).sum(axis=1)) / (2 * h)
    got = bf16_to_f64(dX)
    scale = np.abs(num).max()
    assert np.abs(got - num).max() <= 6e-3 * scale                # one bf16 rounding of the result (2^-8 relative)
    want_out, _ = fwd64(x, w)
    assert bf16_ulp_diff(Xout, f32_to_bf16(want_out.astype(np.float32))).max() <= 1


def test_bwd_x_accumulates_and_is_orthogonal_to_x_for_unit_scale(oracle):
    rng = np.random.default_rng(5)
    rows, cols = 4, 128
    X, G = normal_bf16(rng, (rows, cols)), normal_bf16(rng, (rows, cols))
    W = f32_to_bf16(np.ones(cols, np.float32))
    x = bf16_to_f64(X)
    rms = fwd64(x, 1.0)[1].astype(np.float32)
    zero = np.zeros((rows, cols), np.uint16)
    oracle.oracle_rms_norm_bwd_x(rows, cols, EPS, ptr(rms), ptr(W), ptr(X), ptr(G), ptr(zero), None)
    d = bf16_to_f64(zero)
    # for w = 1 the gradient of a scale-invariant function is orthogonal to x (up to eps and bf16 rounding)
    assert np.abs((d * x).sum(axis=1)).max() <= 2e-2 * np.abs(d * x).sum(axis=1).max()
    # accumulation: starting from a non-zero dX adds the same derivative (one more rounding)
    start = normal_bf16(rng, (rows, cols))
    acc = start.copy()
    oracle.oracle_rms_norm_bwd_x(rows, cols, EPS, ptr(rms), ptr(W), ptr(X), ptr(G), ptr(acc), None)
    assert np.abs(bf16_to_f64(acc) - (bf16_to_f64(start) + d)).max() <= 2.0 ** -7 * np.abs(bf16_to_f64(acc)).max()


@pytest.mark.parametrize("rows,cols,seed", [(1, 8, 0), (50, 72, 1), (513, 256, 2)])
def test_bwd_w_is_the_column_sum(oracle, rows, cols, seed):
    rng = np.random.default_rng(seed)
    X, G = normal_bf16(rng, (rows, cols)), normal_bf16(rng, (rows, cols))
    rms = (0.5 + rng.random(rows)).astype(np.float32)
    start = normal_bf16(rng, (cols,))
    dW = start.copy()
    oracle.oracle_rms_norm_bwd_w(rows, cols, EPS, ptr(rms), ptr(X), ptr(G), ptr(dW))
    want = bf16_to_f64(start) + (bf16_to_f64(G) * bf16_to_f64(X) * rms.astype(np.float64)[:, None]).sum(axis=0)
    assert bf16_ulp_diff(dW, f32_to_bf16(want.astype(np.float32))).max() <= 1
