"""Pins the oracle's floating-point functions against fp64 closed forms, special cases and finite differences.

Tolerances: outputs are bf16 (8 significant bits), so one rounding is <= 2^-9 relative; the oracle's own
fp32 intermediates add ~1e-7.  Checks are stated in bf16 ulps (2^-7 relative): a correctly rounded result is within 0.5 ulp.
"""
import ctypes as C

import numpy as np
import pytest

import oracle_lib as O
from util import f32_to_bf16, bf16_to_f32, bf16_to_f64, normal_bf16, bf16_ulp_diff

ULP = 2.0 ** -7      # spacing of bf16 numbers relative to the value, at most


def assert_bf16_close(got_bits, want_f64, ulps=1.0, floor=1e-30):
    got = bf16_to_f64(got_bits)
    err = np.abs(got - want_f64)
    tol = ulps * ULP * np.maximum(np.abs(want_f64), floor) + 1e-38
    bad = err > tol
    assert not bad.any(), "max err %g (tol %g) at %s" % (err.max(), tol.ravel()[np.argmax(err)], np.argwhere(bad)[:3])


def test_bf16_round_trip_and_rne(oracle):
    assert oracle.oracle_f32_to_bf16(1.0) == 0x3F80
    # 1 + 2^-8 is exactly half way between 1.0 and the next bf16: ties go to even (1.0)
    assert oracle.oracle_f32_to_bf16(1.0 + 2.0 ** -8) == 0x3F80
    assert oracle.oracle_f32_to_bf16(1.0 + 3 * 2.0 ** -8) == 0x3F82
    rng = np.random.default_rng(0)
    x = rng.standard_normal(1000).astype(np.float32)
    mine = f32_to_bf16(x)
    theirs = np.array([oracle.oracle_f32_to_bf16(float(v)) for v in x], dtype=np.uint16)
    assert (mine == theirs).all()


@pytest.mark.parametrize("transa,transb", [(1, 0), (0, 0), (0, 1), (1, 1)])
@pytest.mark.parametrize("M,K,N", [(16, 24, 8), (33, 7, 5), (1, 64, 3)])
def test_matmul_layouts_against_numpy_fp64(oracle, transa, transb, M, K, N):
    rng = np.random.default_rng(M * 100 + K * 10 + N + transa * 2 + transb)
    A = normal_bf16(rng, (M, K) if transa else (K, M))
    Bm = normal_bf16(rng, (K, N) if transb else (N, K))
    Cin = normal_bf16(rng, (N, M))
    opA = bf16_to_f64(A) if transa else bf16_to_f64(A).T          # [M,K]
    opB = bf16_to_f64(Bm) if transb else bf16_to_f64(Bm).T        # [K,N]
    want = (opA @ opB).T                                          # stored [N][M]
    got = O.matmul(oracle, transa, transb, M, K, N, A, Bm)
    assert_bf16_close(got, want, ulps=0.51, floor=1e-3)
    got2 = O.matmul(oracle, transa, transb, M, K, N, A, Bm, alpha=0.5, beta=2.0, Cin=Cin)
    assert_bf16_close(got2, 0.5 * want + 2.0 * bf16_to_f64(Cin), ulps=0.51, floor=1e-3)


def test_matmul_identity_and_one_hot(oracle):
    rng = np.random.default_rng(3)
    X = normal_bf16(rng, (5, 16))                     # B operand [N][K]
    eye = f32_to_bf16(np.eye(16, dtype=np.float32))    # A operand [M][K] = I
    assert (O.matmul(oracle, 1, 0, 16, 16, 5, eye, X) == X).all()
    onehot = np.zeros((1, 16), dtype=np.float32)
    onehot[0, 7] = 1.0
    col = O.matmul(oracle, 1, 0, 1, 16, 5, f32_to_bf16(onehot), X)
    assert (col[:, 0] == X[:, 7]).all()


def test_matmul_beta_zero_ignores_c_and_zero_rows(oracle):
    rng = np.random.default_rng(4)
    A, Bm = normal_bf16(rng, (8, 8)), normal_bf16(rng, (4, 8))
    nan_c = np.full((4, 8), 0x7FC0, dtype=np.uint16)
    got = O.matmul(oracle, 1, 0, 8, 8, 4, A, Bm, alpha=1.0, beta=0.0, Cin=nan_c)
    assert np.isfinite(bf16_to_f32(got)).all()
    assert O.matmul(oracle, 1, 0, 8, 8, 0, A, Bm[:0]).shape == (0, 8)


def typed_operand(rng, shape, kind, scale=1.0):
    """random operand of an element kind as the oracle takes it (float32 array, or uint16 bit patterns) and its fp64 value"""
    x = (rng.standard_normal(shape) * scale).astype(np.float32)
    if kind == O.ELEM_FP32:
        return x, x.astype(np.float64)
    if kind == O.ELEM_FP16:
        h = x.astype(np.float16)
        return h.view(np.uint16), h.astype(np.float64)
    b = f32_to_bf16(x)
    return b, bf16_to_f64(b)


def typed_value(bits, kind):
    if kind == O.ELEM_FP32:
        return bits.astype(np.float64)
    if kind == O.ELEM_FP16:
        return bits.view(np.float16).astype(np.float64)
    return bf16_to_f64(bits)


@pytest.mark.parametrize("ab,cd", [(O.ELEM_FP32, O.ELEM_FP32), (O.ELEM_FP16, O.ELEM_FP16), (O.ELEM_FP16, O.ELEM_FP32), (O.ELEM_BF16, O.ELEM_FP32)])
@pytest.mark.parametrize("transa,transb", [(1, 0), (0, 0), (0, 1), (1, 1)])
def test_typed_matmul_against_numpy_fp64(oracle, ab, cd, transa, transb):
    """Pins oracle_matmul_typed: numpy's fp64 matmul of the operands' exact values, rounded through fp32 to the output type by
    numpy's own conversions (a library routine for every step), must give the same bits: a transposed operand, a wrong
    leading dimension or a dropped alpha / beta term changes them."""
    M, K, N = 9, 21, 6
    rng = np.random.default_rng(ab * 31 + cd * 7 + transa * 2 + transb)
    A, a64 = typed_operand(rng, (M, K) if transa else (K, M), ab)
    Bm, b64 = typed_operand(rng, (K, N) if transb else (N, K), ab)
    Cin, c64 = typed_operand(rng, (N, M), cd)
    opA = a64 if transa else a64.T
    opB = b64 if transb else b64.T
    want = (opA @ opB).T

    def rounded(v):
        v32 = v.astype(np.float32)
        return v32 if cd == O.ELEM_FP32 else v32.astype(np.float16).view(np.uint16)

    got = O.matmul_typed(oracle, ab, cd, transa, transb, M, K, N, A, Bm)
    assert (got == rounded(want)).all()
    got2 = O.matmul_typed(oracle, ab, cd, transa, transb, M, K, N, A, Bm, alpha=0.5, beta=2.0, Cin=Cin)
    assert (got2 == rounded(0.5 * want + 2.0 * c64)).all()
    # the identity as A returns B's values in the output type
    eye = np.eye(K, dtype=np.float32)
    eye = eye if ab == O.ELEM_FP32 else (eye.astype(np.float16).view(np.uint16) if ab == O.ELEM_FP16 else f32_to_bf16(eye))
    Xb, x64 = typed_operand(rng, (N, K), ab)
    assert (O.matmul_typed(oracle, ab, cd, 1, 0, K, K, N, eye, Xb) == rounded(x64)).all()
    assert oracle.oracle_matmul_typed(7, 0, 1, 0, 1, 1, 1, 1.0, 0.0, None, None, None, None) == -1


def test_swiglu_forward_closed_form(oracle):
    rng = np.random.default_rng(5)
    x1, x3 = normal_bf16(rng, (7, 64), 3.0), normal_bf16(rng, (7, 64), 2.0)
    out = np.zeros_like(x1)
    oracle.oracle_swiglu(7, 64, O.ptr(x1), O.ptr(x3), O.ptr(out))
    a, b = bf16_to_f64(x1), bf16_to_f64(x3)
    assert_bf16_close(out, a / (1 + np.exp(-a)) * b, ulps=0.52)
    # aliasing: out may be x1
    x1c = x1.copy()
    oracle.oracle_swiglu(7, 64, O.ptr(x1c), O.ptr(x3), O.ptr(x1c))
    assert (x1c == out).all()


def test_swiglu_backward_closed_form_and_finite_difference(oracle):
    rng = np.random.default_rng(6)
    x1, x3, g = normal_bf16(rng, (4, 32), 2.0), normal_bf16(rng, (4, 32), 2.0), normal_bf16(rng, (4, 32))
    d1, d3 = np.zeros_like(x1), np.zeros_like(x1)
    oracle.oracle_swiglu_bwd_x(4, 32, O.ptr(x1), O.ptr(x3), O.ptr(g), O.ptr(d1), O.ptr(d3))
    a, b, gg = bf16_to_f64(x1), bf16_to_f64(x3), bf16_to_f64(g)
    f = lambda a_, b_: a_ / (1 + np.exp(-a_)) * b_
    eps = 1e-6
    fd1 = gg * (f(a + eps, b) - f(a - eps, b)) / (2 * eps)
    fd3 = gg * (f(a, b + eps) - f(a, b - eps)) / (2 * eps)
    assert_bf16_close(d1, fd1, ulps=0.6, floor=1e-4)
    assert_bf16_close(d3, fd3, ulps=0.6, floor=1e-4)


def test_fp16_conversions_equal_numpy(oracle):
    """every one of the 65536 half patterns widens like numpy's float16; rounding to half equals numpy's (nearest even)
    on random values, on the ties between neighbouring halves, around the overflow threshold and among subnormals"""
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([oracle.oracle_fp16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert (np.isnan(got) == nan).all() and (got[~nan].view(np.uint32) == want[~nan].view(np.uint32)).all()
    rng = np.random.default_rng(3)
    finite = bits[(bits & 0x7C00) != 0x7C00]
    lo = finite.view(np.float16).astype(np.float64)
    with np.errstate(over="ignore"):
        hi = np.nextafter(finite.view(np.float16), np.float16(np.inf)).astype(np.float64)
    ties = ((lo + hi) / 2)[np.isfinite(hi)].astype(np.float32)          # exactly representable in fp32
    samples = np.concatenate([
        (rng.standard_normal(20000) * 10 ** rng.uniform(-9, 5, 20000)).astype(np.float32), ties,
        np.nextafter(ties, np.float32(np.inf)), np.nextafter(ties, np.float32(-np.inf)),
        np.array([65504.0, 65519.996, 65520.0, 65536.0, 1e9, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26, 0.0, -0.0,
                  np.inf, -np.inf], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want16 = samples.astype(np.float16).view(np.uint16)
    got16 = np.array([oracle.oracle_f32_to_fp16(float(v)) for v in samples], dtype=np.uint16)
    assert (got16 == want16).all(), samples[got16 != want16][:5]


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_swiglu_fp32_fp16_closed_form_and_finite_difference(oracle, dtype):
    rng = np.random.default_rng(8)
    x1 = (rng.standard_normal((5, 64)) * 3).astype(dtype)
    x3 = (rng.standard_normal((5, 64)) * 2).astype(dtype)
    g = rng.standard_normal((5, 64)).astype(dtype)
    a, b, gg = x1.astype(np.float64), x3.astype(np.float64), g.astype(np.float64)
    f = lambda a_, b_: a_ / (1 + np.exp(-a_)) * b_
    ulp = 2.0 ** -24 if dtype == np.float32 else 2.0 ** -11                  # half a step of the element type, relative
    out = O.swiglu_typed(oracle, x1, x3)
    want = f(a, b)
    assert (np.abs(out.astype(np.float64) - want) <= 4 * ulp * np.abs(want) + 1e-7).all()
    d1, d3 = O.swiglu_bwd_x_typed(oracle, x1, x3, g)
    s = 1 / (1 + np.exp(-a))
    want1, want3 = gg * b * (s + a * s * (1 - s)), gg * a * s
    assert (np.abs(d1.astype(np.float64) - want1) <= 6 * ulp * np.abs(want1) + 1e-6).all()
    assert (np.abs(d3.astype(np.float64) - want3) <= 6 * ulp * np.abs(want3) + 1e-6).all()
    eps = 1e-6                                                               # and the closed form is the derivative
    np.testing.assert_allclose(want1, gg * (f(a + eps, b) - f(a - eps, b)) / (2 * eps), rtol=1e-5, atol=1e-7)
    np.testing.assert_allclose(want3, gg * (f(a, b + eps) - f(a, b - eps)) / (2 * eps), rtol=1e-5, atol=1e-7)
    if dtype == np.float16:
        # one rounding to half at the end: the fp32 value of the same expression, rounded by numpy, is the result
        o32 = O.swiglu_typed(oracle, x1.astype(np.float32), x3.astype(np.float32))
        assert (o32.astype(np.float16).view(np.uint16) == out.view(np.uint16)).all()


def make_routing(rng, T, E, K):
    chosen = np.stack([rng.permutation(E)[:K] for _ in range(T)]).astype(np.uint16)
    bc = np.bincount(chosen.ravel(), minlength=E)
    order = np.argsort(chosen.ravel(), kind="stable")
    tmap = np.empty(T * K, dtype=np.int32)
    tmap[order] = np.arange(T * K, dtype=np.int32)
    emap = (order // K).astype(np.int32)
    return chosen, bc.astype(np.int32), np.cumsum(bc).astype(np.int32), emap, tmap.reshape(T, K)


def test_dispatch_is_a_pure_copy(oracle):
    rng = np.random.default_rng(7)
    T, D, E, K = 50, 24, 8, 3
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    X = normal_bf16(rng, (T, D))
    zones = np.zeros((T * K, D), dtype=np.uint16)
    oracle.oracle_prepare_experts(T, D, K, O.ptr(X), O.ptr(tmap), O.ptr(zones))
    assert (zones == X[emap]).all()
    for e in (0, 3, 7):
        z = np.zeros((counts[e], D), dtype=np.uint16)
        oracle.oracle_prepare_expert_zone(D, O.ptr(X), e, O.ptr(counts), O.ptr(incl), O.ptr(emap), O.ptr(z))
        assert (z == zones[incl[e] - counts[e]:incl[e]]).all()


def test_combine_equals_dense_one_hot_matmul(oracle):
    rng = np.random.default_rng(8)
    T, D, E, K = 40, 16, 6, 2
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    zones = normal_bf16(rng, (T * K, D))
    w = rng.random((T, K)).astype(np.float32)
    resid = normal_bf16(rng, (T, D))
    out = resid.copy()
    oracle.oracle_merge_experts(T, D, K, O.ptr(zones), O.ptr(tmap), O.ptr(w), O.ptr(out))
    S = np.zeros((T, T * K))
    for t in range(T):
        for k in range(K):
            S[t, tmap[t, k]] = w[t, k]
    want = bf16_to_f64(resid) + S @ bf16_to_f64(zones)
    assert_bf16_close(out, want, ulps=0.55, floor=1e-3)
    # w == NULL: plain index-add
    out2 = np.zeros((T, D), dtype=np.uint16)
    oracle.oracle_merge_experts(T, D, K, O.ptr(zones), O.ptr(tmap), None, O.ptr(out2))
    want2 = np.zeros((T, D))
    np.add.at(want2, emap, bf16_to_f64(zones))
    assert_bf16_close(out2, want2, ulps=0.55, floor=1e-3)


def test_per_expert_combine_accumulates_like_the_fused_one_up_to_rounding(oracle):
    rng = np.random.default_rng(9)
    T, D, E, K = 30, 16, 5, 2
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    zones = normal_bf16(rng, (T * K, D))
    w = (rng.random((T, K)) + 0.1).astype(np.float32)
    out = np.zeros((T, D), dtype=np.uint16)
    for e in range(E):
        z = zones[incl[e] - counts[e]:incl[e]]
        oracle.oracle_merge_expert_result(int(counts[e]), D, K, O.ptr(np.ascontiguousarray(z)), e, O.ptr(incl), O.ptr(emap),
                                          O.ptr(w), O.ptr(chosen), O.ptr(out))
    want = np.zeros((T, D))
    mag = np.zeros((T, D))
    for t in range(T):
        for k in range(K):
            want[t] += w[t, k] * bf16_to_f64(zones[tmap[t, k]])
            mag[t] += np.abs(w[t, k] * bf16_to_f64(zones[tmap[t, k]]))
    # K roundings to bf16 (one per expert pass) instead of one, each relative to a partial sum <= mag
    assert (np.abs(bf16_to_f64(out) - want) <= (0.5 * K + 0.1) * ULP * mag + 1e-30).all()


def test_router_bwd_x_identities(oracle):
    rng = np.random.default_rng(10)
    T, D, E, K = 25, 32, 6, 3
    chosen, counts, incl, emap, tmap = make_routing(rng, T, E, K)
    y = normal_bf16(rng, (T * K, D))
    dY = normal_bf16(rng, (T, D))
    w = (rng.random((T, K)) + 0.05).astype(np.float32)
    dlog = np.zeros((T, E), dtype=np.uint16)
    zones = y.copy()
    for e in range(E):
        seg = zones[incl[e] - counts[e]:incl[e]]       # a view: in/out alias like the reference's call
        oracle.oracle_router_bwd_x(int(counts[e]), D, E, K, e, O.ptr(incl), O.ptr(emap), O.ptr(chosen), O.ptr(w),
                                   seg.ctypes.data, O.ptr(dY), O.ptr(dlog), seg.ctypes.data)
    yf, gf = bf16_to_f64(y), bf16_to_f64(dY)
    want_dlog = np.zeros((T, E))
    for t in range(T):
        for k in range(K):
            want_dlog[t, chosen[t, k]] = yf[tmap[t, k]] @ gf[t]
    assert_bf16_close(dlog, want_dlog, ulps=0.52, floor=1e-2)
    # scaled rows: bf16(dY * bf16(w)), exactly one rounding of an exact product
    for t in range(T):
        for k in range(K):
            wb = bf16_to_f32(f32_to_bf16(np.array([w[t, k]], dtype=np.float32)))[0]
            want_row = f32_to_bf16(bf16_to_f32(dY[t]) * wb)
            assert (zones[tmap[t, k]] == want_row).all()


def test_router_gate_bwd_is_softmax_jacobian(oracle):
    rng = np.random.default_rng(12)
    T, E, K = 20, 10, 4
    chosen, *_ = make_routing(rng, T, E, K)
    logits_sel = rng.standard_normal((T, K))
    p = np.exp(logits_sel - logits_sel.max(1, keepdims=True))
    p = (p / p.sum(1, keepdims=True)).astype(np.float32)
    d_full = np.zeros((T, E), dtype=np.float32)
    up = rng.standard_normal((T, K)).astype(np.float32)
    np.put_along_axis(d_full, chosen.astype(np.int64), up, axis=1)
    d_bits = f32_to_bf16(d_full)
    before = bf16_to_f64(d_bits)
    oracle.oracle_router_gate_bwd_x(T, E, K, O.ptr(chosen), O.ptr(p), O.ptr(d_bits))
    upb = np.take_along_axis(before, chosen.astype(np.int64), axis=1)
    # dL/dlogit_i = sum_j dL/dp_j * dp_j/dlogit_i with the softmax Jacobian diag(p) - p p^T
    pj = p.astype(np.float64)
    jac = np.einsum("tk,kj->tkj", pj, np.eye(K)) - np.einsum("tk,tj->tkj", pj, pj)
    want_sel = np.einsum("tj,tjk->tk", upb, jac)
    want = np.zeros((T, E))
    np.put_along_axis(want, chosen.astype(np.int64), want_sel, axis=1)
    assert_bf16_close(d_bits, want, ulps=0.6, floor=1e-2)
    mask = np.ones((T, E), dtype=bool)
    np.put_along_axis(mask, chosen.astype(np.int64), False, axis=1)
    assert (d_bits[mask] == 0).all()
