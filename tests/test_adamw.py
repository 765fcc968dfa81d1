"""AdamW step of the layer's weights: the oracle pinned against the fp64 closed form, the HIP kernel against the
oracle through the C ABI.  Values: one bf16 rounding of the result plus the fp32 rounding of its terms (the moment update can cancel; powf, sqrtf,
the divisions and fused multiply-adds differ by an fp32 rounding between libm / the host compiler and the device)."""
import numpy as np
import pytest

import oracle_lib as O
from util import f32_to_bf16, bf16_to_f64, normal_bf16, bf16_ulp_diff

HP = dict(lr=1e-3, beta1=0.9, beta2=0.999, weight_decay=0.01, epsilon=1e-8)


def near(got_bits, want, scale, rel=2.0 ** -8):
    """one bf16 rounding of the result (2^-8 relative) plus fp32 rounding of the terms it is made of: the moment update
    beta * m + (1 - beta) * g can cancel, and then the fp32 rounding of its terms is what is left"""
    got, want = bf16_to_f64(got_bits), np.asarray(want, dtype=np.float64)
    assert (np.abs(got - want) <= rel * np.abs(want) + 4e-7 * scale).all()


def make(rng, n):
    param, grad, mean = normal_bf16(rng, (n,), 0.05), normal_bf16(rng, (n,), 0.01), normal_bf16(rng, (n,), 0.005)
    var = f32_to_bf16((rng.random(n).astype(np.float32) * 1e-4))
    return param, grad, mean, var


def closed_form(param, grad, mean, var, step, lr, beta1, beta2, weight_decay, epsilon):
    p, g, m, v = (bf16_to_f64(a) for a in (param, grad, mean, var))
    b1, b2 = np.float64(np.float32(beta1)), np.float64(np.float32(beta2))
    lr, wd, eps = (np.float64(np.float32(x)) for x in (lr, weight_decay, epsilon))
    m_t = b1 * m + (1 - b1) * g
    v_t = b2 * v + (1 - b2) * g * g
    m_hat, v_hat = m_t / (1 - b1 ** step), v_t / (1 - b2 ** step)
    return p - lr * (m_hat / (np.sqrt(v_hat) + eps) + wd * p), m_t, v_t


@pytest.mark.parametrize("n,step", [(1, 1), (1000, 1), (4099, 7), (65536, 1000)])
def test_oracle_is_the_closed_form(oracle, n, step):
    rng = np.random.default_rng(n + step)
    param, grad, mean, var = make(rng, n)
    want = closed_form(param, grad, mean, var, step, **HP)
    p, m, v = param.copy(), mean.copy(), var.copy()
    oracle.oracle_adamw_step(n, step, HP["lr"], HP["beta1"], HP["beta2"], HP["weight_decay"], HP["epsilon"], O.ptr(p), O.ptr(grad), O.ptr(m), O.ptr(v))
    scales = (np.abs(bf16_to_f64(param)).max(), max(np.abs(bf16_to_f64(mean)).max(), np.abs(bf16_to_f64(grad)).max()), np.abs(bf16_to_f64(var)).max())
    for got, w, sc in zip((p, m, v), want, scales):
        near(got, w, sc)


def test_oracle_fixed_points(oracle):
    n = 64
    zero = np.zeros(n, np.uint16)
    param = f32_to_bf16(np.linspace(-1, 1, n).astype(np.float32))
    p, m, v = param.copy(), zero.copy(), zero.copy()
    # zero gradient and zero moments: only the decoupled weight decay acts, the moments stay zero
    oracle.oracle_adamw_step(n, 3, 0.5, 0.9, 0.999, 0.25, 1e-8, O.ptr(p), O.ptr(zero), O.ptr(m), O.ptr(v))
    assert (m == 0).all() and (v == 0).all()
    np.testing.assert_allclose(bf16_to_f64(p), bf16_to_f64(param) * (1 - 0.5 * 0.25), rtol=2.0 ** -8)
    # first step from zero moments with no decay: the update is -lr * sign(g) (bias correction cancels beta)
    g = f32_to_bf16(np.where(np.arange(n) % 2, 0.01, -0.02).astype(np.float32))
    p, m, v = param.copy(), zero.copy(), zero.copy()
    oracle.oracle_adamw_step(n, 1, 0.125, 0.9, 0.999, 0.0, 1e-12, O.ptr(p), O.ptr(g), O.ptr(m), O.ptr(v))
    np.testing.assert_allclose(bf16_to_f64(p), bf16_to_f64(param) - 0.125 * np.sign(bf16_to_f64(g)), atol=2.0 ** -8)


@pytest.mark.gpu
@pytest.mark.parametrize("n,step,offset", [(8, 1, 0), (2048, 1, 0), (100003, 5, 0), (1 << 22, 300, 0), (5000, 2, 1)])
def test_gpu_matches_oracle(backend, oracle, n, step, offset):
    """offset 1: arrays that start 2 bytes off a 16-byte boundary take the element-wise path"""
    from ml_dataflow_amd import binding as B
    print("case adamw n=%d step=%d offset=%d" % (n, step, offset), flush=True)
    be = backend
    rng = np.random.default_rng(n)
    param, grad, mean, var = make(rng, n + offset)
    bufs = [be.upload(a) for a in (param, grad, mean, var)]
    ptrs = [b.ptr + 2 * offset for b in bufs]
    BF = B.DATAFLOW_BF16
    assert be.lib.dataflow_submit_default_adamw_step(be.hp, 1, BF, BF, BF, BF, n, step, HP["lr"], HP["beta1"], HP["beta2"], HP["weight_decay"],
                                                     HP["epsilon"], *ptrs) == 0
    be.sync(1)
    p, g, m, v = param[offset:].copy(), grad[offset:].copy(), mean[offset:].copy(), var[offset:].copy()
    oracle.oracle_adamw_step(n, step, HP["lr"], HP["beta1"], HP["beta2"], HP["weight_decay"], HP["epsilon"], O.ptr(p), O.ptr(g), O.ptr(m), O.ptr(v))
    got = [be.read(q, (n,), np.uint16) for q in (ptrs[0], ptrs[2], ptrs[3])]
    scales = (np.abs(bf16_to_f64(param)).max(), max(np.abs(bf16_to_f64(mean)).max(), np.abs(bf16_to_f64(grad)).max()), np.abs(bf16_to_f64(var)).max())
    for g_, w_, sc in zip(got, (p, m, v), scales):
        near(g_, bf16_to_f64(w_), sc, rel=2.0 ** -7)          # two rounded results: one bf16 step apart at most
        assert np.percentile(bf16_ulp_diff(g_, w_), 99.9) <= 1
    assert (be.read(ptrs[1], (n,), np.uint16) == grad[offset:]).all()           # the gradient is read only
    if offset:
        assert be.read(bufs[0].ptr, (1,), np.uint16)[0] == param[0]             # nothing written in front of the arrays
    # step numbers below 1 are rejected
    assert be.lib.dataflow_submit_default_adamw_step(be.hp, 1, BF, BF, BF, BF, n, 0, 1e-3, 0.9, 0.999, 0.0, 1e-8, *ptrs) == -1
