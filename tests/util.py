"""Shared helpers for the test-suite: bf16 <-> numpy, seeded synthetic tensors, error metrics."""
import numpy as np

from ml_dataflow_amd.synthetic import f32_to_bf16, bf16_to_f32, normal_bf16, zipf_bias, SKEWED_ROUTING_BIAS_SCALE  # noqa: F401


def bf16_to_f64(b):
    return bf16_to_f32(b).astype(np.float64)


def max_rel_err(got, want, floor):
    """max |got - want| / max(|want|, floor): elementwise relative error with an absolute floor for tiny targets."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float(np.max(np.abs(got - want) / np.maximum(np.abs(want), floor))) if got.size else 0.0


def bf16_ulp_diff(a_bits, b_bits):
    """distance in bf16 representable steps between two bf16 arrays (finite values)."""
    def key(u):
        u = u.astype(np.int32)
        return np.where(u & 0x8000, 0x8000 - u, u)
    return np.abs(key(np.asarray(a_bits, dtype=np.uint16)) - key(np.asarray(b_bits, dtype=np.uint16)))


def close(got_bits, want_bits, tol=1e-2, steps=2, what=""):
    """The value bar of the parity tests for bf16 arrays given as bit patterns.  With rms the root mean square of the
    expected tensor (the magnitude of its typical element and of the rounded intermediates it is summed from) and a
    bf16 step being 2^-8 of a value's magnitude (0.4 to 0.8 % relative):
      (a) every element:                   |got - want| <= tol * max|want|               (the stated 1e-2 tolerance)
      (b) every element:                   |got - want| <= steps * 2^-8 * (|want| + 2 rms)
      (c) every element with |want| >= rms: got is at most `steps` representable bf16 values away from want
    steps=None asks for (a) only.  (b) and (c) are element-wise: an entry that is wrong while the tensor's largest entries are right fails them.  (c)
    is not asked of entries far below rms: those are differences of larger rounded terms, and one rounding step of
    such a term (fp32 against the oracle's fp64 accumulation) moves them by many of their own steps; (b) bounds them
    by the step of the terms instead."""
    got_bits, want_bits = np.asarray(got_bits, dtype=np.uint16), np.asarray(want_bits, dtype=np.uint16)
    assert got_bits.shape == want_bits.shape, "%s: shape %s vs %s" % (what, got_bits.shape, want_bits.shape)
    if got_bits.size == 0:
        return
    g, w = bf16_to_f64(got_bits), bf16_to_f64(want_bits)
    aw = np.abs(w)
    scale = max(float(aw.max()), 1e-30)
    rms = max(float(np.sqrt(np.mean(w * w))), 1e-30)
    err = np.abs(g - w)
    assert float(err.max()) <= tol * scale, "%s: max err %g vs scale %g" % (what, float(err.max()), scale)
    if steps is None:
        return
    ratio = float((err / (aw + 2.0 * rms)).max()) * 256.0
    assert ratio <= steps, "%s: an element is %.2f steps (of |want| + 2 rms) off, allowed %d" % (what, ratio, steps)
    worst = int(bf16_ulp_diff(got_bits, want_bits)[aw >= rms].max(initial=0))
    assert worst <= steps, "%s: %d bf16 steps apart on an element of at least rms magnitude (allowed %d)" % (what, worst, steps)
