"""Shared helpers for the test-suite: bf16 <-> numpy, seeded synthetic tensors, error metrics."""
import numpy as np


def f32_to_bf16(x):
    """float32 array -> uint16 bf16 bits, round to nearest even (NaN kept quiet)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    nan = (bits & 0x7FFFFFFF) > 0x7F800000
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) >> 16
    rounded = np.where(nan, (bits >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def bf16_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def bf16_to_f64(b):
    return bf16_to_f32(b).astype(np.float64)


def normal_bf16(rng, shape, std=1.0):
    return f32_to_bf16((rng.standard_normal(shape, dtype=np.float32) * np.float32(std)))


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


def zipf_bias(rng, E, scale, s=1.2):
    """per-expert router bias b_e = scale / rank_e**s with a seeded random ranking"""
    ranks = rng.permutation(E) + 1
    return (scale / ranks.astype(np.float64) ** s).astype(np.float32)
