"""Synthetic inputs of the benchmark workloads: bf16 conversion and the seeded tensors / router bias the
configurations name.  Plain numpy on the host; nothing here touches the device."""
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


def normal_bf16(rng, shape, std=1.0):
    """N(0, std) rounded to bf16 (nearest even), generated in chunks so that large tensors stay within memory"""
    out = np.empty(shape, dtype=np.uint16)
    flat = out.reshape(-1)
    step = 1 << 24
    for lo in range(0, flat.size, step):
        x = rng.standard_normal(min(step, flat.size - lo), dtype=np.float32)
        if std != 1.0:
            x *= np.float32(std)
        b = x.view(np.uint32)
        flat[lo:lo + x.size] = ((b + np.uint32(0x7FFF) + ((b >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
    return out


def zipf_bias(rng, E, scale, s=1.2):
    """per-expert router bias b_e = scale / rank_e**s with a seeded random ranking"""
    ranks = rng.permutation(E) + 1
    return (scale / ranks.astype(np.float64) ** s).astype(np.float32)


# Zipf(s = 1.2) bias scale of the skewed-routing workload (8192 tokens, 32 experts, top-4): the most loaded expert
# receives about 7.7 times the mean number of rows (8 times would be every token)
SKEWED_ROUTING_BIAS_SCALE = 3.0
