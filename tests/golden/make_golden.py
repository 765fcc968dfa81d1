#!/usr/bin/env python3
"""Writes the golden fixtures of the MoE layer: seeded inputs and the outputs of the C oracle for them.

The reference holds no known-answer vectors for this path (its correctness checks compare dumps of a CUDA run
with a PyTorch model at run time), so the fixtures are produced by this repository's oracle, whose functions are
pinned separately against closed forms, library routines and brute force.  The fixtures freeze those results:
a later change of the oracle or of the GPU path that alters any integer output, or moves a value by more than
rounding, fails the fixture tests.

    python3 tests/golden/make_golden.py        (needs oracle/libmoe_oracle.so: make -C oracle)

Every case is checked to have a routing margin: the K-th and (K+1)-th largest logit of every token differ by
more than 4 bf16 steps, so a one-step difference in the router product cannot change the selection and the GPU
path must reproduce the integer outputs exactly.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.join(os.path.dirname(os.path.dirname(HERE)), "oracle"))
import oracle_lib as O                                             # noqa: E402
from util import normal_bf16, bf16_to_f32, bf16_ulp_diff           # noqa: E402

CASES = [   # name, T, D, E, K, H, seed
    ("moe_T64_D32_E8_K2_H64", 64, 32, 8, 2, 64, 1234),
    ("moe_T48_D64_E12_K4_H24", 48, 64, 12, 4, 24, 4321),
]


def generate(lib, T, D, E, K, H, seed):
    while True:
        rng = np.random.default_rng(seed)
        Wr = normal_bf16(rng, (E, D), 0.5)
        W1, W3, W2 = normal_bf16(rng, (E, H, D), 0.1), normal_bf16(rng, (E, H, D), 0.1), normal_bf16(rng, (E, D, H), 0.1)
        X, resid, dY = normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D)), normal_bf16(rng, (T, D))
        ol = O.Layer(lib, T, D, E, K, H, Wr, W1, W3, W2)
        out = ol.forward(X, resid)
        srt = np.sort(bf16_to_f32(ol.logits), axis=1)[:, ::-1]
        from util import f32_to_bf16
        margin = bf16_ulp_diff(f32_to_bf16(srt[:, K - 1]), f32_to_bf16(srt[:, K])).min()
        if margin > 4:
            break
        seed += 1                                                  # a near tie: try the next seed
    dX = ol.backward(X, dY)
    return dict(seed=np.int64(seed), Wr=Wr, W1=W1, W3=W3, W2=W2, X=X, residual=resid, dY=dY,
                logits=ol.logits.copy(), weights=ol.weights.copy(), chosen=ol.chosen.copy(), counts=ol.counts[:E].copy(),
                cumsum_inclusive=ol.cumsum.copy(), expert_mapping=ol.expert_mapping.copy(), token_mapping=ol.token_mapping.copy(),
                x1=ol.x1.copy(), x3=ol.x3.copy(), out=out, dX=dX, dx1=ol.dx1.copy(), dx3=ol.dx3.copy(), dlogits=ol.dlogits.copy(),
                dWr=ol.dWr.copy(), dW1=ol.dW1.copy(), dW3=ol.dW3.copy(), dW2=ol.dW2.copy())


def main():
    lib = O.load()
    for name, T, D, E, K, H, seed in CASES:
        data = generate(lib, T, D, E, K, H, seed)
        path = os.path.join(HERE, name + ".npz")
        np.savez_compressed(path, **data)
        print(path, os.path.getsize(path), "bytes, seed", int(data["seed"]))


if __name__ == "__main__":
    main()
