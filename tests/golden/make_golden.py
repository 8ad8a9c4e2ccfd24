"""Writes tests/golden/oracle_vectors.npz: small seeded inputs and the outputs of the CPU oracle.

The reference holds no golden vectors for these kernels (its tests compute expectations at run
time against ONNX Runtime) and cannot be built here, so these vectors freeze the oracle as it
stood when tests/test_oracle.py pinned it.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle  # noqa: E402
from altius_amd import synth  # noqa: E402


def main():
    x = synth.normal(9001, (3, 5, 197), std=1.5)
    y = synth.uniform(9002, (5, 1)) + np.float32(0.5)
    gamma = synth.normal(9003, (197,), mean=1.0, std=0.02)
    beta = synth.normal(9004, (197,), mean=0.0, std=0.02)
    out = {
        "x": x, "y": y, "gamma": gamma, "beta": beta,
        "div": oracle.binary(oracle.DIV, x, y),
        "erf": oracle.unary(oracle.ERF, x),
        "gelu": oracle.unary(oracle.GELU, x),
        "sigmoid": oracle.unary(oracle.SIGMOID, x),
        "hardsigmoid": oracle.unary(oracle.HARDSIGMOID, x, 1.0 / 6.0, 0.5),
        "softmax": oracle.softmax(x),
        "layernorm": oracle.layer_norm(x, gamma, beta, 1e-5),
        "reduce_mean": oracle.reduce(oracle.REDUCE_MEAN, x, [-1], True),
        "reduce_max_axis1": oracle.reduce(oracle.REDUCE_MAX, x, [1], False),
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "oracle_vectors.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
