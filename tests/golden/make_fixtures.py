"""Writes tests/golden/ring_fixtures.npz: seeded inputs and fp64 expected outputs of the time loop.

The reference holds no golden vectors for this path, so these are REGRESSION fixtures: inputs from a seeded numpy
generator, expected values from the fp64 oracle (oracle/ring_oracle.py), which the tests in tests/test_oracle_*.py
pin by closed forms, brute force and autograd.  They freeze today's numbers so that a later change of the oracle or
of a kernel shows up as a diff against a committed file.  Shapes: the reference's own tiny self-test shape
(legacy/bwd_fp32.py:553-576: N=8, a_dim=4, T=10, B=4, tanh) and a ragged two-channel case for every activation.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import ring_oracle as O  # noqa: E402

CASES = {  # name: (seed, B, T, k, N, activation, J0, J1)
    "tiny_tanh": (11, 4, 10, 4, 8, "tanh", -0.1, 0.1),
    "ragged_relu": (12, 5, 7, 2, 24, "relu", 0.02, 0.6),
    "ragged_gelu": (13, 5, 7, 2, 24, "gelu", -0.1, 0.5),
    "ragged_silu": (14, 5, 7, 2, 24, "silu", -0.1, 0.5),
}


def build(seed, B, T, k, N, act, J0, J1):
    rng = np.random.default_rng(seed)
    Wo = (rng.standard_normal((N, N)) / np.sqrt(N)).astype(np.float32)
    Wa = (rng.standard_normal((k, N, N)) / np.sqrt(N)).astype(np.float32)
    A = (rng.random((B, T, k)) * 0.3).astype(np.float32)
    r0 = O.create_initial_bump(rng.random(B) * 2 * np.pi, N).astype(np.float32)
    G = rng.standard_normal((T, B, N)).astype(np.float32)
    hist, _ = O.forward_dense(A, Wa, J0, J1, Wo, r0, 0.15, act)
    g = O.backward_dense(G, A, Wa, J0, J1, Wo, hist, r0, 0.15, act)
    return dict(A=A, Wa=Wa, Wo=Wo, r0=r0, G=G, J=np.array([J0, J1]), hist=hist, grad_Wo=g["grad_Wo"],
                grad_Wa=g["grad_Wa"], grad_A=g["grad_A"], grad_r_init=g["grad_r_init"])


if __name__ == "__main__":
    out = {}
    for name, cfg in CASES.items():
        for key, val in build(*cfg).items():
            out[f"{name}/{key}"] = val
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ring_fixtures.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes")
