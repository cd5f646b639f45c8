"""Seeded synthetic problems shared by the GPU parity tests, the smoke check and the benchmark.
Input recipe: weights ~ N(0, 1/N); angular velocity from the oracle's generator (10 % leading zeros,
U(-0.1*pi, 0.1*pi), per-trial zero ratio), L = relu(-av), R = relu(av); Gaussian initial bump at the
trial's initial angle."""
import math

import numpy as np

from oracle import ring_oracle as O


def make_problem(seed, B, T, k, N, zero_ratios=(0.2, 0.5, 0.8), action="lr", bump="gauss"):
    rng = np.random.default_rng(seed)
    Wo = (rng.standard_normal((N, N)) / math.sqrt(N)).astype(np.float32)
    Wa = (rng.standard_normal((k, N, N)) / math.sqrt(N)).astype(np.float32)
    av, angle = O.generate_av_integration_data(B, T, rng, zero_ratios_in_rest=zero_ratios)
    if action == "lr":
        A = O.av_to_action_signal_nd(av, k, zero_padding=True) if k >= 2 else np.maximum(av, 0.0)[..., None]
    elif action == "spread":
        A = O.av_to_action_signal_nd(av, k, zero_padding=False)
    else:  # dense random gates exercise every action matrix
        A = rng.random((B, T, k)) * 0.3
    r0 = (O.create_initial_bump if bump == "gauss" else O.von_mises_bump)(angle[:, 0], N)
    G = rng.standard_normal((T, B, N)).astype(np.float32)
    return dict(A=A.astype(np.float32), Wa=Wa, Wo=Wo, r0=r0.astype(np.float32), G=G,
                angle=angle.astype(np.float32), av=av.astype(np.float32))
