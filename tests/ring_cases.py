"""Seeded synthetic problems shared by the GPU parity tests, the smoke check and the benchmark.
Input recipe: weights ~ N(0, 1/N); angular velocity from the oracle's generator (10 % leading zeros,
U(-0.1*pi, 0.1*pi), per-trial zero ratio), L = relu(-av), R = relu(av); Gaussian initial bump at the
trial's initial angle."""
import math

import numpy as np

from oracle import ring_oracle as O


def perfect_weights(N, k):
    """The reference's 'perfect' initialisation (train_general_ring_no_gain.py:56-74, root script):
    Wo = cos(d); k == 2: Wl/Wr = cos(d +- pi/4); otherwise cos(d + 2*pi*c/k)."""
    idx = np.arange(N, dtype=np.float64)
    d = 2 * np.pi * (idx[:, None] - idx[None, :]) / N
    if k == 2:
        Wa = np.stack([np.cos(d + np.pi / 4), np.cos(d - np.pi / 4)])
    else:
        Wa = np.stack([np.cos(d + c * 2 * np.pi / k) for c in range(k)])
    return np.cos(d).astype(np.float32), Wa.astype(np.float32)


def make_problem(seed, B, T, k, N, zero_ratios=(0.2, 0.5, 0.8), action="lr", bump="gauss", weights="random"):
    rng = np.random.default_rng(seed)
    Wo = (rng.standard_normal((N, N)) / math.sqrt(N)).astype(np.float32)
    Wa = (rng.standard_normal((k, N, N)) / math.sqrt(N)).astype(np.float32)
    if weights == "perfect":
        Wo, Wa = perfect_weights(N, k)
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
