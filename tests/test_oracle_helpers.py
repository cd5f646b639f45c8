"""Pins the oracle's read-out, losses, decoders, initial bumps and input generator with closed
forms and structural invariants, and the torch twins used for loss-head gradients."""
import math

import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from oracle import torch_port as TP


def test_w_delta7_closed_form():
    N = 12
    W = O.w_delta7(N)
    for i, j in [(0, 0), (3, 1), (1, 3), (11, 0), (5, 11)]:
        assert abs(W[i, j] - math.cos(2 * math.pi * (i - j) / N)) < 1e-15
    np.testing.assert_allclose(W, W.T, atol=1e-15)             # cos is even
    np.testing.assert_allclose(np.roll(np.roll(W, 1, 0), 1, 1), W, atol=1e-15)   # circulant
    np.testing.assert_allclose(TP.w_delta7(N, torch.float64).numpy(), W, atol=1e-15)


def test_readout_of_cosine_bump_is_unit_peak_cosine():
    N = 64
    theta = 2 * np.pi * np.arange(N) / N
    bump = 0.3 + np.cos(theta - 1.0)[None, :]
    out = O.readout(bump)
    # the constant is annihilated by the zero-mean cosine filter; the result is a cosine with max 1
    assert abs(out.max() - 1.0) < 1e-12
    k = int(np.argmax(out[0]))
    assert abs(theta[k] - 1.0) < 2 * np.pi / N
    np.testing.assert_allclose(TP.readout(torch.tensor(bump)).numpy(), out, atol=1e-12)


def test_initial_bump_is_unit_norm_centred_and_circular():
    N = 120
    ang = np.array([0.0, math.pi, 2 * math.pi * 117.0 / N])
    b = O.create_initial_bump(ang, N)
    np.testing.assert_allclose(np.linalg.norm(b, axis=1), 1.0, rtol=1e-14)
    assert np.argmax(b[0]) == 0 and np.argmax(b[1]) == 60 and np.argmax(b[2]) == 117
    # closed form of one entry: centre 60, index 48 -> distance 12 = sigma
    raw = math.exp(-(12.0 ** 2) / (2 * 12.0 ** 2))
    assert abs(b[1, 48] / b[1, 60] - raw) < 1e-14
    # wrap-around: neurons 1 and N-1 are both at distance 1 from centre 0
    assert abs(b[0, 1] - b[0, N - 1]) < 1e-15
    v = O.von_mises_bump(ang, N, 4.0)
    np.testing.assert_allclose(np.linalg.norm(v, axis=1), 1.0, rtol=1e-14)
    assert np.argmax(v[1]) == 60
    assert abs(v[1, 30] / v[1, 60] - math.exp(4.0 * (math.cos(math.pi / 2) - 1))) < 1e-13


def test_population_vector_decodes_cosine_bump_and_wraps():
    N = 360
    pa = O.preferred_angles(N)
    assert pa[0] == 0.0 and abs(pa[-1] - 2 * np.pi) < 1e-15           # end point included
    for theta0 in [0.5, 3.0, 6.0]:
        act = np.cos(pa - theta0)[None, None, :]
        dec = O.decode_angle_from_population_vector(act)
        assert abs(dec[0, 0] - theta0) < 2e-2                         # end-point skew only
        assert 0 <= dec[0, 0] < 2 * np.pi
    onehot = np.zeros((1, 1, N))
    onehot[0, 0, 90] = 1.0
    assert O.decode_angle_from_argmax(onehot)[0, 0] == pa[90]


def test_cosine_similarity_loss_closed_forms():
    N = 360
    pa = O.preferred_angles(N)
    wave = np.cos(pa - 1.2)[None, None, :]
    dec = O.decode_angle_from_population_vector(wave)
    assert O.cosine_similarity_loss(wave, dec) < 1e-28                 # decoded == true => 0
    # opposite direction: |u - (-u)|^2 = 4
    assert abs(O.cosine_similarity_loss(wave, dec + np.pi) - 4.0) < 1e-12
    # quarter turn: |u - v|^2 = 2
    assert abs(O.cosine_similarity_loss(wave, dec + np.pi / 2) - 2.0) < 1e-12
    assert abs(float(TP.cosine_similarity_loss(torch.tensor(wave), torch.tensor(dec + 0.3)))
               - O.cosine_similarity_loss(wave, dec + 0.3)) < 1e-13


def test_bump_amplitude_loss_closed_forms():
    bump = np.ones((2, 3, 4))
    assert O.bump_amplitude_loss(bump) == 0.0
    bump[:, 1, :] = -2.0       # L1 mass 8 vs 4 at step 0 -> deviation 4 on one of three steps
    assert abs(O.bump_amplitude_loss(bump) - 16.0 / 3.0) < 1e-14
    assert abs(O.bump_amplitude_loss(bump, target_amplitude=8.0) - 2 * 16.0 / 3.0) < 1e-14
    assert abs(float(TP.bump_amplitude_loss(torch.tensor(bump))) - 16.0 / 3.0) < 1e-14


def test_perfect_weights_integrate_angle_sanity():
    """debug_perfect recipe (train/train_ring_attractor.py:327-348): cos(d), cos(d +- pi/4), N=360, gelu,
    gains bypassed => cosine loss < 0.5."""
    N, B, T = 360, 4, 60
    rng = np.random.default_rng(0)
    idx = np.arange(N, dtype=np.float64)
    d = 2 * np.pi * (idx[:, None] - idx[None, :]) / N
    Wo, Wl, Wr = np.cos(d), np.cos(d + np.pi / 4), np.cos(d - np.pi / 4)
    av, angle = O.generate_av_integration_data(B, T, rng)
    A = O.av_to_action_signal(av)
    r0 = O.create_initial_bump(angle[:, 0], N)
    hist, _ = O.forward_dense(A, np.stack([Wl, Wr]), -0.1, 0.1, Wo, r0, 0.15, "gelu")
    wave = O.readout(hist.transpose(1, 0, 2))
    assert O.cosine_similarity_loss(wave, angle) < 0.5


def test_av_generator_structure():
    rng = np.random.default_rng(5)
    B, T = 64, 120
    av, angle = O.generate_av_integration_data(B, T, rng)
    n0 = int(T * 0.1)
    rest = T - n0
    assert (av[:, :n0] == 0).all()
    assert np.abs(av).max() <= 0.1 * np.pi
    nz = (av[:, n0:] != 0).sum(axis=1)
    allowed = {rest - int(np.float32(rest) * np.float32(z)) for z in (0.2, 0.5, 0.8)}
    assert set(nz.tolist()) <= allowed and len(set(nz.tolist())) > 1
    assert ((angle >= 0) & (angle < 2 * np.pi)).all()
    np.testing.assert_allclose(angle[:, 1:], (angle[:, :1] + np.cumsum(av[:, :-1], axis=1)) % (2 * np.pi), atol=1e-12)
    A = O.av_to_action_signal(av)
    assert A.shape == (B, T, 2) and (A >= 0).all() and (A[..., 0] * A[..., 1] == 0).all()
    np.testing.assert_array_equal(A[..., 1] - A[..., 0], av)
    A16 = O.av_to_action_signal_nd(av, 16, zero_padding=True)
    np.testing.assert_array_equal(A16[..., :2], A)
    assert (A16[..., 2:] == 0).all()
    sc = O.av_to_action_signal_nd(av, 5, zero_padding=False)
    np.testing.assert_allclose(sc[..., 4], np.maximum(av, 0.0))
    np.testing.assert_allclose(sc[..., 0], np.maximum(-av, 0.0))
    assert (sc[..., 2] == 0).all()


def test_comparison_helpers():
    a = np.array([1.0, 2.0, 3.0])
    assert abs(O.cosine(a, 2 * a) - 1.0) < 1e-15
    assert abs(O.cosine(a, -a) + 1.0) < 1e-15
    assert abs(O.max_rel_err(a + np.array([0, 0, 0.3]), a) - 0.1) < 1e-15


def test_rank_two_loss_head_matches_the_literal_chain_and_its_autograd():
    """loss_pair_rank2 (what the fused loss kernels implement) against the reference's chain of tensor ops:
    read-out through W_delta7, max normalisation, atan2 decode, both losses, and torch autograd of all that."""
    import torch
    from oracle import torch_port as TP
    rng = np.random.default_rng(5)
    for (T, B, N, own) in [(6, 5, 24, True), (4, 3, 33, False), (3, 2, 256, True)]:
        angle = rng.random((B, T)) * 2 * np.pi
        centre = rng.random((T, B)) * 2 * np.pi
        idx = np.arange(N)
        bump = 0.3 * np.exp(2.0 * (np.cos(2 * np.pi * idx / N - centre[..., None]) - 1.0)) + 0.02 * rng.standard_normal((T, B, N))
        tgt = None if own else rng.random(B) + 1.0
        total, lc, la, grad = O.loss_pair_rank2(bump, angle, 0.2, tgt)
        h = torch.tensor(bump, dtype=torch.float64, requires_grad=True)
        ref = TP.loss_pair(h, torch.tensor(angle), 0.2, None if own else torch.tensor(tgt).reshape(B, 1))
        ref.backward()
        assert abs(total - float(ref)) <= 1e-10 * max(1.0, abs(float(ref)))
        np.testing.assert_allclose(grad, h.grad.numpy(), rtol=0, atol=1e-9 * np.abs(h.grad.numpy()).max() + 1e-14)
        # the parts
        b = np.transpose(bump, (1, 0, 2))
        assert abs(lc - O.cosine_similarity_loss(O.readout(b), angle)) <= 1e-10
        assert abs(la - O.bump_amplitude_loss(b, None if own else tgt.reshape(B, 1))) <= 1e-10
