"""Pins the oracle's manual BPTT: independent torch autograd, fp64 gradcheck at the reference's own
tiny shape (legacy/bwd_fp32.py:553-576), central finite differences for the two gradients the
reference never produces (grad_A, grad_r_init), and dense == per-sample."""
import math

import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from oracle import torch_port as TP

ACTS = ["relu", "gelu", "tanh", "silu"]


def _problem(seed, B, T, k, N):
    rng = np.random.default_rng(seed)
    A = rng.random((B, T, k)) * 0.4
    Wa = rng.standard_normal((k, N, N)) / math.sqrt(N)
    Wo = rng.standard_normal((N, N)) / math.sqrt(N)
    r0 = rng.random((B, N)) + 0.05
    G = rng.standard_normal((T, B, N))
    return A, Wa, Wo, r0, G


@pytest.mark.parametrize("name", ACTS)
def test_manual_bptt_equals_torch_autograd(name):
    B, T, k, N = 4, 10, 4, 8
    A, Wa, Wo, r0, G = _problem(11, B, T, k, N)
    J0, J1, alpha = -0.1, 0.1, 0.15
    hist, _ = O.forward_per_sample(A, Wa, J0, J1, Wo, r0, alpha, name)
    got = O.backward_manual(G, A, Wa, J0, J1, Wo, hist, r0, alpha, name)

    t = lambda x, g=False: torch.tensor(x, dtype=torch.float64, requires_grad=g)
    At, Wat, Wot, r0t = t(A, True), t(Wa, True), t(Wo, True), t(r0, True)
    TP.ring_forward(At, Wat, J0, J1, Wot, r0t, alpha, name).backward(t(G))
    np.testing.assert_allclose(got["grad_Wa"], Wat.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(got["grad_Wo"], Wot.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(got["grad_A"], At.grad.numpy(), rtol=0, atol=1e-12)
    np.testing.assert_allclose(got["grad_r_init"], r0t.grad.numpy(), rtol=0, atol=1e-12)


def test_torch_port_passes_fp64_gradcheck_at_reference_shape():
    # N=8, k=4, T=10, B=4, tanh, alpha=0.15
    A, Wa, Wo, r0, _ = _problem(12, 4, 10, 4, 8)
    t = lambda x, g=False: torch.tensor(x, dtype=torch.float64, requires_grad=g)
    At, r0t = t(A), t(r0)
    fn = lambda Wa_, Wo_: TP.ring_forward(At, Wa_, -0.1, 0.1, Wo_, r0t, 0.15, "tanh")
    assert torch.autograd.gradcheck(fn, (t(Wa, True), t(Wo, True)), eps=1e-6, atol=1e-6)


@pytest.mark.parametrize("name", ["gelu", "tanh", "silu"])
def test_grad_A_and_grad_r_init_by_central_differences(name):
    B, T, k, N = 2, 5, 2, 6
    A, Wa, Wo, r0, G = _problem(13, B, T, k, N)
    J0, J1, alpha = -0.2, 0.3, 0.15

    def loss(A_, r0_):
        return float((O.forward_per_sample(A_, Wa, J0, J1, Wo, r0_, alpha, name)[0] * G).sum())

    hist, _ = O.forward_per_sample(A, Wa, J0, J1, Wo, r0, alpha, name)
    got = O.backward_manual(G, A, Wa, J0, J1, Wo, hist, r0, alpha, name)
    h = 1e-6
    for idx in [(0, 0, 0), (1, 2, 1), (0, 4, 1), (1, 3, 0)]:
        Ap, Am = A.copy(), A.copy()
        Ap[idx] += h
        Am[idx] -= h
        fd = (loss(Ap, r0) - loss(Am, r0)) / (2 * h)
        assert abs(got["grad_A"][idx] - fd) < 1e-7
    for idx in [(0, 0), (1, 3), (0, 5)]:
        rp, rm = r0.copy(), r0.copy()
        rp[idx] += h
        rm[idx] -= h
        fd = (loss(A, rp) - loss(A, rm)) / (2 * h)
        assert abs(got["grad_r_init"][idx] - fd) < 1e-7


@pytest.mark.parametrize("name", ACTS)
def test_weight_gradients_by_central_differences(name):
    B, T, k, N = 2, 4, 2, 5
    A, Wa, Wo, r0, G = _problem(14, B, T, k, N)
    if name == "relu":   # keep pre-activations away from the kink
        Wo = np.abs(Wo) + 0.2
    J0, J1, alpha = 0.05, 0.7, 0.15
    hist, _ = O.forward_per_sample(A, Wa, J0, J1, Wo, r0, alpha, name)
    got = O.backward_manual(G, A, Wa, J0, J1, Wo, hist, r0, alpha, name)
    h = 1e-6
    f = lambda Wa_, Wo_: float((O.forward_per_sample(A, Wa_, J0, J1, Wo_, r0, alpha, name)[0] * G).sum())
    for idx in [(0, 1, 2), (1, 4, 0), (1, 0, 3)]:
        p, m = Wa.copy(), Wa.copy()
        p[idx] += h
        m[idx] -= h
        assert abs(got["grad_Wa"][idx] - (f(p, Wo) - f(m, Wo)) / (2 * h)) < 1e-6
    for idx in [(1, 2), (4, 0), (0, 3)]:       # [i,j] vs [j,i] would fail here
        p, m = Wo.copy(), Wo.copy()
        p[idx] += h
        m[idx] -= h
        assert abs(got["grad_Wo"][idx] - (f(Wa, p) - f(Wa, m)) / (2 * h)) < 1e-6


@pytest.mark.parametrize("name", ACTS)
@pytest.mark.parametrize("shape", [(4, 6, 2, 8), (3, 5, 5, 7)])
def test_dense_bptt_equals_per_sample_bptt(name, shape):
    B, T, k, N = shape
    A, Wa, Wo, r0, G = _problem(15, B, T, k, N)
    hist, _ = O.forward_per_sample(A, Wa, -0.1, 0.1, Wo, r0, 0.15, name)
    a = O.backward_manual(G, A, Wa, -0.1, 0.1, Wo, hist, r0, 0.15, name)
    b = O.backward_dense(G, A, Wa, -0.1, 0.1, Wo, hist, r0, 0.15, name)
    for key in a:
        np.testing.assert_allclose(a[key], b[key], rtol=0, atol=1e-12, err_msg=key)


def test_single_step_gradient_closed_form():
    # T=1: grad_Wo = J1 * (alpha*F'(re)*G)^T r0 exactly; pins J1 scaling and the outer-product order.
    B, T, k, N = 3, 1, 2, 4
    A, Wa, Wo, r0, G = _problem(16, B, T, k, N)
    hist, re = O.forward_per_sample(A, Wa, -0.1, 0.25, Wo, r0, 0.15, "tanh")
    got = O.backward_manual(G, A, Wa, -0.1, 0.25, Wo, hist, r0, 0.15, "tanh")
    g = 0.15 * (1 - np.tanh(re[0]) ** 2) * G[0]
    np.testing.assert_allclose(got["grad_Wo"], 0.25 * g.T @ r0, rtol=0, atol=1e-14)
    np.testing.assert_allclose(got["grad_Wa"][1], (A[:, 0, 1:2] * g).T @ r0, rtol=0, atol=1e-14)
