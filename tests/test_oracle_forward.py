"""Pins the oracle's activations and forward recurrence by mathematics (the reference holds no
golden vectors for this path): library routines, brute-force element loops, closed forms."""
import math

import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from oracle import torch_port as TP

ACTS = ["relu", "gelu", "tanh", "silu"]


def _rand_problem(rng, B, T, k, N, scale=None):
    scale = 1.0 / math.sqrt(N) if scale is None else scale
    A = rng.random((B, T, k)) * 0.3
    Wa = rng.standard_normal((k, N, N)) * scale
    Wo = rng.standard_normal((N, N)) * scale
    r0 = rng.random((B, N))
    return A, Wa, Wo, r0


@pytest.mark.parametrize("name", ACTS)
def test_activation_matches_torch_functional(name):
    x = np.linspace(-6, 6, 4001)
    xt = torch.tensor(x, dtype=torch.float64)
    ref = {"relu": torch.relu, "gelu": torch.nn.functional.gelu, "tanh": torch.tanh,
           "silu": torch.nn.functional.silu}[name](xt).numpy()
    np.testing.assert_allclose(O.activation(x, name), ref, rtol=0, atol=1e-14)


@pytest.mark.parametrize("name", ACTS)
def test_activation_derivative_matches_autograd_and_finite_difference(name):
    x = np.linspace(-5, 5, 1001) + 1e-3          # keep off relu's kink at 0
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    TP.non_linear(xt, name).sum().backward()
    np.testing.assert_allclose(O.activation_derivative(x, name), xt.grad.numpy(), rtol=0, atol=1e-13)
    h = 1e-6
    fd = (O.activation(x + h, name) - O.activation(x - h, name)) / (2 * h)
    np.testing.assert_allclose(O.activation_derivative(x, name), fd, rtol=0, atol=1e-8)


def test_gelu_derivative_uses_normal_density_constant():
    # F'(x) = Phi(x) + x*phi(x) with phi(1) = exp(-1/2)/sqrt(2*pi); a 1/sqrt(pi) constant fails this.
    x = np.array([1.0])
    phi = math.exp(-0.5) / math.sqrt(2 * math.pi)
    Phi = 0.5 * (1 + math.erf(1 / math.sqrt(2)))
    assert abs(O.activation_derivative(x, "gelu")[0] - (Phi + phi)) < 1e-15


def test_invalid_activation_raises():
    with pytest.raises(ValueError):
        O.activation(np.zeros(2), "sigmoid")
    with pytest.raises(ValueError):
        O.activation_derivative(np.zeros(2), "linear")


@pytest.mark.parametrize("name", ACTS)
def test_forward_matches_brute_force_element_loops(name):
    """Orientation pin: re[b,i] = sum_j W_eff[b,i,j] * r[b,j], written as scalar loops."""
    rng = np.random.default_rng(1)
    B, T, k, N = 3, 4, 3, 5
    A, Wa, Wo, r0 = _rand_problem(rng, B, T, k, N, scale=0.7)
    J0, J1, alpha = -0.1, 0.1, 0.15
    hist, re_hist = O.forward_per_sample(A, Wa, J0, J1, Wo, r0, alpha, name)
    r = r0.copy()
    for t in range(T):
        new = np.zeros_like(r)
        for b in range(B):
            for i in range(N):
                acc = 0.0
                for j in range(N):
                    w = J0 + J1 * Wo[i, j]
                    for c in range(k):
                        w += A[b, t, c] * Wa[c, i, j]
                    acc += w * r[b, j]
                assert abs(re_hist[t, b, i] - acc) < 1e-12
                new[b, i] = (1 - alpha) * r[b, i] + alpha * O.activation(np.array(acc), name)
        r = new
        np.testing.assert_allclose(hist[t], r, rtol=0, atol=1e-12)


@pytest.mark.parametrize("name", ACTS)
@pytest.mark.parametrize("shape", [(4, 5, 2, 8), (2, 3, 3, 7), (5, 6, 1, 16)])
def test_dense_form_equals_per_sample_form(name, shape):
    rng = np.random.default_rng(2)
    B, T, k, N = shape
    A, Wa, Wo, r0 = _rand_problem(rng, B, T, k, N)
    a, ra = O.forward_per_sample(A, Wa, -0.1, 0.1, Wo, r0, 0.15, name)
    b, rb = O.forward_dense(A, Wa, -0.1, 0.1, Wo, r0, 0.15, name)
    np.testing.assert_allclose(a, b, rtol=0, atol=1e-12)
    np.testing.assert_allclose(ra, rb, rtol=0, atol=1e-12)


def test_tensor_J0_is_accepted_by_the_per_sample_form():
    # torch models hold J0 as an N x N constant (train/train_ring_attractor.py:89)
    rng = np.random.default_rng(3)
    A, Wa, Wo, r0 = _rand_problem(rng, 2, 3, 2, 6)
    a, _ = O.forward_per_sample(A, Wa, -0.1 * np.ones((6, 6)), 0.1, Wo, r0, 0.15, "tanh")
    b, _ = O.forward_dense(A, Wa, -0.1, 0.1, Wo, r0, 0.15, "tanh")
    np.testing.assert_allclose(a, b, rtol=0, atol=1e-13)


def test_alpha_zero_freezes_state():
    rng = np.random.default_rng(4)
    A, Wa, Wo, r0 = _rand_problem(rng, 3, 5, 2, 6)
    hist, _ = O.forward_dense(A, Wa, -0.1, 0.1, Wo, r0, 0.0, "gelu")
    for t in range(5):
        np.testing.assert_array_equal(hist[t], r0)


@pytest.mark.parametrize("name", ACTS)
def test_zero_weights_give_geometric_decay(name):
    # F(0) = 0 for all four activations => r_t = (1-alpha)^(t+1) r_0
    rng = np.random.default_rng(5)
    B, T, k, N = 2, 6, 2, 5
    A = rng.random((B, T, k))
    r0 = rng.random((B, N))
    hist, _ = O.forward_per_sample(A, np.zeros((k, N, N)), 0.0, 1.0, np.zeros((N, N)), r0, 0.15, name)
    for t in range(T):
        np.testing.assert_allclose(hist[t], 0.85 ** (t + 1) * r0, rtol=1e-13)


def test_relu_with_pure_inhibition_is_pure_decay():
    rng = np.random.default_rng(6)
    B, T, k, N = 2, 5, 2, 6
    A = rng.random((B, T, k))
    r0 = rng.random((B, N))
    hist, re = O.forward_dense(A, np.zeros((k, N, N)), -0.3, 1.0, np.zeros((N, N)), r0, 0.15, "relu")
    assert (re <= 0).all()
    for t in range(T):
        np.testing.assert_allclose(hist[t], 0.85 ** (t + 1) * r0, rtol=1e-13)


def test_zero_action_reduces_to_plain_leaky_rnn_matmul():
    rng = np.random.default_rng(7)
    B, T, k, N = 3, 4, 2, 6
    _, Wa, Wo, r0 = _rand_problem(rng, B, T, k, N)
    hist, _ = O.forward_per_sample(np.zeros((B, T, k)), Wa, -0.1, 0.1, Wo, r0, 0.15, "tanh")
    r = torch.tensor(r0)
    M = torch.tensor(-0.1 + 0.1 * Wo)
    for t in range(T):
        r = 0.85 * r + 0.15 * torch.tanh(torch.matmul(r, M.T))
        np.testing.assert_allclose(hist[t], r.numpy(), rtol=0, atol=1e-13)


def test_linear_regime_matches_matrix_power():
    # tiny state => tanh(x) = x - x^3/3: r_t = ((1-a)I + a*W_eff)^t r_0 up to O(|x|^3)
    rng = np.random.default_rng(8)
    B, T, k, N = 2, 7, 2, 5
    A = np.tile(rng.random((B, 1, k)), (1, T, 1))      # constant action => one W_eff per sample
    Wa = rng.standard_normal((k, N, N)) * 0.3
    Wo = rng.standard_normal((N, N)) * 0.3
    r0 = rng.standard_normal((B, N)) * 1e-4
    hist, _ = O.forward_per_sample(A, Wa, -0.1, 0.1, Wo, r0, 0.15, "tanh")
    W_eff = O.effective_weights(A[:, 0, :], Wa, -0.1, 0.1, Wo)
    for b in range(B):
        M = 0.85 * np.eye(N) + 0.15 * W_eff[b]
        np.testing.assert_allclose(hist[T - 1, b], np.linalg.matrix_power(M, T) @ r0[b], rtol=0, atol=1e-11)


@pytest.mark.parametrize("name", ACTS)
def test_torch_port_forward_equals_numpy_oracle(name):
    rng = np.random.default_rng(9)
    B, T, k, N = 4, 6, 3, 9
    A, Wa, Wo, r0 = _rand_problem(rng, B, T, k, N)
    hist, _ = O.forward_per_sample(A, Wa, -0.1, 0.1, Wo, r0, 0.15, name)
    t = lambda x: torch.tensor(x, dtype=torch.float64)
    hist_t = TP.ring_forward(t(A), t(Wa), -0.1, 0.1, t(Wo), t(r0), 0.15, name)
    np.testing.assert_allclose(hist, hist_t.numpy(), rtol=0, atol=1e-13)


def test_long_sequence_at_its_own_gain_where_bf16_weights_leave_the_tolerance():
    """BASELINE's long-sequence configuration at its own parameters (N = 512, T = 512, tanh, J0 = -1/N, J1 = 1,
    weights ~ N(0, 1/N); a small batch here).  What the parity tests may and may not demand there:
      * the dynamics are NOT chaotic: a 1e-9 perturbation of the initial state is still ~1e-9 after 512 steps, and
        the fp32 torch port of the reference formulation (train/train_ring_attractor.py:158-177) agrees with fp64
        to 1e-4 at every step -- an implementation that computes in fp32 has no excuse here;
      * they are marginally stable, so a FIXED perturbation of the network accumulates: with the MFMA operands
        rounded to bf16 the per-step deviation from fp64 (relative to the step's largest state) passes 1e-2 at
        t ~ 166 and reaches ~1e-1 at t = 511; the GPU parity test of this configuration therefore holds the
        kernels to fp64 over the first 150 steps and to the rounding-aware model over all 512;
      * all of it comes from rounding Wo: rounding only Wa, or only the state operand, stays under 6e-3 to the end,
        and Wo carried as two bf16 operands (hi + lo, the operator's precise_wo option) under 5e-3."""
    import torch
    from oracle import ring_oracle_bf16 as OB
    from oracle import torch_port as TP
    from tests.ring_cases import make_problem
    N, B, T, k = 512, 8, 512, 2
    J0, J1 = -1.0 / N, 1.0
    p = make_problem(3, B, T, k, N, bump="vm")
    args = (p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, "tanh")
    ref, _ = O.forward_dense(*args)

    def per_step(x):
        return np.array([O.max_rel_err(x[t], ref[t]) for t in range(T)])

    bumped = p["r0"].astype(np.float64) * (1.0 + 1e-9 * np.sign(np.random.default_rng(0).standard_normal(p["r0"].shape)))
    e_pert = per_step(O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], bumped, 0.15, "tanh")[0])
    assert e_pert.max() <= 1e-8
    t_ = lambda x: torch.tensor(x)
    with torch.no_grad():
        f32 = TP.ring_forward(t_(p["A"]), t_(p["Wa"]), J0, J1, t_(p["Wo"]), t_(p["r0"]), 0.15, "tanh").numpy()
    assert per_step(f32.astype(np.float64)).max() <= 1e-4
    e_bf16 = per_step(OB.forward_backward(*args)["bump_history"])
    horizon = int(np.nonzero(e_bf16 > 1e-2)[0][0])
    print(f"[measured] N=512 T=512 J1=1 tanh: bf16-operand model leaves 1e-2 at t = {horizon}, "
          f"error at t = 511 {e_bf16[-1]:.2e}; fp32 port max {per_step(f32.astype(np.float64)).max():.1e}")
    assert 150 <= horizon <= 250 and e_bf16[:150].max() <= 1e-2 and e_bf16[-1] > 5e-2
    Wo_hi = OB.round_bf16(p["Wo"])
    e_wo = per_step(O.forward_dense(p["A"], p["Wa"], J0, J1, Wo_hi, p["r0"], 0.15, "tanh")[0])
    e_wa = per_step(O.forward_dense(p["A"], OB.round_bf16(p["Wa"]), J0, J1, p["Wo"], p["r0"], 0.15, "tanh")[0])
    e_r = per_step(OB.forward_backward(*args, only=("r",))["bump_history"])
    assert e_wo[-1] > 0.8 * e_bf16[-1] and e_wa.max() <= 6e-3 and e_r.max() <= 6e-3
    # Wo = hi + lo as two bf16 operands, Wa and the state operand rounded as always
    Wo_lo = OB.round_bf16(p["Wo"].astype(np.float64) - Wo_hi)
    split = OB.forward_backward(p["A"], OB.round_bf16(p["Wa"]), J0, J1, Wo_hi + Wo_lo, p["r0"], 0.15, "tanh", only=("r",))
    assert per_step(split["bump_history"]).max() <= 5e-3
