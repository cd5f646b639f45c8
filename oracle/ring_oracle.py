"""fp64 numpy restatement of the leaky ring-attractor time loop and its BPTT.

TEST INFRASTRUCTURE ONLY: this file is the checker the HIP kernels are compared
against.  It is never imported by the shipped package.

Each function cites the reference file:line whose behaviour it restates (paths
are relative to the reference repository root).  Nothing here is executed from
the reference; the formulas are written out again in numpy.

Parity status.  The reference holds no golden vectors, fixtures or known-answer
tests for this path, so every function below is pinned by mathematics instead
(tests/test_oracle_*.py): closed forms, special cases that reduce to a library
routine, brute-force element loops on tiny inputs, finite differences and an
independent torch-autograd restatement.  Functions without such a check are
listed here as "parity unpinned": (none at present).
"""
from __future__ import annotations

import math

import numpy as np
from scipy.special import erf as _erf

ACTIVATION_IDS = {"relu": 0, "gelu": 1, "tanh": 2, "silu": 3}  # cpp/ring_rnn_cuda.py:63


# --------------------------------------------------------------------------- activations
def activation(x: np.ndarray, name: str) -> np.ndarray:
    """F(x).  train/train_ring_attractor.py:10-18 (tanh, relu, exact-erf gelu);
    legacy/bwd_fp32.py:415-430 adds silu; device twin cpp/cuda_common.cuh:58-70."""
    if name == "relu":
        return np.maximum(x, 0.0)
    if name == "gelu":
        return x * 0.5 * (1.0 + _erf(x / math.sqrt(2.0)))
    if name == "tanh":
        return np.tanh(x)
    if name == "silu":
        return x / (1.0 + np.exp(-x))
    raise ValueError(f"Invalid activation '{name}'. Must be one of {list(ACTIVATION_IDS)}.")


def activation_derivative(x: np.ndarray, name: str) -> np.ndarray:
    """F'(x).  legacy/bwd_fp32.py:433-461.  The gelu density uses 1/sqrt(2*pi)
    (the torch path), not the 1/sqrt(pi) constant of cpp/cuda_common.cuh:79."""
    if name == "relu":
        return (x > 0.0).astype(x.dtype)
    if name == "gelu":
        cdf = 0.5 * (1.0 + _erf(x / math.sqrt(2.0)))
        pdf = np.exp(-0.5 * x * x) / math.sqrt(2.0 * math.pi)
        return cdf + x * pdf
    if name == "tanh":
        th = np.tanh(x)
        return 1.0 - th * th
    if name == "silu":
        s = 1.0 / (1.0 + np.exp(-x))
        return s * (1.0 + x * (1.0 - s))
    raise ValueError(f"Invalid activation '{name}'. Must be one of {list(ACTIVATION_IDS)}.")


# --------------------------------------------------------------------------- forward
def effective_weights(A_t, Wa, J0, J1, Wo):
    """W_eff[b] = J0 + J1*Wo + sum_k A_t[b,k]*Wa[k]  -> [B,N,N].
    train/train_ring_attractor.py:164-166 (k=2: L*Wl + R*Wr);
    train/train_general_ring_no_gain.py:111-118 (general k).  J0 may be a scalar
    (cpp API) or an N x N array (torch models)."""
    return J0 + J1 * Wo[None] + np.einsum("bk,kij->bij", A_t, Wa)


def forward_per_sample(A, Wa, J0, J1, Wo, r_init, alpha, activation_name):
    """The reference's own formulation: materialise W_eff per sample, batched
    mat-vec, activation, leak.  train/train_ring_attractor.py:158-177,
    legacy/bwd_fp32.py:510-528.  A: [B,T,k]; returns (bump_history [T,B,N],
    re_history [T,B,N]) in the operator's [T,B,N] layout (cpp/ring_rnn_cuda.py:62)."""
    A = np.asarray(A, np.float64)
    Wa = np.asarray(Wa, np.float64)
    Wo = np.asarray(Wo, np.float64)
    r = np.array(r_init, np.float64)
    B, T, k = A.shape
    N = Wo.shape[0]
    hist = np.empty((T, B, N))
    re_hist = np.empty((T, B, N))
    for t in range(T):
        W_eff = effective_weights(A[:, t, :], Wa, J0, J1, Wo)
        re = np.einsum("bij,bj->bi", W_eff, r)
        r = (1.0 - alpha) * r + alpha * activation(re, activation_name)
        hist[t] = r
        re_hist[t] = re
    return hist, re_hist


def forward_dense(A, Wa, J0, J1, Wo, r_init, alpha, activation_name):
    """Algebraically identical dense form (scalar J0 only):
    re = J0*sum_j r + J1*(r @ Wo^T) + sum_k A_k * (r @ Wa_k^T).
    Same reference lines as forward_per_sample; this is the form the HIP kernels
    evaluate, so tests assert the two agree."""
    A = np.asarray(A, np.float64)
    Wa = np.asarray(Wa, np.float64)
    Wo = np.asarray(Wo, np.float64)
    r = np.array(r_init, np.float64)
    B, T, k = A.shape
    N = Wo.shape[0]
    Wcat_T = np.concatenate([Wo.T] + [Wa[i].T for i in range(k)], axis=1)  # [N,(1+k)N]
    hist = np.empty((T, B, N))
    re_hist = np.empty((T, B, N))
    for t in range(T):
        P = (r @ Wcat_T).reshape(B, 1 + k, N)
        re = J0 * r.sum(axis=1, keepdims=True) + J1 * P[:, 0, :]
        re = re + np.einsum("bk,bkn->bn", A[:, t, :], P[:, 1:, :])
        r = (1.0 - alpha) * r + alpha * activation(re, activation_name)
        hist[t] = r
        re_hist[t] = re
    return hist, re_hist


# --------------------------------------------------------------------------- backward
def backward_manual(grad_output, A, Wa, J0, J1, Wo, bump_history, r_init, alpha, activation_name):
    """Reverse-time BPTT in the reference's per-sample form.
    legacy/bwd_fp32.py:86-109 (loop body) with re recomputed from r_prev as the
    CUDA operator does (cpp/ring_rnn_cuda.py:106, bwd kernel :53-269).
    grad_output/bump_history: [T,B,N].  Returns grad_Wa, grad_Wo (the two the
    reference returns, cpp/ring_rnn_cuda.py:144) plus grad_A [B,T,k] and
    grad_r_init [B,N], which the reference leaves as None."""
    G_out = np.asarray(grad_output, np.float64)
    A = np.asarray(A, np.float64)
    Wa = np.asarray(Wa, np.float64)
    Wo = np.asarray(Wo, np.float64)
    hist = np.asarray(bump_history, np.float64)
    r0 = np.asarray(r_init, np.float64)
    B, T, k = A.shape
    N = Wo.shape[0]
    grad_Wa = np.zeros_like(Wa)
    grad_Wo = np.zeros_like(Wo)
    grad_A = np.zeros_like(A)
    carry = np.zeros((B, N))
    for t in range(T - 1, -1, -1):
        r_prev = r0 if t == 0 else hist[t - 1]
        W_eff = effective_weights(A[:, t, :], Wa, J0, J1, Wo)
        re = np.einsum("bij,bj->bi", W_eff, r_prev)
        G = G_out[t] + carry
        g = activation_derivative(re, activation_name) * G * alpha
        outer = np.einsum("bi,bj->bij", g, r_prev)          # dL/dW_eff per sample
        grad_Wo += J1 * outer.sum(axis=0)
        grad_Wa += np.einsum("bk,bij->kij", A[:, t, :], outer)
        grad_A[:, t, :] = np.einsum("bij,kij->bk", outer, Wa)
        carry = np.einsum("bij,bi->bj", W_eff, g) + (1.0 - alpha) * G
    return {"grad_Wa": grad_Wa, "grad_Wo": grad_Wo, "grad_A": grad_A, "grad_r_init": carry}


def backward_dense(grad_output, A, Wa, J0, J1, Wo, bump_history, r_init, alpha, activation_name):
    """Same BPTT in dense form (scalar J0): no per-sample N x N objects, so it
    runs at the benchmark shapes.  g = alpha*F'(re)*G;
    carry = (1-alpha)G + J0*sum_i g + J1*(g@Wo) + sum_k A_k*(g@Wa_k);
    grad_Wo = J1 * g^T r_prev;  grad_Wa[k] = (A_k*g)^T r_prev;
    grad_A[b,t,k] = sum_j r_prev[b,j]*(g@Wa_k)[b,j].
    Same reference lines as backward_manual."""
    G_out = np.asarray(grad_output, np.float64)
    A = np.asarray(A, np.float64)
    Wa = np.asarray(Wa, np.float64)
    Wo = np.asarray(Wo, np.float64)
    hist = np.asarray(bump_history, np.float64)
    r0 = np.asarray(r_init, np.float64)
    B, T, k = A.shape
    N = Wo.shape[0]
    Wcat_T = np.concatenate([Wo.T] + [Wa[i].T for i in range(k)], axis=1)  # [N,(1+k)N]
    Wcat = np.concatenate([Wo] + [Wa[i] for i in range(k)], axis=1)        # [N,(1+k)N] rows i
    grad_Wa = np.zeros_like(Wa)
    grad_Wo = np.zeros_like(Wo)
    grad_A = np.zeros_like(A)
    carry = np.zeros((B, N))
    for t in range(T - 1, -1, -1):
        r_prev = r0 if t == 0 else hist[t - 1]
        P = (r_prev @ Wcat_T).reshape(B, 1 + k, N)
        re = J0 * r_prev.sum(axis=1, keepdims=True) + J1 * P[:, 0, :]
        re = re + np.einsum("bk,bkn->bn", A[:, t, :], P[:, 1:, :])
        G = G_out[t] + carry
        g = activation_derivative(re, activation_name) * G * alpha
        Q = (g @ Wcat).reshape(B, 1 + k, N)                                 # Q_m = g @ W_m
        carry = (1.0 - alpha) * G + J0 * g.sum(axis=1, keepdims=True) + J1 * Q[:, 0, :]
        carry = carry + np.einsum("bk,bkn->bn", A[:, t, :], Q[:, 1:, :])
        grad_Wo += J1 * (g.T @ r_prev)
        for c in range(k):
            grad_Wa[c] += (A[:, t, c:c + 1] * g).T @ r_prev
        grad_A[:, t, :] = np.einsum("bkn,bn->bk", Q[:, 1:, :], r_prev)
    return {"grad_Wa": grad_Wa, "grad_Wo": grad_Wo, "grad_A": grad_A, "grad_r_init": carry}


# --------------------------------------------------------------------------- read-out, losses, decoders
def w_delta7(N: int) -> np.ndarray:
    """cos(2*pi*(i-j)/N).  train/train_ring_attractor.py:82-86."""
    idx = np.arange(N, dtype=np.float64)
    return np.cos(2.0 * np.pi * (idx[:, None] - idx[None, :]) / N)


def readout(bump: np.ndarray) -> np.ndarray:
    """(bump @ W_delta7) / row-max over neurons.  train/train_ring_attractor.py:181-183;
    train_general_ring_no_gain.py:113-116 (root script, CUDA-backed path)."""
    N = bump.shape[-1]
    proj = bump @ w_delta7(N)
    return proj / proj.max(axis=-1, keepdims=True)


def create_initial_bump(initial_angles, N: int, bump_width_factor: float = 10.0) -> np.ndarray:
    """Gaussian of the circular index distance, sigma = N/width_factor, L2-normalised per row.
    train/train_ring_attractor.py:21-52."""
    ang = np.asarray(initial_angles, np.float64)
    centre = (ang * N / (2.0 * np.pi))[:, None]
    idx = np.arange(N, dtype=np.float64)[None, :]
    d = np.abs(idx - centre)
    d = np.minimum(d, N - d)
    sigma = N / bump_width_factor
    bump = np.exp(-(d * d) / (2.0 * sigma * sigma))
    return bump / np.linalg.norm(bump, axis=1, keepdims=True)


def von_mises_bump(initial_angles, N: int, kappa: float = 4.0) -> np.ndarray:
    """Benchmark-config initial state: exp(kappa*(cos(theta_i-theta0)-1)), theta_i = 2*pi*i/N,
    L2-normalised.  (Not a reference function: the benchmark configs name it.)"""
    ang = np.asarray(initial_angles, np.float64)[:, None]
    theta = 2.0 * np.pi * np.arange(N, dtype=np.float64)[None, :] / N
    bump = np.exp(kappa * (np.cos(theta - ang) - 1.0))
    return bump / np.linalg.norm(bump, axis=1, keepdims=True)


def preferred_angles(N: int) -> np.ndarray:
    """linspace(0, 2*pi, N) with the end point INCLUDED.  train/train_ring_attractor.py:197-198, 245, 260."""
    return np.linspace(0.0, 2.0 * np.pi, N)


def cosine_similarity_loss(wave: np.ndarray, true_angle: np.ndarray) -> float:
    """MSE between the unit vectors of the decoded and the true angle.
    train/train_ring_attractor.py:190-220."""
    pa = preferred_angles(wave.shape[-1])
    px = (wave * np.cos(pa)).sum(axis=-1)
    py = (wave * np.sin(pa)).sum(axis=-1)
    theta = np.arctan2(py, px)
    return float(np.mean((np.cos(theta) - np.cos(true_angle)) ** 2 + (np.sin(theta) - np.sin(true_angle)) ** 2))


def bump_amplitude_loss(bump: np.ndarray, target_amplitude=None) -> float:
    """Mean squared deviation of the per-step L1 mass from a target (default: step 0's).
    bump: [B,T,N].  train/train_ring_attractor.py:275-298."""
    total = np.abs(bump).sum(axis=2)
    if target_amplitude is None:
        target_amplitude = total[:, 0:1]
    return float(np.mean((total - target_amplitude) ** 2))


def decode_angle_from_population_vector(activity: np.ndarray) -> np.ndarray:
    """atan2 of the sin/cos-weighted sums, wrapped to [0, 2*pi).
    train/train_ring_attractor.py:257-272."""
    pa = preferred_angles(activity.shape[-1])
    x = (activity * np.cos(pa)).sum(axis=-1)
    y = (activity * np.sin(pa)).sum(axis=-1)
    return (np.arctan2(y, x) + 2.0 * np.pi) % (2.0 * np.pi)


def decode_angle_from_argmax(activity: np.ndarray) -> np.ndarray:
    """Preferred angle of the most active neuron.  train/train_ring_attractor.py:242-254."""
    pa = preferred_angles(activity.shape[-1])
    return pa[np.argmax(activity, axis=-1)]


# --------------------------------------------------------------------------- inputs
def generate_av_integration_data(num_trials, seq_len, rng, zero_padding_start_ratio=0.1,
                                 zero_ratios_in_rest=(0.2, 0.5, 0.8), max_av=0.1 * np.pi):
    """Angular-velocity trials and their integrated angle.
    utils/generate_av_integration_data.py:11-58: the first int(T*ratio) steps are zero; of the
    remaining len_rest steps exactly len_rest - floor(len_rest*zero_ratio) randomly placed ones
    carry U(-max_av, max_av) draws; angle[:,0] = U(0,2*pi), angle[:,1:] = (angle0 + cumsum(av[:,:-1])) % 2*pi.
    `rng` is a numpy Generator; the random stream is this file's own (same distribution, not the
    same bits as torch's)."""
    av = np.zeros((num_trials, seq_len))
    n0 = int(seq_len * zero_padding_start_ratio)
    rest = seq_len - n0
    angle0 = rng.random(num_trials) * 2.0 * np.pi
    ratios = np.asarray(zero_ratios_in_rest, np.float64)[rng.integers(0, len(zero_ratios_in_rest), num_trials)]
    # float32 product as in the reference (torch default dtype), then truncation
    n_nonzero = rest - (np.float32(rest) * ratios.astype(np.float32)).astype(np.int64)
    if rest > 0:
        values = (rng.random((num_trials, rest)) - 0.5) * 2.0 * max_av
        order = np.argsort(rng.random((num_trials, rest)), axis=1)
        av[:, n0:] = values * (order < n_nonzero[:, None])
    angle = np.zeros((num_trials, seq_len))
    angle[:, 0] = angle0
    angle[:, 1:] = (angle0[:, None] + np.cumsum(av[:, :-1], axis=1)) % (2.0 * np.pi)
    return av, angle


def av_to_action_signal(av: np.ndarray) -> np.ndarray:
    """[L, R] = [relu(-av), relu(av)] -> [B,T,2].  train_general_ring_no_gain.py:176-188 (root)."""
    return np.stack([np.maximum(-av, 0.0), np.maximum(av, 0.0)], axis=2)


def av_to_action_signal_nd(av: np.ndarray, action_dim: int = 16, zero_padding: bool = True) -> np.ndarray:
    """k-channel action signal.  train_general_ring_no_gain.py:200-229 (root): with zero padding
    channels 0/1 are L/R and the rest stay zero; otherwise relu(av * linspace(-1,1,k))."""
    if zero_padding:
        out = np.zeros(av.shape + (action_dim,))
        out[..., 0] = np.maximum(-av, 0.0)
        out[..., 1] = np.maximum(av, 0.0)
        return out
    scales = np.linspace(-1.0, 1.0, action_dim)
    return np.maximum(av[..., None] * scales, 0.0)


# --------------------------------------------------------------------------- comparison helpers
def cosine(a: np.ndarray, b: np.ndarray) -> float:
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(a @ b / (np.linalg.norm(a) * np.linalg.norm(b) + 1e-300))


def max_rel_err(x: np.ndarray, ref: np.ndarray) -> float:
    """max|x-ref| / max|ref|: the scale-normalised maximum error used for the trajectory and
    gradient tolerances (an element-wise ratio is undefined where ref crosses zero)."""
    x = np.asarray(x, np.float64)
    ref = np.asarray(ref, np.float64)
    return float(np.max(np.abs(x - ref)) / (np.max(np.abs(ref)) + 1e-300))


def elementwise_rel_err(x: np.ndarray, ref: np.ndarray, floor_frac: float = 0.1) -> float:
    """max over the entries with |ref| >= floor_frac * max|ref| of |x - ref| / |ref|: an element-wise relative error
    on the entries that carry the signal (below the floor the ratio measures rounding noise against near-zeros)."""
    x = np.asarray(x, np.float64)
    ref = np.asarray(ref, np.float64)
    big = np.abs(ref) >= floor_frac * np.max(np.abs(ref))
    if not big.any():
        return 0.0
    return float(np.max(np.abs(x - ref)[big] / np.abs(ref)[big]))


def loss_pair_rank2(bump_tbn, target_angle, bump_weight=0.2, target_amplitude=None):
    """The training loss pair and its gradient through the rank-two form of the read-out.

    Restates root train_general_ring_no_gain.py:113-116, 324-330 and train/train_ring_attractor.py:190-220,
    275-298: W_delta7[i][j] = cos(phi_i - phi_j) makes proj_j = C cos(phi_j) + S sin(phi_j) with
    C = sum_i r_i cos(phi_i), S = sum_i r_i sin(phi_i); the positive row maximum cancels in atan2.
    Returns (total, cos_loss, amp_loss, d total / d bump_tbn).  Pinned in tests/test_oracle_helpers.py against the
    literal chain (read-out, normalisation, decode, both losses) and its autograd gradient."""
    r = np.asarray(bump_tbn, np.float64)
    T, B, N = r.shape
    a = np.asarray(target_angle, np.float64).T                      # [T,B]
    j = np.arange(N)
    phi = 2 * np.pi * j / N
    pa = np.linspace(0.0, 2 * np.pi, N)
    a1, a2 = np.sum(np.cos(phi) * np.cos(pa)), np.sum(np.sin(phi) * np.cos(pa))
    b1, b2 = np.sum(np.cos(phi) * np.sin(pa)), np.sum(np.sin(phi) * np.sin(pa))
    C, S = r @ np.cos(phi), r @ np.sin(phi)
    X, Y = C * a1 + S * a2, C * b1 + S * b2
    theta = np.arctan2(Y, X)
    cos_loss = np.mean((np.cos(theta) - np.cos(a)) ** 2 + (np.sin(theta) - np.sin(a)) ** 2)
    amp = np.abs(r).sum(axis=2)                                      # [T,B]
    own = target_amplitude is None
    tgt = amp[0] if own else np.asarray(target_amplitude, np.float64).reshape(B)
    dev = amp - tgt[None, :]
    amp_loss = np.mean(dev ** 2)
    rows = T * B
    dth = 2 * np.sin(theta - a) / np.maximum(X * X + Y * Y, 1e-300) / rows
    kc, ks = dth * (X * b1 - Y * a1), dth * (X * b2 - Y * a2)
    beta = 2 * dev
    if own:
        beta[0] -= 2 * dev.sum(axis=0)
    beta = beta * bump_weight / rows
    grad = kc[..., None] * np.cos(phi) + ks[..., None] * np.sin(phi) + beta[..., None] * np.sign(r)
    return cos_loss + bump_weight * amp_loss, cos_loss, amp_loss, grad


# ---------------------------------------------------------------------------------------------------
# Gain networks of the action signal (train/train_ring_attractor.py:70-79, 136-146;
# train/train_general_ring_attractor.py:38-46, 99-109): per channel c a network
# Linear(1,h) -> GELU (exact erf) -> Linear(h,1) -> Softplus (beta 1, threshold 20) on |x|, and A = x * gain.
# params[c] = [w1[0..h) | b1[0..h) | w2[0..h) | b2].
# ---------------------------------------------------------------------------------------------------
def _gain_internals(x, params):
    x = np.asarray(x, np.float64)
    params = np.asarray(params, np.float64)
    h = (params.shape[1] - 1) // 3
    w1, b1, w2, b2 = params[:, :h], params[:, h:2 * h], params[:, 2 * h:3 * h], params[:, 3 * h]
    m = np.abs(x)
    u = m[..., None] * w1 + b1                              # [B,T,k,h]
    a = activation(u, "gelu")
    z = (a * w2).sum(axis=-1) + b2                          # [B,T,k]
    s = np.where(z > 20.0, z, np.log1p(np.exp(np.minimum(z, 20.0))))
    ds = np.where(z > 20.0, 1.0, 1.0 / (1.0 + np.exp(-np.minimum(z, 20.0))))
    return x, m, u, a, z, s, ds, w1, w2


def gain_forward(x, params):
    """[B,T,k] base signal, [k,3h+1] parameters -> [B,T,k] gated signal x * softplus(net(|x|))."""
    x, _, _, _, _, s, _, _, _ = _gain_internals(x, params)
    return x * s


def gain_backward(x, params, grad_A):
    """Returns (grad_params [k,3h+1], grad_x [B,T,k]) of sum(grad_A * gain_forward(x, params))."""
    x, m, u, a, z, s, ds, w1, w2 = _gain_internals(x, params)
    g = np.asarray(grad_A, np.float64)
    dz = g * x * ds                                          # [B,T,k]
    du = dz[..., None] * w2 * activation_derivative(u, "gelu")
    gw2 = (dz[..., None] * a).sum(axis=(0, 1))
    gb2 = dz.sum(axis=(0, 1))
    gb1 = du.sum(axis=(0, 1))
    gw1 = (du * m[..., None]).sum(axis=(0, 1))
    grad_params = np.concatenate([gw1, gb1, gw2, gb2[:, None]], axis=1)
    dm = (du * w1).sum(axis=-1)
    grad_x = g * s + np.sign(x) * dm
    return grad_params, grad_x
