"""Torch restatement of the reference's pure-PyTorch recurrence (autograd does BPTT).

TEST INFRASTRUCTURE ONLY.  Used (a) as an independent check of the numpy oracle's
manual BPTT, (b) to produce loss-head gradients for tests and the benchmark, and
(c) as the timed CPU baseline ("port" of the reference formulation) on the host
cores.  Never imported by the shipped package.

Formulation follows train/train_ring_attractor.py:158-177 and
train/train_general_ring_no_gain.py:102-128: W_eff is materialised per sample,
the recurrent input is a batched mat-vec, autograd differentiates the loop.
"""
from __future__ import annotations

import math

import torch


def non_linear(x: torch.Tensor, name: str) -> torch.Tensor:
    """train/train_ring_attractor.py:10-18 (+ silu, legacy/bwd_fp32.py:422-423)."""
    if name == "tanh":
        return torch.tanh(x)
    if name == "relu":
        return torch.relu(x)
    if name == "gelu":
        return torch.nn.functional.gelu(x)
    if name == "silu":
        return torch.nn.functional.silu(x)
    raise ValueError(f"Invalid activation '{name}'.")


def ring_forward(action_signal, Wa, J0, J1, Wo, r_init, alpha, activation):
    """Returns bump_history [T,B,N] (the operator's layout, cpp/ring_rnn_cuda.py:62)."""
    B, T, k = action_signal.shape
    N = Wo.shape[0]
    r = r_init
    out = []
    Wa_flat = Wa.reshape(k, N * N)
    for t in range(T):
        W_eff = J0 + J1 * Wo + (action_signal[:, t, :] @ Wa_flat).view(B, N, N)
        re = torch.bmm(W_eff, r.unsqueeze(2)).squeeze(2)
        r = r * (1 - alpha) + non_linear(re, activation) * alpha
        out.append(r)
    return torch.stack(out, dim=0)


def w_delta7(N, dtype=torch.float32, device="cpu"):
    idx = torch.arange(N, dtype=dtype, device=device)
    return torch.cos(2 * math.pi * (idx[:, None] - idx[None, :]) / N)


def readout(bump_btn: torch.Tensor) -> torch.Tensor:
    """train_general_ring_no_gain.py:113-116 (root)."""
    proj = bump_btn @ w_delta7(bump_btn.shape[-1], bump_btn.dtype, bump_btn.device)
    return proj / proj.max(dim=-1, keepdim=True)[0]


def cosine_similarity_loss(wave, true_angle):
    """train/train_ring_attractor.py:190-220."""
    N = wave.shape[-1]
    pa = torch.linspace(0, 2 * math.pi, N, device=wave.device, dtype=wave.dtype)
    px = (wave * torch.cos(pa)).sum(-1)
    py = (wave * torch.sin(pa)).sum(-1)
    th = torch.atan2(py, px)
    return torch.mean((torch.cos(th) - torch.cos(true_angle)) ** 2 + (torch.sin(th) - torch.sin(true_angle)) ** 2)


def bump_amplitude_loss(bump_btn, target_amplitude=None):
    """train/train_ring_attractor.py:275-298."""
    total = bump_btn.abs().sum(dim=2)
    if target_amplitude is None:
        target_amplitude = total[:, 0:1]
    return torch.mean((total - target_amplitude) ** 2)


def loss_pair(bump_tbn: torch.Tensor, target_angle: torch.Tensor, bump_weight: float = 0.2,
              target_amplitude=None) -> torch.Tensor:
    """total = cos-sim loss(readout) + 0.2 * bump-amplitude loss.
    train_general_ring_no_gain.py:324-330 (root)."""
    bump_btn = bump_tbn.permute(1, 0, 2)
    return cosine_similarity_loss(readout(bump_btn), target_angle) + \
        bump_weight * bump_amplitude_loss(bump_btn, target_amplitude)


def fwd_bwd_autograd(action_signal, Wa, J0, J1, Wo, r_init, alpha, activation, grad_output=None,
                     target_angle=None):
    """One forward + autograd backward.  Either an explicit grad_output [T,B,N] (MSE-vs-random-target
    style, legacy/bwd_fp32.py:612-619) or the loss pair on target_angle drives the backward."""
    Wa = Wa.detach().clone().requires_grad_(True)
    Wo = Wo.detach().clone().requires_grad_(True)
    hist = ring_forward(action_signal, Wa, J0, J1, Wo, r_init, alpha, activation)
    if grad_output is not None:
        hist.backward(grad_output)
    else:
        loss_pair(hist, target_angle).backward()
    return hist.detach(), Wa.grad, Wo.grad
