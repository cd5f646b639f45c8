"""Device-side companions of the time loop: the synthetic input generator in front of it and the optimizer tail
(gradient clipping + Adam) behind it, both as HIP kernels behind the C ABI.

`generate_inputs` replaces generate_av_integration_data_ultra_fast + av_to_action_signal(_ND) + create_initial_bump
of the reference (utils/generate_av_integration_data.py:11-58, root train_general_ring_no_gain.py:176-229,
train/train_ring_attractor.py:21-52) with one call that stages nothing from the host; `FusedClipAdam` replaces
clip_grad_norm_ + torch.optim.Adam.step() (root train_general_ring_no_gain.py:333-336)."""
from __future__ import annotations

import ctypes
import math

import torch

from . import _lib


def generate_inputs(seed, batch_size, seq_len, num_neurons, action_dim=2, zero_padding_start_ratio=0.1,
                    zero_ratios_in_rest=None, max_av=0.1 * math.pi, zero_padding=True, bump="gauss", bump_param=None,
                    device="cuda"):
    """Returns (av [B,T], angle [B,T], action_signal [B,T,k], r_init [B,N]) on `device`, a function of `seed` only.
    bump: "gauss" (the reference's, width N / bump_param, default 10) or "vm" (von Mises, kappa = bump_param, default 4)."""
    ratios = [0.2, 0.5, 0.8] if zero_ratios_in_rest is None else [float(r) for r in zero_ratios_in_rest]
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("generate_inputs runs on the GPU; there is no CPU path")
    kind = {"gauss": 0, "vm": 1}[bump]
    if bump_param is None:
        bump_param = 10.0 if kind == 0 else 4.0
    B, T, k, N = int(batch_size), int(seq_len), int(action_dim), int(num_neurons)
    with torch.cuda.device(dev):
        av = torch.empty(B, T, device=dev)
        angle = torch.empty(B, T, device=dev)
        action = torch.empty(B, T, k, device=dev)
        r0 = torch.empty(B, N, device=dev)
        arr = (ctypes.c_float * len(ratios))(*ratios)
        _lib.check(_lib.load().ringattr_generate_inputs(
            int(seed) & 0xFFFFFFFFFFFFFFFF, N, k, T, B, float(zero_padding_start_ratio), arr, len(ratios), float(max_av),
            0 if zero_padding else 1, kind, float(bump_param), av.data_ptr(), angle.data_ptr(), action.data_ptr(),
            r0.data_ptr(), torch.cuda.current_stream(dev).cuda_stream))
    if zero_padding and k > 2:
        from .ring_rnn_cuda import DRIVEN_ATTR
        setattr(action, DRIVEN_ATTR, (0, 1))      # by construction channels 2.. are identically zero
    return av, angle, action, r0


class FusedClipAdam:
    """clip_grad_norm_(params, max_norm) + Adam.step() in three launches for all parameter tensors.

    Same update as torch.optim.Adam (no weight decay, no amsgrad) after torch.nn.utils.clip_grad_norm_; state
    (exp_avg, exp_avg_sq, step) is kept per tensor as torch does.  `last_grad_norm` is a device scalar (the norm
    before clipping) that is only valid after the step has run on the stream; reading it synchronises.
    capturable=True keeps Adam's step number in a device counter that every step advances itself, so a training step
    recorded into a HIP graph goes on counting when the graph is replayed (the host-side `step_count` still counts
    the calls made from Python, not the replays)."""

    def __init__(self, params, lr=1e-3, betas=(0.9, 0.999), eps=1e-8, max_norm=1.0, capturable=False):
        self.params = [p for p in params if p.requires_grad]
        if not 1 <= len(self.params) <= 16:
            raise ValueError(f"FusedClipAdam handles 1..16 parameter tensors, got {len(self.params)}")
        for p in self.params:
            if not p.is_cuda or p.dtype != torch.float32 or not p.is_contiguous():
                raise TypeError("FusedClipAdam needs contiguous float32 GPU parameters")
        self.lr, self.betas, self.eps, self.max_norm = float(lr), (float(betas[0]), float(betas[1])), float(eps), float(max_norm)
        self.exp_avg = [torch.zeros_like(p) for p in self.params]
        self.exp_avg_sq = [torch.zeros_like(p) for p in self.params]
        self.step_count = 0
        self.step_counter = torch.zeros(1, dtype=torch.int32, device=self.params[0].device) if capturable else None
        n = len(self.params)
        self._numel = (ctypes.c_size_t * n)(*[p.numel() for p in self.params])
        lib = _lib.load()
        nbytes = lib.ringattr_clip_adam_workspace_bytes(n, self._numel)
        if nbytes == 0:
            _lib.check(1)
        self._ws = torch.empty(nbytes, dtype=torch.uint8, device=self.params[0].device)
        self._ws_bytes = nbytes
        total = sum(self._chunks())
        self.last_grad_norm = self._ws.view(torch.float32)[total:total + 1]

    def _chunks(self):
        return [(p.numel() + 4095) // 4096 for p in self.params]

    def zero_grad(self):
        for p in self.params:
            p.grad = None

    def step(self):
        grads = []
        for p in self.params:
            if p.grad is None:
                raise RuntimeError("FusedClipAdam.step(): a parameter has no gradient")
            if not p.grad.is_contiguous():
                p.grad = p.grad.contiguous()
            grads.append(p.grad)
        self.step_count += 1
        n = len(self.params)
        ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
        dev = self.params[0].device
        with torch.cuda.device(dev), torch.no_grad():
            lib, stream = _lib.load(), torch.cuda.current_stream(dev).cuda_stream
            common = (n, ptrs(self.params), ptrs(grads), ptrs(self.exp_avg), ptrs(self.exp_avg_sq), self._numel, self.lr,
                      self.betas[0], self.betas[1], self.eps, self.max_norm)
            if self.step_counter is not None:
                _lib.check(lib.ringattr_clip_adam_counted(*common, self.step_counter.data_ptr(), self._ws.data_ptr(),
                                                          self._ws_bytes, stream))
            else:
                _lib.check(lib.ringattr_clip_adam(*common, self.step_count, self._ws.data_ptr(), self._ws_bytes, stream))
