"""Fused decode + loss head: the training script's loss pair computed from bump_history in two HIP passes.

    total, cos_loss, amp_loss = ring_loss_pair(bump_history, target_angle, bump_weight=0.2)

equals, for bump_history [T,B,N] straight from `ring_rnn_cuda_func` and target_angle [B,T],

    bump = bump_history.permute(1, 0, 2); proj = bump @ W_delta7
    cos_loss = cosine_similarity_loss(proj / proj.max(dim=2, keepdim=True)[0], target_angle)
    amp_loss = bump_amplitude_loss(bump, target_amplitude)
    total = cos_loss + bump_weight * amp_loss

(root train_general_ring_no_gain.py:113-116, 324-330 and train/train_ring_attractor.py:190-220, 275-298 of the
reference), and is differentiable with respect to bump_history.  The torch chain makes about a dozen passes over
B*T*N values; this makes one forward and one backward.  A state that is identically zero gives NaN in the torch
chain (0/0 in the normalisation) and a finite loss here.
"""
from __future__ import annotations

import torch
from torch.autograd import Function

from . import _lib


def _check(name, t, shape, device):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    if not t.is_cuda or t.device != device:
        raise RuntimeError(f"{name} must be on {device} (got {t.device}); there is no CPU path")


class RingLossPair(Function):
    @staticmethod
    def forward(ctx, bump_history, target_angle, bump_weight, target_amplitude):
        if bump_history.dim() != 3:
            raise ValueError(f"bump_history must be [T, B, N], got {tuple(bump_history.shape)}")
        T, B, N = bump_history.shape
        dev = bump_history.device
        hist = bump_history.contiguous()
        angle = target_angle.contiguous()
        _check("bump_history", hist, (T, B, N), dev)
        _check("target_angle", angle, (B, T), dev)
        amp = None
        if target_amplitude is not None:
            amp = target_amplitude.reshape(-1).contiguous()
            _check("target_amplitude", amp, (B,), dev)
        lib = _lib.load()
        with torch.cuda.device(dev):
            nbytes = lib.ringattr_loss_workspace_bytes(N, T, B)
            if nbytes == 0:
                _lib.check(1)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            out = torch.empty(3, dtype=torch.float32, device=dev)
            _lib.check(lib.ringattr_loss_fwd(hist.data_ptr(), angle.data_ptr(), amp.data_ptr() if amp is not None else None,
                                             float(bump_weight), out.data_ptr(), N, T, B, ws.data_ptr(), nbytes,
                                             torch.cuda.current_stream(dev).cuda_stream))
        ctx.save_for_backward(hist, angle, ws, amp if amp is not None else torch.empty(0, device=dev))
        ctx.has_amp, ctx.bump_weight = amp is not None, float(bump_weight)
        ctx.mark_non_differentiable(out)          # the parts are returned for logging; total carries the gradient
        return out[0].clone(), out
        # (out[0] is cloned so that the differentiable result does not alias the logging tensor)

    @staticmethod
    def backward(ctx, grad_total, _grad_parts):
        hist, angle, ws, amp = ctx.saved_tensors
        T, B, N = hist.shape
        dev = hist.device
        grad = torch.empty_like(hist)
        up = grad_total.to(torch.float32).reshape(1).contiguous()
        lib = _lib.load()
        with torch.cuda.device(dev):
            _lib.check(lib.ringattr_loss_bwd(hist.data_ptr(), angle.data_ptr(), amp.data_ptr() if ctx.has_amp else None,
                                             ctx.bump_weight, up.data_ptr(), grad.data_ptr(), N, T, B, ws.data_ptr(),
                                             ws.numel(), torch.cuda.current_stream(dev).cuda_stream))
        return grad, None, None, None


def ring_loss_pair(bump_history, target_angle, bump_weight=0.2, target_amplitude=None):
    """Returns (total, cos_loss, amp_loss) as 0-dim tensors; only `total` is differentiable."""
    total, parts = RingLossPair.apply(bump_history, target_angle, bump_weight, target_amplitude)
    return total, parts[1], parts[2]
