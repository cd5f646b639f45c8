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
from .rnn_cuda import fwd_cuda, bwd_cuda, saved_nbytes


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


class RingRnnLossFunc(Function):
    """The time loop and the loss pair as one differentiable operator: forward = `ring_rnn_cuda_func` followed by
    the fused loss head; backward = one library call in which the BPTT kernel forms the loss gradient itself
    (weight-resident geometry) instead of reading a [T,B,N] grad_output tensor that a loss backward wrote."""

    @staticmethod
    def forward(ctx, action_signal, Wa, J0, J1, Wo, r_init, alpha, activation_name, target_angle, bump_weight,
                target_amplitude, grad_mode=None):
        from .ring_rnn_cuda import _activation_id
        act = _activation_id(activation_name)
        B, T, k = action_signal.shape
        N = Wa.shape[1]
        dev = action_signal.device
        A, Wa_c, Wo_c, r0 = action_signal.contiguous(), Wa.contiguous(), Wo.contiguous(), r_init.contiguous()
        angle = target_angle.contiguous()
        _check("target_angle", angle, (B, T), dev)
        amp = None
        if target_amplitude is not None:
            amp = target_amplitude.reshape(-1).contiguous()
            _check("target_amplitude", amp, (B,), dev)
        hist = torch.empty(T, B, N, device=dev, dtype=A.dtype)
        # autograd switches gradient mode off in here and needs_input_grad stays True under no_grad(): the wrapper says
        needs_grad = grad_mode is not False and any(ctx.needs_input_grad[i] for i in (0, 1, 4, 5))
        ctx.extra_inputs = 0 if grad_mode is None else 1
        saved = torch.empty(saved_nbytes(N, k, T, B), dtype=torch.uint8, device=dev) if needs_grad else None
        lib = _lib.load()
        with torch.cuda.device(dev):
            nbytes = lib.ringattr_loss_workspace_bytes(N, T, B)
            if nbytes == 0:
                _lib.check(1)
            lws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            out = torch.empty(3, dtype=torch.float32, device=dev)
        # time loop and loss head in one call: the weight-resident forward kernel forms the loss's row sums itself
        fwd_cuda.fwd(A=A, Wa=Wa_c, J0=J0, J1=J1, Wo=Wo_c, r_init=r0, bump_history=hist, alpha=alpha,
                     activation_type=act, saved=saved, loss=(angle, amp, float(bump_weight), out, lws))
        ctx.save_for_backward(A, Wa_c, Wo_c, hist, r0, saved, lws, angle, amp)
        ctx.J0, ctx.J1, ctx.alpha, ctx.act, ctx.bump_weight = J0, J1, alpha, act, float(bump_weight)
        ctx.mark_non_differentiable(out, hist)
        ctx.set_materialize_grads(False)         # no [T,B,N] tensor of zeros for the history's unused gradient
        return out[0].clone(), out, hist

    @staticmethod
    def backward(ctx, grad_total, _grad_parts, _grad_hist):
        A, Wa, Wo, hist, r0, saved, lws, angle, amp = ctx.saved_tensors
        grad_Wa, grad_Wo = torch.empty_like(Wa), torch.empty_like(Wo)    # written, not accumulated into
        grad_A = torch.empty_like(A) if ctx.needs_input_grad[0] else None
        grad_r0 = torch.empty_like(r0) if ctx.needs_input_grad[5] else None
        if grad_total is None:                   # (gradients are not materialised: the total went unused)
            grad_total = torch.zeros((), device=hist.device)
        up = grad_total.to(torch.float32).reshape(1).contiguous()
        T, B, N = hist.shape
        lib = _lib.load()
        if not lib.ringattr_bwd_loss_available(N, A.shape[2], T, B):
            # the step-per-launch kernels (wide rings) read grad_output: the loss head writes it, the backward reads it
            grad_hist = torch.empty_like(hist)
            dev = hist.device
            with torch.cuda.device(dev):
                _lib.check(lib.ringattr_loss_bwd(hist.data_ptr(), angle.data_ptr(), amp.data_ptr() if amp is not None else None,
                                                 ctx.bump_weight, up.data_ptr(), grad_hist.data_ptr(), N, T, B,
                                                 lws.data_ptr(), lws.numel(), torch.cuda.current_stream(dev).cuda_stream))
            bwd_cuda.bwd(grad_output=grad_hist, A=A, Wa=Wa, J0=ctx.J0, J1=ctx.J1, Wo=Wo, bump_history=hist, r_init=r0,
                         grad_Wa=grad_Wa, grad_Wo=grad_Wo, alpha=ctx.alpha, activation_type=ctx.act, saved=saved,
                         grad_A=grad_A, grad_r_init=grad_r0, accumulate=False)
            return (grad_A, grad_Wa, None, None, grad_Wo, grad_r0, None, None, None, None, None) + (None,) * ctx.extra_inputs
        bwd_cuda.bwd(grad_output=None, A=A, Wa=Wa, J0=ctx.J0, J1=ctx.J1, Wo=Wo, bump_history=hist, r_init=r0,
                     grad_Wa=grad_Wa, grad_Wo=grad_Wo, alpha=ctx.alpha, activation_type=ctx.act, saved=saved,
                     grad_A=grad_A, grad_r_init=grad_r0, loss_workspace=lws, loss_upstream=up, accumulate=False)
        return (grad_A, grad_Wa, None, None, grad_Wo, grad_r0, None, None, None, None, None) + (None,) * ctx.extra_inputs


def ring_rnn_loss_func(action_signal, Wa, J0, J1, Wo, r_init, alpha, activation, target_angle, bump_weight=0.2,
                       target_amplitude=None, driven_channels=None):
    """`ring_rnn_cuda_func(...)` and `ring_loss_pair(...)` in one operator.

    Returns (total, cos_loss, amp_loss, bump_history); only `total` is differentiable (w.r.t. Wa, Wo and, when they
    require it, action_signal and r_init); bump_history [T,B,N] is returned detached for decoding and logging."""
    from .ring_rnn_cuda import _silent_channel_view
    compact = _silent_channel_view(action_signal, Wa, driven_channels)
    if compact is not None:
        action_signal, Wa = compact
    total, parts, hist = RingRnnLossFunc.apply(action_signal, Wa, J0, J1, Wo, r_init, alpha, activation, target_angle,
                                               bump_weight, target_amplitude, torch.is_grad_enabled())
    return total, parts[1], parts[2], hist
