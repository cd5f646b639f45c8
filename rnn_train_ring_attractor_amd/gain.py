"""Gain networks of the action signal as one HIP operator (forward and backward).

`ring_gain_func(base_signal, params)` evaluates, per channel c, the reference models' gain network
nn.Sequential(Linear(1,h), GELU, Linear(h,1), Softplus) on |x| and returns x * gain (train/train_ring_attractor.py:70-79,
136-146; train/train_general_ring_attractor.py:38-46, 99-109).  `params` is [k, 3h+1] = per channel [w1 | b1 | w2 | b2];
`pack_gain_nets` builds it from the nn.Sequential modules with differentiable torch ops, so autograd carries the
operator's parameter gradients back into the modules.
"""
from __future__ import annotations

import torch
from torch.autograd import Function

from . import _lib


def pack_gain_nets(nets):
    """[k, 3h+1] parameter block of a list of nn.Sequential(Linear(1,h), GELU, Linear(h,1), Softplus)."""
    rows = []
    for net in nets:
        lin1, lin2 = net[0], net[2]
        rows.append(torch.cat([lin1.weight.reshape(-1), lin1.bias.reshape(-1), lin2.weight.reshape(-1),
                               lin2.bias.reshape(-1)]))
    return torch.stack(rows)


def _check(name, t, shape):
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor (device {t.device}); there is no CPU path")
    if t.dtype != torch.float32:
        raise TypeError(f"{name} must be float32, got {t.dtype}")
    if tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")


class RingGainFunc(Function):
    @staticmethod
    def forward(ctx, base_signal, params):
        if base_signal.dim() != 3:
            raise ValueError(f"base_signal must be [batch, seq_len, a_dim], got {tuple(base_signal.shape)}")
        B, T, k = base_signal.shape
        if params.dim() != 2 or params.shape[0] != k or (params.shape[1] - 1) % 3 != 0:
            raise ValueError(f"params must be [a_dim, 3*hidden+1] with a_dim = {k}, got {tuple(params.shape)}")
        h = (params.shape[1] - 1) // 3
        x, prm = base_signal.contiguous(), params.contiguous()
        _check("base_signal", x, (B, T, k))
        _check("params", prm, (k, 3 * h + 1))
        lib = _lib.load()
        out = torch.empty_like(x)
        with torch.cuda.device(x.device):
            _lib.check(lib.ringattr_gain_fwd(x.data_ptr(), prm.data_ptr(), out.data_ptr(), k, h, T, B,
                                             torch.cuda.current_stream(x.device).cuda_stream))
        ctx.save_for_backward(x, prm)
        ctx.dims = (B, T, k, h)
        return out

    @staticmethod
    def backward(ctx, grad_out):
        x, prm = ctx.saved_tensors
        B, T, k, h = ctx.dims
        lib = _lib.load()
        g = grad_out.contiguous()
        grad_prm = torch.empty_like(prm)
        grad_x = torch.empty_like(x) if ctx.needs_input_grad[0] else None
        with torch.cuda.device(x.device):
            nbytes = lib.ringattr_gain_workspace_bytes(k, h, T, B)
            if nbytes == 0:
                _lib.check(1)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
            _lib.check(lib.ringattr_gain_bwd(x.data_ptr(), prm.data_ptr(), g.data_ptr(), grad_prm.data_ptr(),
                                             grad_x.data_ptr() if grad_x is not None else None, k, h, T, B,
                                             ws.data_ptr(), nbytes, torch.cuda.current_stream(x.device).cuda_stream))
        return grad_x, grad_prm


def ring_gain_func(base_signal, params):
    """[B,T,k] base signal, [k,3h+1] packed gain-network parameters -> [B,T,k] gated action signal."""
    return RingGainFunc.apply(base_signal, params)
