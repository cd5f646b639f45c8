"""`fwd_cuda` / `bwd_cuda`: the two extension objects the operator calls, HIP-backed.

Mirrors the module-level interface of the reference loader cpp/rnn_cuda.py:59-91 and the keyword
signatures of its pybind modules (cpp/fwd.cpp:49-55, cpp/bwd.cpp:101-123):

    fwd_cuda.fwd(A=, Wa=, J0=, J1=, Wo=, r_init=, bump_history=, alpha=, activation_type=)
    bwd_cuda.bwd(grad_output=, A=, Wa=, J0=, J1=, Wo=, bump_history=, re_history=, r_init=,
                 grad_Wa=, grad_Wo=, alpha=, activation_type=, grad_r=, W_eff_temp=, grad_re_temp=,
                 grad_W_eff_temp_bf16=, A_t_temp_bf16=, grad_re_temp_T=, cublas_handle=)

Differences from the reference, all at the edges:
  * every tensor is checked for dtype float32, device and shape as well as contiguity (the
    reference checks contiguity only; a wrong dtype is silent garbage there);
  * the reference's workspace tensors and cublas_handle are accepted and ignored -- the scratch
    this implementation needs is sized by the library and taken from torch's caching allocator;
  * optional keywords `saved=` (forward: buffer to fill; backward: buffer to consume),
    `grad_r_init=` [B,N] and `grad_A=` [B,T,a_dim] (both overwritten, not accumulated) and `stream=`;
  * work goes to torch's CURRENT stream, not the legacy default stream;
  * importing this module needs no GPU; calling it does (RuntimeError otherwise).
"""
from __future__ import annotations

import torch

from . import _lib

_ACT_IDS = (0, 1, 2, 3)


def _contig(name, t):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")       # wording of cpp/fwd.cpp:31-35


def _f32_cuda(specs):
    """specs: (name, tensor, shape) triples.  Dtype and shape of every tensor are checked before any
    device check, so malformed calls are reported the same way with or without a GPU."""
    for name, t, shape in specs:
        _contig(name, t)
        if t.dtype != torch.float32:
            raise TypeError(f"{name} must be float32, got {t.dtype}")
        if tuple(t.shape) != tuple(shape):
            raise ValueError(f"{name} must have shape {tuple(shape)}, got {tuple(t.shape)}")
    device = specs[0][1].device
    for name, t, _ in specs:
        if not t.is_cuda:
            raise RuntimeError(f"{name} must be a GPU tensor (device {t.device}); there is no CPU path")
        if t.device != device:
            raise RuntimeError(f"{name} is on {t.device}, expected {device}")


def _scalar(name, v) -> float:
    if isinstance(v, torch.Tensor):
        if v.numel() != 1:
            raise TypeError(f"{name} must be a scalar (got a tensor of shape {tuple(v.shape)}); "
                            "the operator takes J0/J1 as floats (cpp/fwd.cpp:22-23)")
        return float(v.item())
    return float(v)


def _shapes(A, Wa):
    if A.dim() != 3:
        raise ValueError(f"A must be [batch, seq_len, a_dim], got {tuple(A.shape)}")
    if Wa.dim() != 3 or Wa.shape[1] != Wa.shape[2]:
        raise ValueError(f"Wa must be [a_dim, N, N], got {tuple(Wa.shape)}")
    B, T, k = A.shape
    if Wa.shape[0] != k:
        raise ValueError(f"Wa has {Wa.shape[0]} action matrices but A has a_dim {k}")
    return int(B), int(T), int(k), int(Wa.shape[1])


def _act(activation_type) -> int:
    a = int(activation_type)
    if a not in _ACT_IDS:
        raise ValueError(f"Invalid activation_type {activation_type}. Must be one of 0 relu, 1 gelu, 2 tanh, 3 silu.")
    return a


def _stream_ptr(stream, device):
    if stream is None:
        stream = torch.cuda.current_stream(device)
    return stream.cuda_stream if hasattr(stream, "cuda_stream") else int(stream)


def _ptr(t):
    return None if t is None else t.data_ptr()


def _workspace(nbytes, device, stream):
    """Scratch for one call, from torch's caching allocator.  The allocator hands a freed block back to later
    allocations on the stream it was ALLOCATED on (the current one) as soon as the tensor is dropped, which is at
    the end of the call, long before the kernels have run.  On the current stream that is safe (the next user's
    work is queued behind the kernels); when the caller passes another stream through `stream=`, the block is
    marked as in use on that stream too, so it is not recycled before the work queued there has finished."""
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    if stream is not None:
        s = stream if isinstance(stream, torch.cuda.Stream) else torch.cuda.ExternalStream(int(stream), device=device)
        if s != torch.cuda.current_stream(device):
            ws.record_stream(s)
    return ws


def saved_nbytes(N, a_dim, seq_len, batch_size) -> int:
    """Size of the opaque saved-activations buffer (uint8 elements)."""
    return int(_lib.load().ringattr_saved_bytes(N, a_dim, seq_len, batch_size))


class _Fwd:
    """Stand-in for the reference's `fwd` extension module (cpp/fwd.cpp:49-55)."""

    @staticmethod
    def fwd(A, Wa, J0, J1, Wo, r_init, bump_history, alpha, activation_type, saved=None, stream=None, loss=None):
        # loss (not in the reference): (target_angle [B,T], target_amplitude [B] or None, bump_weight, loss_out [3],
        # loss_workspace uint8) -- the loss head's forward runs in the same call (ringattr_fwd_loss)
        for name, t in (("A", A), ("Wa", Wa), ("Wo", Wo), ("r_init", r_init), ("bump_history", bump_history)):
            _contig(name, t)
        B, T, k, N = _shapes(A, Wa)
        act = _act(activation_type)
        J0, J1, alpha = _scalar("J0", J0), _scalar("J1", J1), _scalar("alpha", alpha)
        dev = A.device
        _f32_cuda([("A", A, (B, T, k)), ("Wa", Wa, (k, N, N)), ("Wo", Wo, (N, N)), ("r_init", r_init, (B, N)),
                   ("bump_history", bump_history, (T, B, N))])
        lib = _lib.load()
        if saved is not None:
            _contig("saved", saved)
            need = lib.ringattr_saved_bytes(N, k, T, B)
            if saved.dtype != torch.uint8 or saved.numel() < need or saved.device != dev:
                raise ValueError(f"saved must be a uint8 tensor of at least {need} bytes on {dev}")
        with torch.cuda.device(dev):
            ws_bytes = lib.ringattr_fwd_workspace_bytes(N, k, T, B)
            if ws_bytes == 0:
                _lib.check(1)
            ws = _workspace(ws_bytes, dev, stream)
            if loss is None:
                rc = lib.ringattr_fwd(_ptr(A), _ptr(Wa), J0, J1, _ptr(Wo), _ptr(r_init), _ptr(bump_history), alpha,
                                      N, k, T, B, act, _ptr(saved), _ptr(ws), ws_bytes, _stream_ptr(stream, dev))
            else:
                angle, amp, bump_weight, loss_out, lws = loss
                rc = lib.ringattr_fwd_loss(_ptr(A), _ptr(Wa), J0, J1, _ptr(Wo), _ptr(r_init), _ptr(bump_history), alpha,
                                           N, k, T, B, act, _ptr(saved), _ptr(ws), ws_bytes, _ptr(angle), _ptr(amp),
                                           float(bump_weight), _ptr(loss_out), _ptr(lws), lws.numel(),
                                           _stream_ptr(stream, dev))
        _lib.check(rc)
        return None


class _Bwd:
    """Stand-in for the reference's `bwd` extension module (cpp/bwd.cpp:101-123)."""

    @staticmethod
    def bwd(grad_output, A, Wa, J0, J1, Wo, bump_history, re_history=None, r_init=None, grad_Wa=None, grad_Wo=None,
            alpha=None, activation_type=None, grad_r=None, W_eff_temp=None, grad_re_temp=None,
            grad_W_eff_temp_bf16=None, A_t_temp_bf16=None, grad_re_temp_T=None, cublas_handle=None,
            saved=None, grad_r_init=None, grad_A=None, stream=None, loss_workspace=None, loss_upstream=None,
            accumulate=True):
        # accumulate=True adds into grad_Wa / grad_Wo as the reference does (its caller zeroes them,
        # cpp/ring_rnn_cuda.py:98-99); False overwrites them, so they may be uninitialised.
        # loss_workspace (what the fused loss head's forward filled for this bump_history) in place of grad_output:
        # the gradient of the loss pair is then formed inside the backward, scaled by loss_upstream (1-element tensor)
        if (grad_output is None) == (loss_workspace is None):
            raise TypeError("bwd() needs exactly one of grad_output and loss_workspace")
        if grad_output is not None:
            _contig("grad_output", grad_output)
        for name, t in (("A", A), ("Wa", Wa), ("Wo", Wo),
                        ("bump_history", bump_history), ("r_init", r_init), ("grad_Wa", grad_Wa), ("grad_Wo", grad_Wo)):
            _contig(name, t)
        # the reference's workspaces: contiguity is all it ever checked (cpp/bwd.cpp:66-72); unused here
        for name, t in (("re_history", re_history), ("grad_r", grad_r), ("W_eff_temp", W_eff_temp),
                        ("grad_re_temp", grad_re_temp), ("grad_W_eff_temp_bf16", grad_W_eff_temp_bf16),
                        ("A_t_temp_bf16", A_t_temp_bf16), ("grad_re_temp_T", grad_re_temp_T)):
            if t is not None:
                _contig(name, t)
        if alpha is None or activation_type is None:
            raise TypeError("bwd() needs alpha and activation_type")
        B, T, k, N = _shapes(A, Wa)
        act = _act(activation_type)
        J0, J1, alpha = _scalar("J0", J0), _scalar("J1", J1), _scalar("alpha", alpha)
        dev = A.device
        specs = [("A", A, (B, T, k)), ("Wa", Wa, (k, N, N)),
                 ("Wo", Wo, (N, N)), ("bump_history", bump_history, (T, B, N)), ("r_init", r_init, (B, N)),
                 ("grad_Wa", grad_Wa, (k, N, N)), ("grad_Wo", grad_Wo, (N, N))]
        if grad_output is not None:
            specs.append(("grad_output", grad_output, (T, B, N)))
        if loss_upstream is not None:
            specs.append(("loss_upstream", loss_upstream, (1,)))
        if grad_r_init is not None:
            specs.append(("grad_r_init", grad_r_init, (B, N)))
        if grad_A is not None:
            specs.append(("grad_A", grad_A, (B, T, k)))
        _f32_cuda(specs)
        lib = _lib.load()
        if saved is not None:
            _contig("saved", saved)
            need = lib.ringattr_saved_bytes(N, k, T, B)
            if saved.dtype != torch.uint8 or saved.numel() < need or saved.device != dev:
                raise ValueError(f"saved must be a uint8 tensor of at least {need} bytes on {dev}")
        if loss_workspace is not None:
            _contig("loss_workspace", loss_workspace)
            need = lib.ringattr_loss_workspace_bytes(N, T, B)
            if need == 0:
                _lib.check(1)
            if loss_workspace.dtype != torch.uint8 or loss_workspace.numel() < need or loss_workspace.device != dev:
                raise ValueError(f"loss_workspace must be a uint8 tensor of at least {need} bytes on {dev}")
            with torch.cuda.device(dev):
                ws_bytes = lib.ringattr_bwd_workspace_bytes(N, k, T, B, 1 if saved is not None else 0)
                if ws_bytes == 0:
                    _lib.check(1)
                ws = _workspace(ws_bytes, dev, stream)
                rc = lib.ringattr_bwd_loss(_ptr(loss_workspace), _ptr(loss_upstream), _ptr(A), _ptr(Wa), J0, J1, _ptr(Wo),
                                           _ptr(bump_history), _ptr(r_init), _ptr(grad_Wa), _ptr(grad_Wo), alpha, N, k, T,
                                           B, act, 1 if accumulate else 0, _ptr(saved), _ptr(grad_A), _ptr(grad_r_init), _ptr(ws), ws_bytes,
                                           _stream_ptr(stream, dev))
            _lib.check(rc)
            return None
        with torch.cuda.device(dev):
            ws_bytes = lib.ringattr_bwd_workspace_bytes(N, k, T, B, 1 if saved is not None else 0)
            if ws_bytes == 0:
                _lib.check(1)
            ws = _workspace(ws_bytes, dev, stream)
            rc = lib.ringattr_bwd(_ptr(grad_output), _ptr(A), _ptr(Wa), J0, J1, _ptr(Wo), _ptr(bump_history),
                                  _ptr(r_init), _ptr(grad_Wa), _ptr(grad_Wo), alpha, N, k, T, B, act,
                                  1 if accumulate else 0, _ptr(saved), _ptr(grad_A), _ptr(grad_r_init), _ptr(ws), ws_bytes,
                                  _stream_ptr(stream, dev))
        _lib.check(rc)
        return None


fwd_cuda = _Fwd()
bwd_cuda = _Bwd()
