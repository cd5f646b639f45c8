"""Host-only checks of the drop-in boundary: the C-ABI library loads and exports every symbol the
header declares, argument validation returns error codes / raises Python exceptions (never exits),
and the workspace-size queries are consistent.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

from rnn_train_ring_attractor_amd import _lib, bwd_cuda, fwd_cuda, ring_rnn_cuda_func
from rnn_train_ring_attractor_amd import rnn_cuda

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _header_symbols():
    text = open(os.path.join(ROOT, "include", "ringattr.h")).read()
    return sorted(set(re.findall(r"RINGATTR_API\s+[\w\s\*]+?\b(\w+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _header_symbols()
    assert {"ringattr_fwd", "ringattr_bwd", "fwd_cuda", "bwd_cuda", "ringattr_saved_bytes", "ringattr_loss_fwd",
            "ringattr_loss_bwd", "ringattr_loss_workspace_bytes", "ringattr_bwd_loss"} <= set(names)
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(_lib.PROTOTYPES) == names          # the ctypes table and the header agree
    assert lib.ringattr_version() >= 1000


def test_size_queries():
    lib = _lib.load()
    N, k, T, B = 256, 2, 120, 4096
    saved = lib.ringattr_saved_bytes(N, k, T, B)
    wpack = 3 * N * N * 2                                              # one bf16 copy of [Wo|Wa0|Wa1]
    assert saved == 2 * T * B * N * 2 + wpack                          # fp16 F' + bf16 r_prev [T,B,N] + transposed weights
    assert lib.ringattr_fwd_workspace_bytes(N, k, T, B) == 3 * N * N * 2
    with_saved = lib.ringattr_bwd_workspace_bytes(N, k, T, B, 1)
    without = lib.ringattr_bwd_workspace_bytes(N, k, T, B, 0)
    assert without - with_saved == saved                               # rebuilt F' and r_prev copy + forward weight pack
    # padding: N=120 -> 128 neurons, B=64 -> 4 batch tiles; odd T rounds the paired buffer up
    assert lib.ringattr_saved_bytes(120, 2, 7, 64) == (7 + 8) * 64 * 128 * 2 + 3 * 128 * 128 * 2
    assert lib.ringattr_saved_bytes(0, 2, 7, 64) == 0 and "positive" in _lib.last_error()
    # 512 < N <= 2048 pads to a multiple of 512 neurons (step-per-launch kernels); beyond that nothing runs
    assert lib.ringattr_saved_bytes(513, 2, 8, 64) == 2 * 8 * 64 * 1024 * 2 + 3 * 1024 * 1024 * 2
    assert lib.ringattr_saved_bytes(2049, 2, 7, 64) == 0 and "2048" in _lib.last_error()


def test_c_abi_rejects_bad_arguments_with_codes_not_exit():
    lib = _lib.load()
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    p = (p + 255) // 256 * 256
    ok_args = [p, p, 0.0, 1.0, p, p, p, 0.15, 64, 2, 4, 16]
    assert lib.ringattr_fwd(*ok_args, 7, None, p, 1 << 20, None) == 1 and "activation_type" in _lib.last_error()
    assert lib.ringattr_fwd(None, *ok_args[1:], 0, None, p, 1 << 20, None) == 1 and "null" in _lib.last_error()
    assert lib.ringattr_fwd(p + 4, *ok_args[1:], 0, None, p, 1 << 20, None) == 1 and "aligned" in _lib.last_error()
    assert lib.ringattr_fwd(*ok_args, 0, None, p, 16, None) == 2 and "workspace" in _lib.last_error()
    assert lib.ringattr_fwd(*ok_args, 0, None, None, 0, None) == 2
    bad_shape = list(ok_args)
    bad_shape[9] = 0                                                    # a_dim
    assert lib.ringattr_fwd(*bad_shape, 0, None, p, 1 << 20, None) == 1
    bwd_args = [p, p, p, 0.0, 1.0, p, p, p, p, p, 0.15, 64, 2, 4, 16, 0, 1]
    assert lib.ringattr_bwd(*bwd_args, None, None, None, p, 16, None) == 2
    wide = list(bwd_args)
    wide[12] = 64                                                       # a_dim beyond what the grad_A path stages in LDS
    assert lib.ringattr_bwd(*wide, None, p, None, p, 1 << 30, None) == 1 and "grad_A" in _lib.last_error()
    assert lib.ringattr_bwd(*bwd_args, None, p + 4, None, p, 1 << 30, None) == 1 and "aligned" in _lib.last_error()
    assert lib.ringattr_profile_read(None, None) == 1
    # the entry point with the built-in scratch rejects shapes whose packed weights exceed it, before any GPU call
    assert lib.ringattr_fwd_noalloc(p, p, 0.0, 1.0, p, p, p, 0.15, 512, 8, 4, 16, 0, None, None) == 2
    assert "built-in scratch" in _lib.last_error()
    assert lib.ringattr_fwd_noalloc(p, p, 0.0, 1.0, p, p, p, 0.15, 64, 2, 4, 16, 9, None, None) == 1
    # forward + loss head in one call: the loss arguments are checked before the time loop is touched
    fl = ok_args + [0, None, p, 1 << 20]
    assert lib.ringattr_fwd_loss(*fl, None, None, 0.2, p, p, 1 << 20, None) == 1 and "null" in _lib.last_error()
    assert lib.ringattr_fwd_loss(*fl, p, None, 0.2, p, p, 16, None) == 2 and "loss workspace" in _lib.last_error()
    assert lib.ringattr_fwd_loss(*fl, p, None, 0.2, p, p + 4, 1 << 20, None) == 1 and "aligned" in _lib.last_error()
    # clip + Adam: host-counted steps start at 1; the device-counted variant needs its counter
    one = (ctypes.c_void_p * 1)(p)
    numel = (ctypes.c_size_t * 1)(16)
    adam = [1, one, one, one, one, numel, 1e-3, 0.9, 0.999, 1e-8, 1.0]
    assert lib.ringattr_clip_adam(*adam, 0, p, 1 << 12, None) == 1 and "counts from 1" in _lib.last_error()
    assert lib.ringattr_clip_adam_counted(*adam, None, p, 1 << 12, None) == 1 and "step counter" in _lib.last_error()
    assert lib.ringattr_clip_adam_counted(*adam, p + 2, p, 1 << 12, None) == 1
    assert lib.ringattr_clip_adam_counted(*adam, p, p, 8, None) == 2 and "workspace" in _lib.last_error()
    with pytest.raises(ValueError):
        _lib.check(1)
    with pytest.raises(RuntimeError):
        _lib.check(3)


def _cpu_problem(B=4, T=3, k=2, N=8):
    return dict(A=torch.zeros(B, T, k), Wa=torch.zeros(k, N, N), Wo=torch.zeros(N, N), r_init=torch.zeros(B, N),
                bump_history=torch.zeros(T, B, N))


def test_python_binding_validation():
    kw = _cpu_problem()
    common = dict(J0=-0.1, J1=0.1, alpha=0.15, activation_type=0)
    with pytest.raises(RuntimeError, match="GPU tensor"):               # there is no CPU path
        fwd_cuda.fwd(**kw, **common)
    bad = dict(kw, A=kw["A"].transpose(0, 1))
    with pytest.raises(RuntimeError, match="A must be contiguous"):     # the reference's TORCH_CHECK wording
        fwd_cuda.fwd(**bad, **common)
    with pytest.raises(TypeError, match="float32"):
        fwd_cuda.fwd(**dict(kw, Wo=kw["Wo"].double()), **common)
    with pytest.raises(ValueError, match="shape"):
        fwd_cuda.fwd(**dict(kw, r_init=torch.zeros(4, 9)), **common)
    with pytest.raises(ValueError, match="action matrices"):
        fwd_cuda.fwd(**dict(kw, Wa=torch.zeros(3, 8, 8)), **common)
    with pytest.raises(ValueError, match="activation_type"):
        fwd_cuda.fwd(**kw, J0=0.0, J1=1.0, alpha=0.15, activation_type=9)
    with pytest.raises(TypeError, match="scalar"):
        fwd_cuda.fwd(**kw, J0=torch.zeros(8, 8), J1=1.0, alpha=0.15, activation_type=0)
    with pytest.raises(TypeError):
        bwd_cuda.bwd(grad_output=kw["bump_history"], A=kw["A"], Wa=kw["Wa"], J0=0.0, J1=1.0, Wo=kw["Wo"],
                     bump_history=kw["bump_history"], r_init=kw["r_init"], grad_Wa=kw["Wa"], grad_Wo=kw["Wo"])
    with pytest.raises(RuntimeError, match="grad_r must be contiguous"):
        bwd_cuda.bwd(grad_output=kw["bump_history"], A=kw["A"], Wa=kw["Wa"], J0=0.0, J1=1.0, Wo=kw["Wo"],
                     bump_history=kw["bump_history"], r_init=kw["r_init"], grad_Wa=kw["Wa"].clone(),
                     grad_Wo=kw["Wo"].clone(), alpha=0.15, activation_type=0, grad_r=torch.zeros(8, 4).t())


def test_operator_rejects_unknown_activation_before_touching_the_gpu():
    kw = _cpu_problem()
    with pytest.raises(ValueError, match="Invalid activation 'sigmoid'"):
        ring_rnn_cuda_func(kw["A"], kw["Wa"], -0.1, 0.1, kw["Wo"], kw["r_init"], 0.15, "sigmoid")


def test_saved_buffer_size_helper_matches_library():
    assert rnn_cuda.saved_nbytes(256, 2, 120, 4096) == _lib.load().ringattr_saved_bytes(256, 2, 120, 4096)


def test_generator_leading_zero_count_is_pythons_over_a_grid():
    """The device generator's count of leading zero steps is int(seq_len * ratio) with the product in double
    precision, as the reference's Python forms it (utils/generate_av_integration_data.py:21).  A float32 product is
    off by one for some pairs (seq_len = 180, ratio 0.35: 63 against 62; ratio 0.7 at seq_len = 10: 6 against 7), so
    the library takes the ratio as a double and the count is checked here against Python's own over a grid, and
    against the host generator's output (host.generate_av_integration_data_ultra_fast, the reference's construction)."""
    import numpy as np
    import torch
    from rnn_train_ring_attractor_amd import _lib, host
    lib = _lib.load()
    ratios = [0.0, 0.01, 0.05, 0.1, 0.15, 0.2, 0.3, 0.35, 0.5, 0.7, 0.9, 1.0]
    float_product_differs = 0
    for ratio in ratios:
        for T in range(1, 4097):
            want = int(T * ratio)
            assert lib.ringattr_generator_initial_zeros(T, ratio) == want, (T, ratio)
            float_product_differs += int(int(np.float32(T) * np.float32(ratio)) != want)
    assert float_product_differs > 0          # the grid contains the pairs a float product gets wrong
    assert lib.ringattr_generator_initial_zeros(180, 0.35) == 62 and lib.ringattr_generator_initial_zeros(10, 0.7) == 7
    assert lib.ringattr_generator_initial_zeros(0, 0.1) == -1 and lib.ringattr_generator_initial_zeros(10, 1.5) == -1
    torch.manual_seed(0)
    for T, ratio in ((180, 0.35), (10, 0.7), (120, 0.1), (77, 0.3)):
        av, _ = host.generate_av_integration_data_ultra_fast(64, T, ratio, [0.0])     # ratio 0: every later step drawn
        n0 = lib.ringattr_generator_initial_zeros(T, ratio)
        assert torch.all(av[:, :n0] == 0)
        assert torch.all(av[:, n0:] != 0)


def test_weight_gradient_segment_count(monkeypatch):
    """Host arithmetic of the weight-gradient kernel's time segments: at most RINGATTR_DW_SEGMENT (default 640) K
    chunks of 32 samples per workgroup and launch, whole time-step pairs per segment."""
    from rnn_train_ring_attractor_amd import _lib
    lib = _lib.load()
    monkeypatch.delenv("RINGATTR_DW_SEGMENT", raising=False)
    assert lib.ringattr_dw_segments(256, 2, 120, 4096) == 1          # 240 chunks per workgroup: one launch
    assert lib.ringattr_dw_segments(512, 2, 512, 8192) == 13         # 8192 chunks per workgroup: 20 pairs per segment
    assert lib.ringattr_dw_segments(1024, 2, 120, 2048) == 3
    assert lib.ringattr_dw_segments(120, 2, 120, 64) == 1            # not the tiled kernel
    monkeypatch.setenv("RINGATTR_DW_SEGMENT", "0")
    assert lib.ringattr_dw_segments(512, 2, 512, 8192) == 1
    monkeypatch.setenv("RINGATTR_DW_SEGMENT", "1")
    assert lib.ringattr_dw_segments(256, 2, 33, 256) == 5            # 64 splits x 1 chunk = 4 of the 17 time-step pairs per segment
    assert lib.ringattr_dw_segments(4096, 2, 8, 16) == -1
