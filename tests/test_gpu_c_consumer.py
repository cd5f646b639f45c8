"""The C ABI from plain C: tests/c_abi/ring_c_consumer.c (C99, built by the host C compiler against
include/ringattr.h; no Python, torch or C++ on its side) allocates device buffers through the HIP runtime, queries the
workspace sizes, calls ringattr_fwd / ringattr_bwd and checks history, dL/d r_init and dL/dWo against a closed form.
It is built as a shared object so that it can run inside this process."""
import ctypes
import os

import pytest

pytestmark = pytest.mark.gpu

LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "c_abi", "libring_c_consumer.so")


@pytest.mark.parametrize("N,B,T", [(64, 16, 6), (256, 32, 6), (200, 21, 5), (640, 16, 4)],
                         ids=["streaming", "resident", "resident_masked", "step_per_launch"])
def test_plain_c_caller(N, B, T, gpu_device):
    from rnn_train_ring_attractor_amd import _lib
    print(f"[case] plain-C caller N={N} B={B} T={T}", flush=True)
    _lib.load()                                   # (also resolves the consumer's dependency on libringattr.so)
    if not os.path.exists(LIB):
        pytest.fail(f"{LIB} is missing: run `python -m rnn_train_ring_attractor_amd.build` first")
    consumer = ctypes.CDLL(LIB)
    consumer.test_c_consumer.restype = ctypes.c_int
    consumer.test_c_consumer.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_char_p, ctypes.c_size_t]
    msg = ctypes.create_string_buffer(512)
    rc = consumer.test_c_consumer(N, B, T, msg, len(msg))
    print(f"[measured] {msg.value.decode()}", flush=True)
    assert rc == 0, msg.value.decode()


def test_reference_side_binding_from_the_integration_guide(gpu_device, monkeypatch, default_kernels):
    """The ctypes stub that the integration guide proposes for the reference's cpp/rnn_cuda.py, executed verbatim from
    the guide: its fwd_cuda.fwd / bwd_cuda.bwd (reference keyword names, no saved buffer, gradients added to) give the
    history of the packaged operator bit for bit and its gradients to rounding."""
    import re

    import numpy as np
    import torch

    from oracle import ring_oracle as O
    from rnn_train_ring_attractor_amd import build as _build, ring_rnn_cuda_func
    from tests.ring_cases import make_problem
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    text = open(os.path.join(root, "INTEGRATION.md")).read()
    code = re.search(r"```python\n(# cpp/rnn_cuda.py \(reference side\).*?)```", text, re.S).group(1)
    monkeypatch.setenv("RINGATTR_LIB", _build.LIB_PATH)
    ns = {}
    exec(compile(code, "INTEGRATION.md:stub", "exec"), ns)
    print("[case] integration-guide stub N=256 B=48 T=12 gelu", flush=True)
    B, T, k, N = 48, 12, 2, 256
    p = make_problem(31, B, T, k, N)
    t = lambda x: torch.tensor(x, device=gpu_device)
    A, Wa, Wo, r0, G = t(p["A"]), t(p["Wa"]), t(p["Wo"]), t(p["r0"]), t(p["G"])
    hist = torch.empty(T, B, N, device=gpu_device)
    ns["fwd_cuda"].fwd(A=A, Wa=Wa, J0=-0.1, J1=0.1, Wo=Wo, r_init=r0, bump_history=hist, alpha=0.15, activation_type=1)
    gWa, gWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
    ns["bwd_cuda"].bwd(grad_output=G, A=A, Wa=Wa, J0=-0.1, J1=0.1, Wo=Wo, bump_history=hist, re_history=None, r_init=r0,
                       grad_Wa=gWa, grad_Wo=gWo, alpha=0.15, activation_type=1, grad_r=None, W_eff_temp=None)
    Wa2, Wo2 = Wa.clone().requires_grad_(True), Wo.clone().requires_grad_(True)
    want = ring_rnn_cuda_func(A, Wa2, -0.1, 0.1, Wo2, r0, 0.15, "gelu")
    want.backward(G)
    torch.cuda.synchronize()
    assert torch.equal(hist, want.detach())
    assert O.max_rel_err(gWo.cpu().numpy(), Wo2.grad.cpu().numpy()) <= 2e-3
    assert O.max_rel_err(gWa.cpu().numpy(), Wa2.grad.cpu().numpy()) <= 2e-3
    assert np.isfinite(gWa.cpu().numpy()).all()
