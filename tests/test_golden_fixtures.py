"""Committed regression fixtures (tests/golden/ring_fixtures.npz, written by tests/golden/make_fixtures.py):
the oracle must keep reproducing them exactly, and the HIP path must meet them within the parity tolerances."""
import os

import numpy as np
import pytest

from oracle import ring_oracle as O
from tests.golden.make_fixtures import CASES

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ring_fixtures.npz")


def _case(name):
    z = np.load(PATH, allow_pickle=False)
    return {k.split("/", 1)[1]: z[k] for k in z.files if k.startswith(name + "/")}


@pytest.mark.parametrize("name", sorted(CASES))
def test_oracle_reproduces_fixture(name):
    f, (_, B, T, k, N, act, J0, J1) = _case(name), CASES[name]
    assert f["hist"].shape == (T, B, N) and f["grad_A"].shape == (B, T, k)
    hist, _ = O.forward_dense(f["A"], f["Wa"], J0, J1, f["Wo"], f["r0"], 0.15, act)
    np.testing.assert_allclose(hist, f["hist"], rtol=0, atol=1e-12)
    # the per-sample-W_eff formulation of the reference's PyTorch path gives the same numbers
    np.testing.assert_allclose(O.forward_per_sample(f["A"], f["Wa"], J0, J1, f["Wo"], f["r0"], 0.15, act)[0], f["hist"],
                               rtol=0, atol=1e-10)
    g = O.backward_dense(f["G"], f["A"], f["Wa"], J0, J1, f["Wo"], hist, f["r0"], 0.15, act)
    for key in ("grad_Wo", "grad_Wa", "grad_A", "grad_r_init"):
        np.testing.assert_allclose(g[key], f[key], rtol=0, atol=1e-11)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(CASES))
def test_hip_path_meets_fixture(name, gpu_device):
    import torch
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    f, (_, B, T, k, N, act, J0, J1) = _case(name), CASES[name]
    print(f"[case] fixture {name}", flush=True)
    t = lambda x: torch.tensor(x, device=gpu_device)
    A, r0 = t(f["A"]).requires_grad_(True), t(f["r0"]).requires_grad_(True)
    Wa, Wo = t(f["Wa"]).requires_grad_(True), t(f["Wo"]).requires_grad_(True)
    hist = ring_rnn_cuda_func(A, Wa, J0, J1, Wo, r0, 0.15, act)
    hist.backward(t(f["G"]))
    torch.cuda.synchronize()
    assert O.max_rel_err(hist.detach().cpu().numpy(), f["hist"]) <= 1e-2
    smooth = act != "relu"          # relu: operand rounding flips derivative kinks, entry-wise bound does not apply
    for key, got in (("grad_Wo", Wo.grad), ("grad_Wa", Wa.grad), ("grad_A", A.grad), ("grad_r_init", r0.grad)):
        got = got.cpu().numpy()
        assert O.cosine(got, f[key]) >= 0.999, key
        if smooth:
            assert O.max_rel_err(got, f[key]) <= 2e-2, key
