"""Fused decode + loss head (ringattr_loss_fwd / ringattr_loss_bwd) against the fp64 oracle, whose rank-two form is
itself pinned against the reference's literal chain of tensor ops and its autograd (tests/test_oracle_helpers.py)."""
import numpy as np
import pytest
import torch

from oracle import ring_oracle as O

pytestmark = pytest.mark.gpu


def _bumps(rng, T, B, N):
    centre = rng.random((T, B)) * 2 * np.pi
    idx = np.arange(N)
    return (0.3 * np.exp(2.0 * (np.cos(2 * np.pi * idx / N - centre[..., None]) - 1.0))
            + 0.02 * rng.standard_normal((T, B, N))).astype(np.float32)


@pytest.mark.parametrize("T,B,N,own", [(20, 37, 256, True), (7, 5, 130, True), (9, 16, 512, False), (3, 4, 24, True),
                                        (5, 3, 700, False), (4, 6, 2048, True), (3, 5, 1130, False)],
                         ids=["n256", "n130_scalar", "n512_given_target", "n24", "n700", "n2048", "n1130_scalar"])
def test_loss_and_gradient_match_the_oracle(T, B, N, own, gpu_device):
    from rnn_train_ring_attractor_amd import ring_loss_pair
    print(f"[case] loss head T={T} B={B} N={N}", flush=True)
    rng = np.random.default_rng(T * 1000 + N)
    bump = _bumps(rng, T, B, N)
    angle = (rng.random((B, T)) * 2 * np.pi).astype(np.float32)
    tgt = None if own else (rng.random(B) + 1.0).astype(np.float32)
    want_total, want_cos, want_amp, want_grad = O.loss_pair_rank2(bump, angle, 0.2, tgt)
    h = torch.tensor(bump, device=gpu_device, requires_grad=True)
    total, lc, la = ring_loss_pair(h, torch.tensor(angle, device=gpu_device), 0.2,
                                   None if own else torch.tensor(tgt, device=gpu_device))
    (3.0 * total).backward()                      # an upstream factor other than one
    torch.cuda.synchronize()
    assert abs(float(total) - want_total) <= 2e-5 * max(1.0, abs(want_total))
    assert abs(float(lc) - want_cos) <= 2e-5 * max(1.0, abs(want_cos))
    assert abs(float(la) - want_amp) <= 2e-5 * max(1.0, abs(want_amp))
    got = h.grad.cpu().numpy()
    assert np.isfinite(got).all()
    assert O.max_rel_err(got, 3.0 * want_grad) <= 2e-4
    assert O.cosine(got, 3.0 * want_grad) >= 0.999999


def test_loss_head_agrees_with_the_torch_chain_on_operator_output(gpu_device):
    """End to end on the GPU: operator -> fused loss head, against operator -> the torch chain of the training script."""
    from rnn_train_ring_attractor_amd import host, ring_loss_pair, ring_rnn_cuda_func
    from tests.ring_cases import make_problem
    print("[case] loss head after the operator N=256 B=48 T=30", flush=True)
    p = make_problem(77, 48, 30, 2, 256, weights="perfect")
    t = lambda x: torch.tensor(x, device=gpu_device)
    angle = t(p["angle"])
    grads = []
    for fused in (True, False):
        Wa, Wo = t(p["Wa"]).requires_grad_(True), t(p["Wo"]).requires_grad_(True)
        hist = ring_rnn_cuda_func(t(p["A"]), Wa, -1.0 / 256, 1.0 / 128, Wo, t(p["r0"]), 0.15, "tanh")
        if fused:
            total, _, _ = ring_loss_pair(hist, angle, 0.2)
        else:
            bump = hist.permute(1, 0, 2)
            idx = torch.arange(256, dtype=torch.float32, device=gpu_device)
            proj = bump @ torch.cos(2 * np.pi * (idx[:, None] - idx[None, :]) / 256)
            total = (host.cosine_similarity_loss(proj / proj.max(dim=2, keepdim=True)[0], angle)
                     + 0.2 * host.bump_amplitude_loss(bump))
        total.backward()
        grads.append((float(total), Wo.grad.cpu().numpy(), Wa.grad.cpu().numpy()))
    torch.cuda.synchronize()
    assert abs(grads[0][0] - grads[1][0]) <= 1e-4 * max(1.0, abs(grads[1][0]))
    assert O.cosine(grads[0][1], grads[1][1]) >= 0.9999 and O.cosine(grads[0][2], grads[1][2]) >= 0.9999
    assert O.max_rel_err(grads[0][1], grads[1][1]) <= 2e-3


@pytest.mark.parametrize("B,T,k,N,act,own,streaming,weights", [
    (64, 24, 2, 256, "gelu", True, "0", "perfect"),   # weight-resident geometry, unmasked kernel
    (48, 12, 2, 256, "tanh", True, "0", "random"),    # amplitude deviations of both signs (own target, drifting bump)
    (37, 9, 2, 200, "tanh", False, "0", "perfect"),   # weight-resident geometry, masked rows and neurons
    (37, 9, 2, 200, "tanh", True, "1", "random"),     # the streaming kernels, four column tiles
    (20, 6, 3, 96, "silu", True, "0", "random"),      # the streaming kernels, two column tiles, three action channels
    (40, 5, 2, 512, "tanh", True, "0", "random"),     # widest tiling
    (24, 5, 2, 1024, "tanh", True, "0", "random"),    # wide ring: the operator chains loss backward and time-loop backward
    (18, 4, 2, 2048, "tanh", True, "0", "random"),    # the widest ring (eight 256-neuron chunks per row in the loss head)
    (18, 4, 2, 1301, "silu", False, "0", "random"),   # six chunks, ragged width (scalar row loads)
], ids=["n256_full", "n256_random", "n200_masked", "n200_streaming", "n96_k3", "n512", "n1024_step", "n2048_step",
        "n1301_step"])
def test_time_loop_and_loss_as_one_operator(B, T, k, N, act, own, streaming, weights, gpu_device, monkeypatch):
    """ring_rnn_loss_func (one backward call, the loss gradient formed inside the BPTT kernel) against
    ring_rnn_cuda_func + ring_loss_pair (the gradient written to HBM and read back), and against the fp64 oracle:
    loss pair of the oracle's trajectory, its gradient pushed through the oracle's BPTT."""
    from rnn_train_ring_attractor_amd import ring_loss_pair, ring_rnn_cuda_func, ring_rnn_loss_func
    from tests.ring_cases import make_problem
    print(f"[case] time loop + loss operator B={B} T={T} k={k} N={N} {act} own_target={own} streaming={streaming}", flush=True)
    monkeypatch.setenv("RINGATTR_STREAMING", streaming)
    p = make_problem(300 + N + B, B, T, k, N, weights=weights)
    J0, J1 = (-1.0 / N, 2.0 / N) if weights == "perfect" else (-0.1, 0.1)
    t = lambda x: torch.tensor(np.ascontiguousarray(x), device=gpu_device)
    rng = np.random.default_rng(5)
    angle = t(p["angle"]) if "angle" in p else t((rng.random((B, T)) * 2 * np.pi).astype(np.float32))
    tgt_np = None if own else (rng.random(B) + 1.0).astype(np.float32)
    tgt = None if own else t(tgt_np)
    res = {}
    for fused in (True, False):
        Wa, Wo = t(p["Wa"]).requires_grad_(True), t(p["Wo"]).requires_grad_(True)
        r0 = t(p["r0"]).requires_grad_(True)
        if fused:
            total, lc, la, hist = ring_rnn_loss_func(t(p["A"]), Wa, J0, J1, Wo, r0, 0.15, act, angle, 0.2, tgt)
        else:
            hist = ring_rnn_cuda_func(t(p["A"]), Wa, J0, J1, Wo, r0, 0.15, act)
            total, lc, la = ring_loss_pair(hist, angle, 0.2, tgt)
        (2.5 * total).backward()
        torch.cuda.synchronize()
        res[fused] = (float(total), float(lc), float(la), hist.detach().cpu().numpy(), Wo.grad.cpu().numpy(),
                      Wa.grad.cpu().numpy(), r0.grad.cpu().numpy())
    f, s = res[True], res[False]
    # the same trajectory; the loss values agree to rounding (the weight-resident forward kernel forms the loss
    # head's row sums itself, in another order than the pass over the history that the two-operator chain runs)
    assert np.array_equal(f[3], s[3])
    for x, y in zip(f[:3], s[:3]):
        assert abs(x - y) <= 2e-6 * max(1.0, abs(y))
    for a, b in zip(f[4:], s[4:]):
        assert np.isfinite(a).all()
        assert O.max_rel_err(a, b) <= 2e-3 and O.cosine(a, b) >= 0.99999
    # fp64: the oracle's trajectory and its loss pair; the loss gradient is taken at the trajectory the kernel saw
    # (it divides by the squared read-out amplitude, so it amplifies the bf16-level trajectory difference, which
    # the trajectory tolerance already covers) and pushed through the oracle's BPTT
    ang_np = angle.cpu().numpy()
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    want_total = O.loss_pair_rank2(ref_hist, ang_np, 0.2, tgt_np)[0]
    gl = O.loss_pair_rank2(f[3], ang_np, 0.2, tgt_np)[3]
    ref = O.backward_dense(2.5 * gl, p["A"], p["Wa"], J0, J1, p["Wo"], ref_hist, p["r0"], 0.15, act)
    assert abs(f[0] - want_total) <= 1e-2 * max(1.0, abs(want_total))
    for got, key in ((f[4], "grad_Wo"), (f[5], "grad_Wa"), (f[6], "grad_r_init")):
        assert O.cosine(got, ref[key]) >= 0.999, key
        assert O.max_rel_err(got, ref[key]) <= 2e-2, key


@pytest.mark.parametrize("B,T,k,N,act", [(24, 8, 2, 120, "tanh"), (20, 6, 2, 256, "gelu"), (18, 5, 3, 300, "silu"),
                                         (16, 4, 2, 640, "tanh")],
                         ids=["n120", "n256", "n300_k3", "n640_step"])
def test_one_operator_also_returns_the_action_signal_gradient(B, T, k, N, act, gpu_device):
    """dL/d action_signal and dL/d r_init through ring_rnn_loss_func (loss gradient formed inside the BPTT kernel
    that also produces dL/dA) against ring_rnn_cuda_func + ring_loss_pair."""
    from rnn_train_ring_attractor_amd import ring_loss_pair, ring_rnn_cuda_func, ring_rnn_loss_func
    from tests.ring_cases import make_problem
    print(f"[case] one operator with grad_A B={B} T={T} k={k} N={N} {act}", flush=True)
    p = make_problem(500 + N, B, T, k, N, action="dense")
    t = lambda x: torch.tensor(np.ascontiguousarray(x), device=gpu_device)
    angle = t((np.random.default_rng(9).random((B, T)) * 2 * np.pi).astype(np.float32))
    res = {}
    for fused in (True, False):
        A, r0 = t(p["A"]).requires_grad_(True), t(p["r0"]).requires_grad_(True)
        Wa, Wo = t(p["Wa"]).requires_grad_(True), t(p["Wo"]).requires_grad_(True)
        if fused:
            total = ring_rnn_loss_func(A, Wa, -0.1, 0.1, Wo, r0, 0.15, act, angle, 0.2)[0]
        else:
            total = ring_loss_pair(ring_rnn_cuda_func(A, Wa, -0.1, 0.1, Wo, r0, 0.15, act), angle, 0.2)[0]
        total.backward()
        torch.cuda.synchronize()
        res[fused] = [x.grad.cpu().numpy() for x in (A, r0, Wa, Wo)]
    for a, b in zip(res[True], res[False]):
        assert np.isfinite(a).all() and np.abs(b).max() > 0
        assert O.max_rel_err(a, b) <= 2e-3 and O.cosine(a, b) >= 0.99999


@pytest.mark.parametrize("B,N", [(32, 256), (21, 200)], ids=["n256_full", "n200_masked"])
def test_one_operator_without_a_backward_returns_the_same_losses(B, N, gpu_device, default_kernels):
    """Under torch.no_grad() the forward keeps no saved record (another variant of the forward kernel forms the loss
    head's row sums); losses and trajectory equal those of the call that prepares a backward."""
    from rnn_train_ring_attractor_amd import ring_rnn_loss_func
    from tests.ring_cases import make_problem
    T, k = 11, 2
    print(f"[case] time loop + loss operator under no_grad B={B} T={T} N={N}", flush=True)
    p = make_problem(77 + N, B, T, k, N, weights="perfect")
    t = lambda x: torch.tensor(np.ascontiguousarray(x), device=gpu_device)
    args = lambda grad: (t(p["A"]), t(p["Wa"]).requires_grad_(grad), -1.0 / N, 2.0 / N, t(p["Wo"]).requires_grad_(grad),
                         t(p["r0"]), 0.15, "gelu", t(p["angle"]), 0.2, None)
    with_grad = ring_rnn_loss_func(*args(True))
    with torch.no_grad():
        without = ring_rnn_loss_func(*args(True))
    torch.cuda.synchronize()
    for a, b in zip(with_grad, without):
        assert torch.equal(a.detach(), b)
    assert not without[0].requires_grad


@pytest.mark.parametrize("family", ["wide", "block11", "block22"])
@pytest.mark.parametrize("B,T,k,N,act", [(40, 5, 3, 640, "silu"), (19, 4, 2, 1100, "tanh")], ids=["n640_k3", "n1100_ragged"])
def test_loss_gradient_inside_the_step_per_launch_backward(B, T, k, N, act, family, gpu_device, monkeypatch):
    """Wide rings: each of the step-per-launch BPTT kernels forms the loss gradient itself (state history rows, the
    loss head's row coefficients and a table of the neurons' angles in place of grad_output); against the chain that
    writes the [T,B,N] gradient and reads it back."""
    from rnn_train_ring_attractor_amd import ring_loss_pair, ring_rnn_cuda_func, ring_rnn_loss_func
    from tests.ring_cases import make_problem
    print(f"[case] fused loss backward, {family} kernels, B={B} T={T} k={k} N={N} {act}", flush=True)
    if family == "wide":
        monkeypatch.setenv("RINGATTR_WIDE", "1")
    else:
        monkeypatch.setenv("RINGATTR_WIDE", "0")
        monkeypatch.setenv("RINGATTR_BLOCK_SHAPE", family[-2:])
    p = make_problem(41 + N, B, T, k, N, action="dense")
    t = lambda x: torch.tensor(np.ascontiguousarray(x), device=gpu_device)
    angle = t(p["angle"])
    res = {}
    for fused in (True, False):
        A = t(p["A"]).requires_grad_(True)
        Wa, Wo, r0 = t(p["Wa"]).requires_grad_(True), t(p["Wo"]).requires_grad_(True), t(p["r0"]).requires_grad_(True)
        if fused:
            total = ring_rnn_loss_func(A, Wa, -0.05, 0.4, Wo, r0, 0.15, act, angle, 0.2)[0]
        else:
            total = ring_loss_pair(ring_rnn_cuda_func(A, Wa, -0.05, 0.4, Wo, r0, 0.15, act), angle, 0.2)[0]
        (1.7 * total).backward()
        torch.cuda.synchronize()
        res[fused] = [float(total)] + [x.grad.cpu().numpy() for x in (Wo, Wa, r0, A)]
    assert abs(res[True][0] - res[False][0]) <= 2e-6 * max(1.0, abs(res[False][0]))
    for name, a, b in zip(("grad_Wo", "grad_Wa", "grad_r_init", "grad_A"), res[True][1:], res[False][1:]):
        assert np.isfinite(a).all() and np.abs(b).max() > 0, name
        assert O.max_rel_err(a, b) <= 2e-3 and O.cosine(a, b) >= 0.99999, name
