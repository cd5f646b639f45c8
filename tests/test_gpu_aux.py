"""GPU checks of the device-side input generator and of the fused clip + Adam step.

Generator (ringattr_generate_inputs): the reference draws from torch's generator, whose stream no test of the
reference pins; what is fixed is the construction (utils/generate_av_integration_data.py:11-58), so the output is
checked against the structural invariants and closed forms of that construction and against the oracle's bump and
action-signal functions on the generated trials, plus simple distribution checks on large samples.
Optimizer (ringattr_clip_adam): against torch.nn.utils.clip_grad_norm_ + torch.optim.Adam on the CPU, step by step."""
import math

import numpy as np
import pytest
import torch

from oracle import ring_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,T,k,N,pad,bump", [(64, 120, 2, 120, True, "vm"), (257, 33, 16, 256, True, "gauss"),
                                               (50, 7, 5, 48, False, "gauss"), (4096, 240, 2, 256, True, "vm")],
                         ids=["config0", "k16_padded", "spread", "full_size"])
def test_generated_inputs_follow_the_reference_construction(B, T, k, N, pad, bump, gpu_device):
    from rnn_train_ring_attractor_amd import generate_inputs
    print(f"[case] generator B={B} T={T} k={k} N={N}", flush=True)
    ratios = [0.2, 0.5, 0.8]
    max_av = 0.1 * math.pi
    av, angle, action, r0 = generate_inputs(123, B, T, N, k, zero_ratios_in_rest=ratios, zero_padding=pad, bump=bump)
    av2, angle2, action2, r02 = generate_inputs(123, B, T, N, k, zero_ratios_in_rest=ratios, zero_padding=pad, bump=bump)
    assert all(torch.equal(a, b) for a, b in ((av, av2), (angle, angle2), (action, action2), (r0, r02)))   # a function of the seed
    other = generate_inputs(124, B, T, N, k, zero_ratios_in_rest=ratios, zero_padding=pad, bump=bump)[0]
    assert not torch.equal(av, other)
    av, angle, action, r0 = (x.cpu().numpy().astype(np.float64) for x in (av, angle, action, r0))
    n0 = int(T * 0.1)
    rest = T - n0
    assert np.all(av[:, :n0] == 0.0)
    assert np.abs(av).max() <= max_av
    allowed = {rest - int(np.float32(rest) * np.float32(r)) for r in ratios}
    counts = (av[:, n0:] != 0).sum(axis=1)
    assert set(np.unique(counts)) <= allowed                    # exactly rest - floor(rest * ratio) non-zero steps per trial
    if B >= 64:
        assert set(np.unique(counts)) == allowed                # every ratio is drawn
    assert np.all((angle[:, 0] >= 0) & (angle[:, 0] < 2 * np.pi))
    want = (angle[:, :1] + np.cumsum(av[:, :-1], axis=1)) % (2 * np.pi)
    diff = np.abs(np.angle(np.exp(1j * (angle[:, 1:] - want))))   # compare on the circle (fp32 wrap at 2 pi)
    assert diff.max() <= 1e-4
    assert np.all((angle >= 0) & (angle < 2 * np.pi + 1e-6))
    want_action = O.av_to_action_signal_nd(av, k, zero_padding=pad) if k != 2 or not pad else O.av_to_action_signal(av)
    np.testing.assert_allclose(action, want_action, rtol=1e-6, atol=1e-9)
    want_bump = (O.von_mises_bump if bump == "vm" else O.create_initial_bump)(angle[:, 0], N)
    assert O.max_rel_err(r0, want_bump) <= 1e-5
    np.testing.assert_allclose(np.linalg.norm(r0, axis=1), 1.0, rtol=1e-5)
    if B * rest >= 200_000:
        # distribution: non-zero values are U(-max_av, max_av); positions are chosen uniformly
        vals = av[:, n0:][av[:, n0:] != 0] / max_av
        assert abs(vals.mean()) <= 0.01 and abs(vals.var() - 1.0 / 3.0) <= 0.01
        assert abs(np.mean(np.abs(vals) < 0.5) - 0.5) <= 0.01
        freq = (av[:, n0:] != 0).mean(axis=0)
        assert freq.max() - freq.min() <= 0.06                  # no position favoured (binomial noise ~ 0.008)
        a0 = angle[:, 0] / (2 * np.pi)
        assert abs(a0.mean() - 0.5) <= 0.02 and abs(a0.var() - 1.0 / 12.0) <= 0.01


@pytest.mark.parametrize("T,ratio", [(180, 0.35), (10, 0.7), (120, 0.01)])
def test_generator_leading_zeros_are_pythons_count(T, ratio, gpu_device):
    """int(T * ratio) as Python forms it (a float32 product gives 63 and 6 for the first two pairs instead of 62
    and 7); with a zero ratio of 0 every later step is drawn, so the leading zeros are exactly the count."""
    from rnn_train_ring_attractor_amd import generate_inputs
    print(f"[case] generator leading zeros T={T} ratio={ratio}", flush=True)
    av = generate_inputs(5, 256, T, 64, 2, zero_padding_start_ratio=ratio, zero_ratios_in_rest=[0.0])[0].cpu().numpy()
    n0 = int(T * ratio)
    assert np.all(av[:, :n0] == 0.0)
    assert np.all(av[:, n0:] != 0.0)


def test_generated_inputs_drive_the_operator(gpu_device):
    """Generated tensors go straight into the time loop (zero-padded action channels state the driven ones)."""
    from rnn_train_ring_attractor_amd import generate_inputs, ring_rnn_cuda_func
    B, T, k, N = 64, 30, 8, 256
    av, angle, action, r0 = generate_inputs(5, B, T, N, k)
    gen = torch.Generator(device=gpu_device).manual_seed(1)
    Wa = torch.randn(k, N, N, device=gpu_device, generator=gen) / N ** 0.5
    Wo = torch.randn(N, N, device=gpu_device, generator=gen) / N ** 0.5
    hist = ring_rnn_cuda_func(action, Wa, -0.1, 0.2, Wo, r0, 0.15, "tanh")
    c = lambda t: t.cpu().numpy()
    ref, _ = O.forward_dense(c(action), c(Wa), -0.1, 0.2, c(Wo), c(r0), 0.15, "tanh")
    assert O.max_rel_err(c(hist), ref) <= 1e-2


@pytest.mark.parametrize("max_norm", [1.0, 1e9, 0.0], ids=["clipping", "not_clipping", "clip_off"])
def test_fused_clip_adam_matches_torch(max_norm, gpu_device):
    from rnn_train_ring_attractor_amd import FusedClipAdam
    torch.manual_seed(3)
    shapes = [(256, 256), (2, 256, 256), (16, 1), (16,), (1, 16), (1,), (5000,)]
    ref = [torch.randn(s).requires_grad_(True) for s in shapes]
    dev = [p.detach().clone().to(gpu_device).requires_grad_(True) for p in ref]
    opt_ref = torch.optim.Adam(ref, lr=3e-3, betas=(0.9, 0.99), eps=1e-8)
    opt_dev = FusedClipAdam(dev, lr=3e-3, betas=(0.9, 0.99), eps=1e-8, max_norm=max_norm)
    for step in range(5):
        grads = [torch.randn(s) * (3.0 if step % 2 == 0 else 0.01) for s in shapes]
        for p, q, g in zip(ref, dev, grads):
            p.grad = g.clone()
            q.grad = g.clone().to(gpu_device)
        if max_norm > 0:
            norm = torch.nn.utils.clip_grad_norm_(ref, max_norm)
        else:
            norm = torch.linalg.vector_norm(torch.stack([g.norm() for g in grads]))
        opt_ref.step()
        opt_dev.step()
        torch.cuda.synchronize()
        assert abs(float(opt_dev.last_grad_norm) - float(norm)) <= 1e-5 * float(norm)
        for p, q in zip(ref, dev):
            np.testing.assert_allclose(q.detach().cpu().numpy(), p.detach().numpy(), rtol=2e-5, atol=2e-7)
            np.testing.assert_allclose(q.grad.cpu().numpy(), p.grad.numpy(), rtol=1e-5, atol=1e-9)
    # repeatable bit for bit (fixed summation order of the norm)
    a = [p.detach().clone() for p in dev]
    opt2 = FusedClipAdam([x.clone().requires_grad_(True) for x in a], lr=1e-3, max_norm=0.5)
    opt3 = FusedClipAdam([x.clone().requires_grad_(True) for x in a], lr=1e-3, max_norm=0.5)
    for o in (opt2, opt3):
        for p, g in zip(o.params, grads):
            p.grad = g.clone().to(gpu_device)
        o.step()
    torch.cuda.synchronize()
    assert all(torch.equal(x, y) for x, y in zip(opt2.params, opt3.params))
