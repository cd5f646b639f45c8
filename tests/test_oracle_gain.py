"""The oracle's gain networks against the reference's own construction: nn.Sequential(Linear(1,h), GELU,
Linear(h,1), Softplus) applied per channel to |x| and multiplied onto x (train/train_ring_attractor.py:70-79,
136-146; train/train_general_ring_attractor.py:38-46, 99-109), forward values and autograd gradients, plus closed
forms that a dropped term or a swapped parameter block would break."""
import numpy as np
import torch
from torch import nn

from oracle import ring_oracle as O


def _nets(k, h, seed):
    torch.manual_seed(seed)
    return [nn.Sequential(nn.Linear(1, h), nn.GELU(), nn.Linear(h, 1), nn.Softplus()).double() for _ in range(k)]


def _pack(nets):
    return np.stack([np.concatenate([n[0].weight.detach().numpy().ravel(), n[0].bias.detach().numpy().ravel(),
                                     n[2].weight.detach().numpy().ravel(), n[2].bias.detach().numpy().ravel()])
                     for n in nets])


def test_gain_forward_and_gradients_match_torch_modules():
    B, T, k, h = 5, 7, 3, 16
    nets = _nets(k, h, 0)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((B, T, k)) * 0.4                 # both signs: the general model feeds |x|
    g = rng.standard_normal((B, T, k))
    xt = torch.tensor(x, requires_grad=True)
    out = torch.stack([nets[c](xt[:, :, c:c + 1].abs()).squeeze(-1) for c in range(k)], dim=2) * xt
    (out * torch.tensor(g)).sum().backward()
    params = _pack(nets)
    np.testing.assert_allclose(O.gain_forward(x, params), out.detach().numpy(), rtol=1e-12, atol=1e-14)
    gp, gx = O.gain_backward(x, params, g)
    want = np.stack([np.concatenate([n[0].weight.grad.numpy().ravel(), n[0].bias.grad.numpy().ravel(),
                                     n[2].weight.grad.numpy().ravel(), n[2].bias.grad.numpy().ravel()]) for n in nets])
    np.testing.assert_allclose(gp, want, rtol=1e-10, atol=1e-13)
    np.testing.assert_allclose(gx, xt.grad.numpy(), rtol=1e-10, atol=1e-13)


def test_gain_closed_forms():
    h = 4
    # zero second layer: gain = softplus(b2) for every input
    p = np.zeros((1, 3 * h + 1))
    p[0, :h] = 0.7
    p[0, 3 * h] = 0.3
    x = np.linspace(-1, 1, 11).reshape(1, 11, 1)
    np.testing.assert_allclose(O.gain_forward(x, p), x * np.log1p(np.exp(0.3)), rtol=1e-13)
    # softplus switches to the identity above 20 (torch's threshold)
    p[0, 3 * h] = 25.0
    np.testing.assert_allclose(O.gain_forward(x, p), x * 25.0, rtol=1e-13)
    # the input of the network is |x|: the gain is even in x, the output odd
    rng = np.random.default_rng(2)
    p = rng.standard_normal((2, 3 * h + 1))
    x = rng.standard_normal((3, 4, 2))
    np.testing.assert_allclose(O.gain_forward(-x, p), -O.gain_forward(x, p), rtol=1e-13)
    # finite differences of the parameter gradient (catches swapped blocks)
    g = rng.standard_normal(x.shape)
    gp, _ = O.gain_backward(x, p, g)
    for (c, o) in ((0, 0), (0, h + 1), (1, 2 * h + 2), (1, 3 * h)):
        d = np.zeros_like(p)
        d[c, o] = 1e-6
        fd = ((O.gain_forward(x, p + d) - O.gain_forward(x, p - d)) * g).sum() / 2e-6
        assert abs(fd - gp[c, o]) <= 1e-6 * max(1.0, abs(fd))
