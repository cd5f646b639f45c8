"""GPU parity of the gain-network operator (ringattr_gain_fwd / ringattr_gain_bwd through the Python operator and
the C ABI) against the fp64 oracle, which is itself pinned to the reference's nn.Sequential construction."""
import numpy as np
import pytest
import torch

from oracle import ring_oracle as O

pytestmark = pytest.mark.gpu


def _case(seed, B, T, k, h, signed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((B, T, k)).astype(np.float32) * 0.3
    if not signed:
        x = np.maximum(x, 0.0)                                # the (L, R) channels are rectified
    params = (rng.standard_normal((k, 3 * h + 1)) / np.sqrt(h)).astype(np.float32)
    g = rng.standard_normal((B, T, k)).astype(np.float32)
    return x, params, g


@pytest.mark.parametrize("B,T,k,h,signed", [(64, 120, 2, 16, False), (37, 9, 3, 16, True), (5, 3, 1, 4, True),
                                            (128, 33, 16, 8, True), (21, 7, 2, 32, False), (19, 5, 4, 20, True)],
                         ids=["lr_h16", "ragged_k3", "tiny_h4", "k16_h8", "h32", "h20_padded"])
def test_gain_operator_matches_oracle(B, T, k, h, signed, gpu_device):
    from rnn_train_ring_attractor_amd import ring_gain_func
    print(f"[case] gain B={B} T={T} k={k} h={h}", flush=True)
    x, params, g = _case(7, B, T, k, h, signed)
    xt = torch.tensor(x, device=gpu_device, requires_grad=True)
    pt = torch.tensor(params, device=gpu_device, requires_grad=True)
    out = ring_gain_func(xt, pt)
    out.backward(torch.tensor(g, device=gpu_device))
    torch.cuda.synchronize()
    ref = O.gain_forward(x, params)
    gp, gx = O.gain_backward(x, params, g)
    # fp32 arithmetic against fp64: relative to the largest magnitude
    assert O.max_rel_err(out.detach().cpu().numpy(), ref) <= 1e-5
    assert O.max_rel_err(pt.grad.cpu().numpy(), gp) <= 1e-4
    assert O.max_rel_err(xt.grad.cpu().numpy(), gx) <= 1e-5
    assert O.cosine(pt.grad.cpu().numpy(), gp) >= 0.999999


def test_gain_gradients_are_repeatable_and_additive_at_full_size(gpu_device):
    """B*T of the gain-network benchmark shape (4096 x 240 samples, two channels): bitwise repeatable parameter
    gradients; two half-batch shards add up to the full batch; a slice agrees with the oracle."""
    from rnn_train_ring_attractor_amd import ring_gain_func
    B, T, k, h = 4096, 240, 2, 16
    gen = torch.Generator(device=gpu_device).manual_seed(11)
    x = torch.relu(torch.randn(B, T, k, device=gpu_device, generator=gen) * 0.2)
    params = torch.randn(k, 3 * h + 1, device=gpu_device, generator=gen) / h ** 0.5
    g = torch.randn(B, T, k, device=gpu_device, generator=gen)

    def run(rows):
        p = params.clone().requires_grad_(True)
        out = ring_gain_func(x[rows].contiguous(), p)
        out.backward(g[rows].contiguous())
        return out.detach(), p.grad

    full, again = run(slice(0, B)), run(slice(0, B))
    assert torch.equal(full[0], again[0]) and torch.equal(full[1], again[1])
    lo, hi = run(slice(0, B // 2)), run(slice(B // 2, B))
    assert O.max_rel_err((lo[1] + hi[1]).cpu().numpy(), full[1].cpu().numpy()) <= 1e-5
    sl = slice(100, 164)
    part = run(sl)
    c = lambda t: t.cpu().numpy()
    assert O.max_rel_err(c(part[0]), O.gain_forward(c(x[sl]), c(params))) <= 1e-5
    gp, _ = O.gain_backward(c(x[sl]), c(params), c(g[sl]))
    assert O.max_rel_err(c(part[1]), gp) <= 1e-4
