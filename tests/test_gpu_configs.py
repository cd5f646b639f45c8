"""GPU parity at the benchmark configurations' own shapes: full-size where the fp64 oracle finishes in
seconds, and size-independent properties (batch-slice invariance, additivity of gradients over batch
shards, bitwise repeatability) at the headline size."""
import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from oracle import ring_oracle_bf16 as OB
from tests.ring_cases import make_problem

pytestmark = pytest.mark.gpu

TRAJ_TOL, GRAD_COS, GRAD_TOL = 1e-2, 0.999, 2e-2      # trajectories / decoded angles; gradient cosine; gradient max error


def _t(x, dev):
    return torch.tensor(np.ascontiguousarray(x), device=dev)


def test_config1_inference_full_size(gpu_device):
    """Forward only: N=256, B=1024, T=120, relu, zero ratio 0.5 (the forward-only inference shape)."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print("[case] config1 N=256 B=1024 T=120 relu", flush=True)
    B, T, k, N = 1024, 120, 2, 256
    p = make_problem(11, B, T, k, N, zero_ratios=(0.5,), weights="perfect", bump="vm")
    with torch.no_grad():
        hist = ring_rnn_cuda_func(_t(p["A"], gpu_device), _t(p["Wa"], gpu_device), -0.1, 0.1, _t(p["Wo"], gpu_device),
                                  _t(p["r0"], gpu_device), 0.15, "gelu")
        hist_relu = ring_rnn_cuda_func(_t(p["A"], gpu_device), _t(p["Wa"] / N, gpu_device), -1.0 / N, 1.0,
                                       _t(p["Wo"] / N, gpu_device), _t(p["r0"], gpu_device), 0.15, "relu")
    got = hist.cpu().numpy().astype(np.float64)
    ref, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, "gelu")
    assert O.max_rel_err(got, ref) <= TRAJ_TOL
    dg = O.decode_angle_from_population_vector(O.readout(got.transpose(1, 0, 2)))
    dr = O.decode_angle_from_population_vector(O.readout(ref.transpose(1, 0, 2)))
    assert np.abs(np.angle(np.exp(1j * (dg - dr)))).max() <= TRAJ_TOL * 2 * np.pi
    # the relu variant of the same network (weights scaled to keep the bump bounded)
    ref_relu, _ = O.forward_dense(p["A"], p["Wa"] / N, -1.0 / N, 1.0, p["Wo"] / N, p["r0"], 0.15, "relu")
    assert O.max_rel_err(hist_relu.cpu().numpy(), ref_relu) <= TRAJ_TOL


def test_config3_geometry_long_sequence(gpu_device):
    """N=512, T=512, tanh (the long-sequence shape at a batch the oracle can follow): 512 leak steps must not drift."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print("[case] config3 N=512 B=32 T=512 tanh", flush=True)
    B, T, k, N = 32, 512, 2, 512
    p = make_problem(12, B, T, k, N, zero_ratios=(0.2,), bump="vm")
    Wa = _t(p["Wa"], gpu_device).requires_grad_(True)
    Wo = _t(p["Wo"], gpu_device).requires_grad_(True)
    hist = ring_rnn_cuda_func(_t(p["A"], gpu_device), Wa, -0.1, 0.1, Wo, _t(p["r0"], gpu_device), 0.15, "tanh")
    hist.backward(_t(p["G"], gpu_device))
    ref, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, "tanh")
    g = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.1, p["Wo"], ref, p["r0"], 0.15, "tanh")
    got = hist.detach().cpu().numpy()
    assert O.max_rel_err(got, ref) <= TRAJ_TOL
    for t in (0, 255, 511):
        assert O.max_rel_err(got[t], ref[t]) <= TRAJ_TOL
    assert O.cosine(Wo.grad.cpu().numpy(), g["grad_Wo"]) >= GRAD_COS
    assert O.max_rel_err(Wo.grad.cpu().numpy(), g["grad_Wo"]) <= GRAD_TOL
    assert O.cosine(Wa.grad.cpu().numpy(), g["grad_Wa"]) >= GRAD_COS
    assert O.max_rel_err(Wa.grad.cpu().numpy(), g["grad_Wa"]) <= GRAD_TOL


def test_headline_size_properties(gpu_device):
    """N=256, B=4096, T=120, gelu (the headline training shape).  The fp64 oracle checks a 64-row slice; the rest
    follows from properties that do not depend on the size."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print("[case] headline N=256 B=4096 T=120 gelu", flush=True)
    B, T, k, N = 4096, 120, 2, 256
    J0, J1 = -1.0 / N, 1.0
    p = make_problem(42, B, T, k, N, bump="vm")
    A, r0, G = _t(p["A"], gpu_device), _t(p["r0"], gpu_device), _t(p["G"], gpu_device)

    def run(rows):
        Wa = _t(p["Wa"], gpu_device).requires_grad_(True)
        Wo = _t(p["Wo"], gpu_device).requires_grad_(True)
        h = ring_rnn_cuda_func(A[rows].contiguous(), Wa, J0, J1, Wo, r0[rows].contiguous(), 0.15, "gelu")
        h.backward(G[:, rows].contiguous())
        return h.detach(), Wa.grad, Wo.grad

    full = run(slice(0, B))
    again = run(slice(0, B))
    assert all(torch.equal(a, b) for a, b in zip(full, again))                 # bitwise repeatable
    # samples are independent: a 64-row slice run alone reproduces its rows of the full batch bit for bit
    part = run(slice(1024, 1088))
    assert torch.equal(part[0], full[0][:, 1024:1088])
    sl = slice(1024, 1088)
    ref, _ = O.forward_dense(p["A"][sl], p["Wa"], J0, J1, p["Wo"], p["r0"][sl], 0.15, "gelu")
    assert O.max_rel_err(part[0].cpu().numpy(), ref) <= TRAJ_TOL
    g = O.backward_dense(p["G"][:, sl], p["A"][sl], p["Wa"], J0, J1, p["Wo"], ref, p["r0"][sl], 0.15, "gelu")
    assert O.cosine(part[2].cpu().numpy(), g["grad_Wo"]) >= GRAD_COS
    assert O.max_rel_err(part[2].cpu().numpy(), g["grad_Wo"]) <= GRAD_TOL
    assert O.cosine(part[1].cpu().numpy(), g["grad_Wa"]) >= GRAD_COS
    assert O.max_rel_err(part[1].cpu().numpy(), g["grad_Wa"]) <= GRAD_TOL
    # gradients are sums over samples: two half-batch shards add up to the full batch (fp32 order noise)
    lo, hi = run(slice(0, B // 2)), run(slice(B // 2, B))
    assert O.max_rel_err((lo[1] + hi[1]).cpu().numpy(), full[1].cpu().numpy()) <= 1e-4
    assert O.max_rel_err((lo[2] + hi[2]).cpu().numpy(), full[2].cpu().numpy()) <= 1e-4
    assert torch.isfinite(full[0]).all()


def test_headline_size_training_objective_as_one_operator(gpu_device):
    """N=256, B=4096, T=120, gelu: time loop and loss head as one operator (row sums formed inside the forward kernel,
    loss gradient inside the BPTT kernel) against the two-operator chain at the full size; the fp64 oracle prices a
    64-row slice of the loss; sample independence: the loss of the full batch is the mean of its shards' losses."""
    from rnn_train_ring_attractor_amd import ring_loss_pair, ring_rnn_cuda_func, ring_rnn_loss_func
    print("[case] headline one-operator objective N=256 B=4096 T=120 gelu", flush=True)
    B, T, k, N = 4096, 120, 2, 256
    J0, J1 = -1.0 / N, 1.0
    p = make_problem(43, B, T, k, N, bump="vm")
    A, r0, angle = _t(p["A"], gpu_device), _t(p["r0"], gpu_device), _t(p["angle"], gpu_device)

    def run(fused, rows=slice(0, B)):
        Wa = _t(p["Wa"], gpu_device).requires_grad_(True)
        Wo = _t(p["Wo"], gpu_device).requires_grad_(True)
        a, r, ang = A[rows].contiguous(), r0[rows].contiguous(), angle[rows].contiguous()
        if fused:
            total = ring_rnn_loss_func(a, Wa, J0, J1, Wo, r, 0.15, "gelu", ang, 0.2)[0]
        else:
            total = ring_loss_pair(ring_rnn_cuda_func(a, Wa, J0, J1, Wo, r, 0.15, "gelu"), ang, 0.2)[0]
        total.backward()
        return float(total.detach()), Wa.grad, Wo.grad

    one, two, again = run(True), run(False), run(True)
    assert np.isfinite(one[0]) and torch.isfinite(one[1]).all() and float(one[2].abs().max()) > 0
    assert one[0] == again[0] and torch.equal(one[1], again[1]) and torch.equal(one[2], again[2])   # repeatable
    assert abs(one[0] - two[0]) <= 2e-6 * max(1.0, abs(two[0]))
    for a, b in zip(one[1:], two[1:]):
        assert O.max_rel_err(a.cpu().numpy(), b.cpu().numpy()) <= 2e-3 and O.cosine(a.cpu().numpy(), b.cpu().numpy()) >= 0.99999
    sl = slice(2048, 2112)
    ref, _ = O.forward_dense(p["A"][sl], p["Wa"], J0, J1, p["Wo"], p["r0"][sl], 0.15, "gelu")
    want = O.loss_pair_rank2(ref, p["angle"][sl], 0.2, None)[0]
    part = run(True, sl)
    assert abs(part[0] - want) <= 1e-2 * max(1.0, abs(want))
    lo, hi = run(True, slice(0, B // 2)), run(True, slice(B // 2, B))
    assert abs(0.5 * (lo[0] + hi[0]) - one[0]) <= 1e-5 * max(1.0, abs(one[0]))
    assert O.max_rel_err((0.5 * (lo[2] + hi[2])).cpu().numpy(), one[2].cpu().numpy()) <= 1e-4


def test_widest_ring_at_a_training_batch(gpu_device):
    """N = 2048 (the reference's widest published ring), B = 512, T = 16, forward + backward on the step-per-launch
    kernels: bitwise repeatable, samples independent (a half-batch shard reproduces its rows bit for bit), gradients
    additive over shards; the fp64 oracle checks a 16-row slice."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print("[case] widest ring N=2048 B=512 T=16 tanh", flush=True)
    B, T, k, N = 512, 16, 2, 2048
    J0, J1 = -1.0 / N, 1.0
    p = make_problem(44, B, T, k, N)
    A, r0, G = _t(p["A"], gpu_device), _t(p["r0"], gpu_device), _t(p["G"], gpu_device)

    def run(rows):
        Wa = _t(p["Wa"], gpu_device).requires_grad_(True)
        Wo = _t(p["Wo"], gpu_device).requires_grad_(True)
        h = ring_rnn_cuda_func(A[rows].contiguous(), Wa, J0, J1, Wo, r0[rows].contiguous(), 0.15, "tanh")
        h.backward(G[:, rows].contiguous())
        return h.detach(), Wa.grad, Wo.grad

    full, again = run(slice(0, B)), run(slice(0, B))
    assert all(torch.equal(a, b) for a, b in zip(full, again)) and torch.isfinite(full[0]).all()
    lo, hi = run(slice(0, B // 2)), run(slice(B // 2, B))
    assert torch.equal(lo[0], full[0][:, :B // 2]) and torch.equal(hi[0], full[0][:, B // 2:])
    for i in (1, 2):
        # (the half batch runs on the other step-per-launch kernel family, which gives the same bits: only the order
        # of the sum over the batch differs between one call and two)
        assert O.max_rel_err((lo[i] + hi[i]).cpu().numpy(), full[i].cpu().numpy()) <= 1e-4
    sl = slice(256, 272)
    part = run(sl)
    ref, _ = O.forward_dense(p["A"][sl], p["Wa"], J0, J1, p["Wo"], p["r0"][sl], 0.15, "tanh")
    assert O.max_rel_err(part[0].cpu().numpy(), ref) <= TRAJ_TOL
    g = O.backward_dense(p["G"][:, sl], p["A"][sl], p["Wa"], J0, J1, p["Wo"], ref, p["r0"][sl], 0.15, "tanh")
    assert O.cosine(part[2].cpu().numpy(), g["grad_Wo"]) >= GRAD_COS
    assert O.max_rel_err(part[2].cpu().numpy(), g["grad_Wo"]) <= GRAD_TOL


@pytest.mark.parametrize("forward", ["cluster", "streaming", "cluster_with_bptt"])
def test_long_sequence_shape_at_full_size(gpu_device, monkeypatch, forward):
    """N=512, B=8192, T=512, tanh at its real size (inputs generated on the device): bitwise repeatable, a 32-row
    slice run alone reproduces its rows of the full batch bit for bit and agrees with the fp64 oracle, the
    gradient is linear in grad_output, two half-batch shards add up to the full batch.  Once per forward kernel of
    this width (left alone the library runs the full batch on the cluster kernel and the small shards on the
    streaming ones, which round Wo differently; the row-for-row identities hold inside one family), and once more with
    the BPTT on the clusters as well (off unless asked for)."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    monkeypatch.setenv("RINGATTR_CLUSTER", "0" if forward == "streaming" else "1")
    if forward == "cluster_with_bptt":
        monkeypatch.setenv("RINGATTR_CLUSTER_BPTT", "1")
    else:
        monkeypatch.delenv("RINGATTR_CLUSTER_BPTT", raising=False)
    print(f"[case] long sequence N=512 B=8192 T=512 tanh (full size), {forward} forward", flush=True)
    B, T, k, N = 8192, 512, 2, 512
    # J1 = 0.5 here: at the configuration's own J1 = 1 the dynamics are marginally stable and the bf16 rounding of Wo
    # (a fixed perturbation of the network) accumulates past 1e-2 after ~166 steps -- shown on the CPU in
    # tests/test_oracle_forward.py and held to what can be demanded in test_long_sequence_at_its_own_gain below
    J0, J1 = -1.0 / N, 0.5
    gen = torch.Generator(device=gpu_device).manual_seed(3)
    Wa0 = torch.randn(k, N, N, device=gpu_device, generator=gen) / N ** 0.5
    Wo0 = torch.randn(N, N, device=gpu_device, generator=gen) / N ** 0.5
    A = torch.rand(B, T, k, device=gpu_device, generator=gen) * 0.3 * (torch.rand(B, T, 1, device=gpu_device, generator=gen) > 0.2)
    r0 = torch.rand(B, N, device=gpu_device, generator=gen)
    r0 = r0 / r0.norm(dim=1, keepdim=True)
    G = torch.randn(T, B, N, device=gpu_device, generator=gen)

    def run(rows, scale=1.0):
        Wa, Wo = Wa0.clone().requires_grad_(True), Wo0.clone().requires_grad_(True)
        h = ring_rnn_cuda_func(A[rows].contiguous(), Wa, J0, J1, Wo, r0[rows].contiguous(), 0.15, "tanh")
        h.backward((G[:, rows] * scale).contiguous())
        return h.detach(), Wa.grad, Wo.grad

    full = run(slice(0, B))
    again = run(slice(0, B))
    assert all(torch.equal(a, b) for a, b in zip(full, again))
    assert torch.isfinite(full[0]).all() and torch.isfinite(full[1]).all() and torch.isfinite(full[2]).all()
    sl = slice(4096, 4128)
    part = run(sl)
    assert torch.equal(part[0], full[0][:, sl])
    c = lambda x: x.cpu().numpy()
    ref, _ = O.forward_dense(c(A[sl]), c(Wa0), J0, J1, c(Wo0), c(r0[sl]), 0.15, "tanh")
    assert O.max_rel_err(c(part[0]), ref) <= TRAJ_TOL
    g = O.backward_dense(c(G[:, sl]), c(A[sl]), c(Wa0), J0, J1, c(Wo0), ref, c(r0[sl]), 0.15, "tanh")
    assert O.cosine(c(part[2]), g["grad_Wo"]) >= GRAD_COS and O.max_rel_err(c(part[2]), g["grad_Wo"]) <= GRAD_TOL
    assert O.cosine(c(part[1]), g["grad_Wa"]) >= GRAD_COS and O.max_rel_err(c(part[1]), g["grad_Wa"]) <= GRAD_TOL
    # the backward without the forward's saved record (the reference's call pattern: nothing but bump_history is
    # kept, the derivative record and the operand copy are recomputed from it) at the full size
    from rnn_train_ring_attractor_amd import bwd_cuda
    gWa, gWo = torch.empty_like(Wa0), torch.empty_like(Wo0)
    bwd_cuda.bwd(grad_output=G, A=A, Wa=Wa0, J0=J0, J1=J1, Wo=Wo0, bump_history=full[0], r_init=r0, grad_Wa=gWa,
                 grad_Wo=gWo, alpha=0.15, activation_type=2, accumulate=False)
    torch.cuda.synchronize()
    assert O.max_rel_err(c(gWa), c(full[1])) <= 1e-3 and O.max_rel_err(c(gWo), c(full[2])) <= 1e-3
    del gWa, gWo
    doubled = run(slice(0, B), 2.0)
    assert O.max_rel_err(c(doubled[2]), 2.0 * c(full[2])) <= 1e-5 and O.max_rel_err(c(doubled[1]), 2.0 * c(full[1])) <= 1e-5
    lo, hi = run(slice(0, B // 2)), run(slice(B // 2, B))
    assert O.max_rel_err(c(lo[1] + hi[1]), c(full[1])) <= 1e-4 and O.max_rel_err(c(lo[2] + hi[2]), c(full[2])) <= 1e-4


def test_long_sequence_at_its_own_gain(gpu_device):
    """BASELINE's long-sequence configuration at its own parameters (N = 512, T = 512, tanh, J0 = -1/N, J1 = 1; a
    32-row batch so that the fp64 oracle finishes in seconds).  bf16 operands: the kernels follow the rounding-aware
    model over all 512 steps and the fp64 oracle over the first 150 (beyond, the rounding of Wo accumulates past
    1e-2 in these marginally stable dynamics, in the model exactly as in the kernels).  precise_wo=True (Wo as two
    bf16 operands): trajectory within 1e-2 of fp64 over all 512 steps, weight gradients within the gradient
    tolerances."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print("[case] long sequence at J1 = 1: N=512 B=32 T=512 tanh", flush=True)
    B, T, k, N = 32, 512, 2, 512
    J0, J1 = -1.0 / N, 1.0
    p = make_problem(3, B, T, k, N, zero_ratios=(0.2,), bump="vm")
    p["G"] = p["G"] / (T * B)
    ref, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, "tanh")
    g = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref, p["r0"], 0.15, "tanh")
    model = OB.forward_backward(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, "tanh", p["G"], folded=False)
    c = lambda x: x.detach().cpu().numpy().astype(np.float64)

    def run(precise):
        Wa, Wo = _t(p["Wa"], gpu_device).requires_grad_(True), _t(p["Wo"], gpu_device).requires_grad_(True)
        h = ring_rnn_cuda_func(_t(p["A"], gpu_device), Wa, J0, J1, Wo, _t(p["r0"], gpu_device), 0.15, "tanh",
                               precise_wo=precise)
        h.backward(_t(p["G"], gpu_device))
        torch.cuda.synchronize()
        return c(h), c(Wa.grad), c(Wo.grad)

    def per_step(x, y):
        return np.array([O.max_rel_err(x[t], y[t]) for t in range(T)])

    h, gWa, gWo = run(False)
    e = per_step(h, ref)
    em = per_step(h, model["bump_history"])
    print(f"[measured] bf16 Wo: vs fp64 per-step max over t < 150 {e[:150].max():.2e}, at t = 511 {e[-1]:.2e}; vs rounding "
          f"model max over all steps {em.max():.2e}; grad_Wo vs fp64 {O.max_rel_err(gWo, g['grad_Wo']):.2e} (cos "
          f"{O.cosine(gWo, g['grad_Wo']):.5f}), vs model {O.max_rel_err(gWo, model['grad_Wo']):.2e}", flush=True)
    assert e[:150].max() <= TRAJ_TOL
    assert em.max() <= 2e-2                       # 512 steps of fp32 against fp64 sums on top of the same operands
    assert O.cosine(gWo, g["grad_Wo"]) >= GRAD_COS and O.cosine(gWa, g["grad_Wa"]) >= GRAD_COS
    assert O.max_rel_err(gWo, model["grad_Wo"]) <= GRAD_TOL and O.max_rel_err(gWa, model["grad_Wa"]) <= GRAD_TOL
    h, gWa, gWo = run(True)
    e = per_step(h, ref)
    whole = O.max_rel_err(h, ref)
    print(f"[measured] Wo as hi + lo: vs fp64 whole trajectory {whole:.2e}, per-step max over all 512 steps {e.max():.2e}; grad_Wo {O.max_rel_err(gWo, g['grad_Wo']):.2e} "
          f"(cos {O.cosine(gWo, g['grad_Wo']):.5f}), grad_Wa {O.max_rel_err(gWa, g['grad_Wa']):.2e} (cos {O.cosine(gWa, g['grad_Wa']):.5f})",
          flush=True)
    # in the max norm of the whole trajectory, as every other parity case; relative to each step's own largest state
    # (which decays from 0.12 to 0.03 along the sequence) the bound is twice as wide (measured 1.1e-2 at B = 32)
    assert whole <= TRAJ_TOL and e.max() <= 2 * TRAJ_TOL
    assert gWa.shape == p["Wa"].shape
    assert O.cosine(gWo, g["grad_Wo"]) >= GRAD_COS and O.max_rel_err(gWo, g["grad_Wo"]) <= GRAD_TOL
    assert O.cosine(gWa, g["grad_Wa"]) >= GRAD_COS and O.max_rel_err(gWa, g["grad_Wa"]) <= GRAD_TOL


def test_streaming_and_resident_kernels_agree(gpu_device, monkeypatch):
    """The generic weight-streaming kernels and the weight-resident ones evaluate the same recurrence."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    B, T, k, N = 80, 33, 2, 200                      # ragged: N < 256 and B not a multiple of 16
    p = make_problem(13, B, T, k, N)
    outs = {}
    for mode in ("0", "1"):
        monkeypatch.setenv("RINGATTR_STREAMING", mode)
        Wa = _t(p["Wa"], gpu_device).requires_grad_(True)
        Wo = _t(p["Wo"], gpu_device).requires_grad_(True)
        h = ring_rnn_cuda_func(_t(p["A"], gpu_device), Wa, -0.1, 0.1, Wo, _t(p["r0"], gpu_device), 0.15, "silu")
        h.backward(_t(p["G"], gpu_device))
        outs[mode] = (h.detach().cpu().numpy(), Wa.grad.cpu().numpy(), Wo.grad.cpu().numpy())
    for a, b in zip(outs["0"], outs["1"]):
        assert O.max_rel_err(a, b) <= 5e-3          # both round the same operands; only the J0 row sums differ
    model = OB.forward_backward(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, "silu", p["G"])
    assert O.max_rel_err(outs["0"][0], model["bump_history"]) <= 5e-3
    assert O.max_rel_err(outs["0"][2], model["grad_Wo"]) <= 5e-3


@pytest.mark.parametrize("B,T,k,N,act,saved", [
    (40, 9, 2, 512, "tanh", True),      # three batch tiles: the second workgroup's partner tile does not exist
    (33, 5, 3, 300, "gelu", True),      # ragged rows and neurons
    (48, 6, 4, 256, "silu", True),      # a_dim > 2 at N <= 256: the four-column-tile geometry
    (40, 7, 2, 512, "tanh", False),     # backward rebuilds the saved record (paired there as well)
])
def test_paired_batch_tiles_equal_single_tiles(B, T, k, N, act, saved, gpu_device, monkeypatch):
    """The streaming kernels may give a workgroup two batch tiles that share every weight fragment it
    fetches.  Per element the arithmetic is that of the one-tile kernels up to how the compiler contracts the
    fp32 epilogue into fused multiply-adds, so history and gradients agree to fp32 rounding; the paired run
    is also held to the oracle."""
    from rnn_train_ring_attractor_amd import rnn_cuda
    print(f"[case] paired tiles B={B} T={T} k={k} N={N} {act} saved={saved}", flush=True)
    p = make_problem(77 + N + k, B, T, k, N)
    acts = {"relu": 0, "gelu": 1, "tanh": 2, "silu": 3}
    outs = {}
    for mode in ("1", "2"):
        monkeypatch.setenv("RINGATTR_ROW_TILES", mode)
        A, Wa, Wo, r0, G = (_t(p[x], gpu_device) for x in ("A", "Wa", "Wo", "r0", "G"))
        hist = torch.empty(T, B, N, device=gpu_device)
        sv = torch.empty(rnn_cuda.saved_nbytes(N, k, T, B), dtype=torch.uint8, device=gpu_device) if saved else None
        rnn_cuda.fwd_cuda.fwd(A=A, Wa=Wa, J0=-0.1, J1=0.3, Wo=Wo, r_init=r0, bump_history=hist, alpha=0.15,
                              activation_type=acts[act], saved=sv)
        gWa, gWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
        gr0 = torch.empty_like(r0)
        rnn_cuda.bwd_cuda.bwd(grad_output=G, A=A, Wa=Wa, J0=-0.1, J1=0.3, Wo=Wo, bump_history=hist, r_init=r0,
                              grad_Wa=gWa, grad_Wo=gWo, alpha=0.15, activation_type=acts[act],
                              saved=sv, grad_r_init=gr0)
        torch.cuda.synchronize()
        outs[mode] = [x.cpu().numpy() for x in (hist, gWa, gWo, gr0)]
    # a last-bit difference in fp32 can flip the bf16 rounding of an operand copy, which the gradients see
    for (a, b), tol in zip(zip(outs["1"], outs["2"]), (1e-4, 2e-3, 2e-3, 2e-3)):
        assert O.max_rel_err(a, b) <= tol
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.3, p["Wo"], p["r0"], 0.15, act)
    assert O.max_rel_err(outs["2"][0], ref_hist) <= TRAJ_TOL
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.3, p["Wo"], ref_hist, p["r0"], 0.15, act)
    assert O.cosine(outs["2"][2], ref["grad_Wo"]) >= 0.999 and O.cosine(outs["2"][1], ref["grad_Wa"]) >= 0.999
    assert O.cosine(outs["2"][3], ref["grad_r_init"]) >= 0.999


@pytest.mark.parametrize("B,T,k,N,act,force,saved", [
    (40, 6, 2, 1024, "tanh", {"RINGATTR_WIDE": ("0", "1")}, True),     # wide ring: block kernels against one-tile kernels
    (24, 5, 3, 700, "gelu", {"RINGATTR_WIDE": ("0", "1")}, False),     # ragged, backward rebuilds the record
    (72, 7, 2, 512, "silu", {"RINGATTR_BLOCK": ("0", "1")}, True),     # persistent streaming against block (two tiles per workgroup)
    (40, 6, 5, 300, "relu", {"RINGATTR_BLOCK": ("0", "1")}, False),
])
def test_step_per_launch_families_agree(B, T, k, N, act, force, saved, gpu_device, monkeypatch):
    """The step-per-launch kernels (block, one-tile) and the persistent streaming kernels evaluate the same recurrence
    on the same bf16 operands.  The two step-per-launch families must agree bit for bit; the persistent streaming
    kernels differ from them in accumulation order and must agree to rounding.  The second run is also held to the
    oracle."""
    from rnn_train_ring_attractor_amd import rnn_cuda
    print(f"[case] step families B={B} T={T} k={k} N={N} {act} {force} saved={saved}", flush=True)
    p = make_problem(31 + N + k, B, T, k, N)
    acts = {"relu": 0, "gelu": 1, "tanh": 2, "silu": 3}
    J0, J1 = (-1.0 / N, 1.0) if act == "relu" else (-0.1, 0.3)
    (var, modes), = force.items()
    outs = {}
    for mode in modes:
        monkeypatch.setenv(var, mode)
        A, Wa, Wo, r0, G = (_t(p[x], gpu_device) for x in ("A", "Wa", "Wo", "r0", "G"))
        hist = torch.empty(T, B, N, device=gpu_device)
        sv = torch.empty(rnn_cuda.saved_nbytes(N, k, T, B), dtype=torch.uint8, device=gpu_device) if saved else None
        rnn_cuda.fwd_cuda.fwd(A=A, Wa=Wa, J0=J0, J1=J1, Wo=Wo, r_init=r0, bump_history=hist, alpha=0.15,
                              activation_type=acts[act], saved=sv)
        gWa, gWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
        gr0 = torch.empty_like(r0)
        rnn_cuda.bwd_cuda.bwd(grad_output=G, A=A, Wa=Wa, J0=J0, J1=J1, Wo=Wo, bump_history=hist, r_init=r0,
                              grad_Wa=gWa, grad_Wo=gWo, alpha=0.15, activation_type=acts[act],
                              saved=sv, grad_r_init=gr0)
        torch.cuda.synchronize()
        outs[mode] = [x.cpu().numpy() for x in (hist, gWa, gWo, gr0)]
    a, b = outs[modes[0]], outs[modes[1]]
    if var == "RINGATTR_WIDE":
        # block and one-tile kernels share layouts and the order of every sum: the same bits, so that which of them
        # the launcher picks for a batch size never shows in a result
        for x, y in zip(a, b):
            assert np.array_equal(x, y)
    assert O.max_rel_err(a[0], b[0]) <= 1e-4
    for x, y in zip(a[1:], b[1:]):
        # a last-bit difference in fp32 can flip the bf16 rounding of an operand copy (or a relu kink)
        assert O.max_rel_err(x, y) <= (2e-2 if act == "relu" else 3e-3)
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    assert O.max_rel_err(b[0], ref_hist) <= TRAJ_TOL
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref_hist, p["r0"], 0.15, act)
    floor = 0.995 if act == "relu" else 0.999       # bf16 operands move samples across the relu kink
    assert O.cosine(b[2], ref["grad_Wo"]) >= floor and O.cosine(b[1], ref["grad_Wa"]) >= floor
    assert O.cosine(b[3], ref["grad_r_init"]) >= floor


@pytest.mark.parametrize("B,T,k,N,act,wide", [(40, 5, 2, 1024, "tanh", "1"), (40, 6, 2, 1024, "gelu", "0"),
                                                (24, 7, 3, 700, "silu", "1"), (24, 1, 2, 640, "tanh", "0")])
def test_step_per_launch_rebuild_equals_saved_record_bitwise(B, T, k, N, act, wide, gpu_device, monkeypatch):
    """Without the forward's saved buffer the step-per-launch families recompute the derivative record and the operand
    copies from bump_history with the forward's own kernel (all steps in one launch), so the backward must give the
    same bits as with the buffer.  Even and odd sequence lengths: the operand copies are written a pair of steps at a
    time, and an odd length leaves half a pair."""
    from rnn_train_ring_attractor_amd import rnn_cuda
    print(f"[case] step rebuild == saved B={B} T={T} k={k} N={N} {act} wide={wide}", flush=True)
    monkeypatch.setenv("RINGATTR_WIDE", wide)
    p = make_problem(57 + N + T, B, T, k, N)
    acts = {"relu": 0, "gelu": 1, "tanh": 2, "silu": 3}
    J0, J1 = -1.0 / N, 0.3
    A, Wa, Wo, r0, G = (_t(p[x], gpu_device) for x in ("A", "Wa", "Wo", "r0", "G"))
    hist = torch.empty(T, B, N, device=gpu_device)
    sv = torch.empty(rnn_cuda.saved_nbytes(N, k, T, B), dtype=torch.uint8, device=gpu_device)
    rnn_cuda.fwd_cuda.fwd(A=A, Wa=Wa, J0=J0, J1=J1, Wo=Wo, r_init=r0, bump_history=hist, alpha=0.15,
                          activation_type=acts[act], saved=sv)
    outs = []
    for saved in (sv, None):
        gWa, gWo, gr0 = torch.zeros_like(Wa), torch.zeros_like(Wo), torch.empty_like(r0)
        rnn_cuda.bwd_cuda.bwd(grad_output=G, A=A, Wa=Wa, J0=J0, J1=J1, Wo=Wo, bump_history=hist, r_init=r0,
                              grad_Wa=gWa, grad_Wo=gWo, alpha=0.15, activation_type=acts[act], saved=saved,
                              grad_r_init=gr0)
        torch.cuda.synchronize()
        outs.append((gWa, gWo, gr0))
    for x, y in zip(*outs):
        assert torch.isfinite(x).all() and torch.equal(x, y)
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref_hist, p["r0"], 0.15, act)
    assert O.cosine(outs[1][1].cpu().numpy(), ref["grad_Wo"]) >= 0.999
    assert O.cosine(outs[1][0].cpu().numpy(), ref["grad_Wa"]) >= 0.999


@pytest.mark.parametrize("B,T,k,N,act", [(72, 5, 3, 1024, "tanh"), (40, 4, 7, 640, "silu")], ids=["n1024_k3", "n640_k7"])
def test_block_kernel_shapes_and_workgroup_orders_agree_bitwise(B, T, k, N, act, gpu_device, monkeypatch):
    """The block kernels come in four shapes (one or two row tiles per workgroup, one or two column tiles per wave)
    and two workgroup orders (plain, or column blocks pinned to an XCD).  Shape and order decide which workgroup
    computes an element, not how: every variant must give the same bits, forward and backward."""
    from rnn_train_ring_attractor_amd import rnn_cuda
    print(f"[case] block shapes B={B} T={T} k={k} N={N} {act}", flush=True)
    p = make_problem(91 + N, B, T, k, N)
    acts = {"relu": 0, "gelu": 1, "tanh": 2, "silu": 3}
    monkeypatch.setenv("RINGATTR_WIDE", "0")
    outs = []
    # (shape "w": the one-tile-per-workgroup family, compared between its two workgroup orders only)
    for shape, xcd in (("12", "1"), ("11", "1"), ("21", "1"), ("22", "1"), ("12", "0"), ("21", "0"), ("w", "1"), ("w", "0")):
        monkeypatch.setenv("RINGATTR_WIDE", "1" if shape == "w" else "0")
        monkeypatch.setenv("RINGATTR_BLOCK_SHAPE", "12" if shape == "w" else shape)
        monkeypatch.setenv("RINGATTR_XCD_MAP", xcd)
        A, Wa, Wo, r0, G = (_t(p[x], gpu_device) for x in ("A", "Wa", "Wo", "r0", "G"))
        hist = torch.empty(T, B, N, device=gpu_device)
        sv = torch.empty(rnn_cuda.saved_nbytes(N, k, T, B), dtype=torch.uint8, device=gpu_device)
        rnn_cuda.fwd_cuda.fwd(A=A, Wa=Wa, J0=-0.1, J1=0.3, Wo=Wo, r_init=r0, bump_history=hist, alpha=0.15,
                              activation_type=acts[act], saved=sv)
        gWa, gWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
        gr0, gA = torch.empty_like(r0), torch.empty_like(A)
        rnn_cuda.bwd_cuda.bwd(grad_output=G, A=A, Wa=Wa, J0=-0.1, J1=0.3, Wo=Wo, bump_history=hist, r_init=r0,
                              grad_Wa=gWa, grad_Wo=gWo, alpha=0.15, activation_type=acts[act],
                              saved=sv, grad_r_init=gr0, grad_A=gA)
        torch.cuda.synchronize()
        outs.append([x.cpu().numpy() for x in (hist, gWa, gWo, gr0, gA)])
    for other in outs[1:6]:
        for a, b in zip(outs[0], other):
            assert np.array_equal(a, b)
    for a, b in zip(outs[6], outs[7]):
        assert np.array_equal(a, b)
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.3, p["Wo"], p["r0"], 0.15, act)
    assert O.max_rel_err(outs[0][0], ref_hist) <= TRAJ_TOL


@pytest.mark.parametrize("driven", [(3, 9), (5,), ()], ids=["two", "one", "none"])
def test_silent_action_channels_are_compacted(driven, gpu_device, monkeypatch):
    """With a_dim > 2 and the caller's statement that at most two named channels are driven, the Python operator runs
    the time loop on those two (the weight-resident kernels at 128 < N <= 256).  Results must agree with the
    uncompacted run on all channels (the streaming kernels), and the silent channels' weight gradients must be
    exactly zero either way."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    B, T, k, N = 40, 12, 12, 256
    print(f"[case] silent channels, driven={driven}", flush=True)
    p = make_problem(91, B, T, k, N, action="dense")
    A = np.zeros_like(p["A"])
    for c in driven:
        A[..., c] = p["A"][..., c]
    outs = {}
    for mode in ("1", "0"):
        monkeypatch.setenv("RINGATTR_COMPACT_CHANNELS", mode)
        Wa, Wo = _t(p["Wa"], gpu_device).requires_grad_(True), _t(p["Wo"], gpu_device).requires_grad_(True)
        r0 = _t(p["r0"], gpu_device).requires_grad_(True)
        h = ring_rnn_cuda_func(_t(A, gpu_device), Wa, -0.1, 0.3, Wo, r0, 0.15, "tanh", driven_channels=driven)
        h.backward(_t(p["G"], gpu_device))
        torch.cuda.synchronize()
        outs[mode] = [x.cpu().numpy() for x in (h.detach(), Wa.grad, Wo.grad, r0.grad)]
        for c in range(k):
            if c not in driven:
                assert np.abs(outs[mode][1][c]).max() == 0.0
    for a, b in zip(outs["1"], outs["0"]):
        assert a.shape == b.shape
        assert O.max_rel_err(a, b) <= 5e-3          # two kernel families: same operands, different row-sum rounding
    ref_hist, _ = O.forward_dense(A, p["Wa"], -0.1, 0.3, p["Wo"], p["r0"], 0.15, "tanh")
    ref = O.backward_dense(p["G"], A, p["Wa"], -0.1, 0.3, p["Wo"], ref_hist, p["r0"], 0.15, "tanh")
    assert O.max_rel_err(outs["1"][0], ref_hist) <= TRAJ_TOL
    assert O.cosine(outs["1"][2], ref["grad_Wo"]) >= GRAD_COS and O.max_rel_err(outs["1"][2], ref["grad_Wo"]) <= GRAD_TOL
    for c in driven:
        assert O.cosine(outs["1"][1][c], ref["grad_Wa"][c]) >= GRAD_COS


def test_driven_channel_statement_is_checked_on_the_device_and_needs_no_read_back(gpu_device):
    """A wrong statement (a channel declared silent carries signal) must not produce a plausible wrong result: every
    output is NaN.  Without a statement the padded signal runs on the general kernels and is correct.  And the call
    does not wait for the device: queued behind a long-running kernel it returns while that kernel still runs."""
    import time
    from rnn_train_ring_attractor_amd import host, ring_rnn_cuda_func
    B, T, k, N = 32, 10, 8, 256
    p = make_problem(92, B, T, k, N, action="dense")
    A = np.zeros_like(p["A"])
    A[..., 0], A[..., 1], A[..., 5] = p["A"][..., 0], p["A"][..., 1], p["A"][..., 5]
    args = (_t(p["Wa"], gpu_device), -0.1, 0.3, _t(p["Wo"], gpu_device), _t(p["r0"], gpu_device), 0.15, "gelu")
    bad = ring_rnn_cuda_func(_t(A, gpu_device), *args, driven_channels=(0, 1))
    assert torch.isnan(bad).all()
    good = ring_rnn_cuda_func(_t(A, gpu_device), *args)
    ref, _ = O.forward_dense(A, p["Wa"], -0.1, 0.3, p["Wo"], p["r0"], 0.15, "gelu")
    assert O.max_rel_err(good.cpu().numpy(), ref) <= TRAJ_TOL
    with pytest.raises(ValueError):
        ring_rnn_cuda_func(_t(A, gpu_device), *args, driven_channels=(0, 1, 5))
    # the helper that zero-pads (L, R) states the driven channels itself
    av = torch.randn(B, T, device=gpu_device) * 0.2
    padded = host.av_to_action_signal_ND(av, k)
    tagged = ring_rnn_cuda_func(padded, *args)
    plain = ring_rnn_cuda_func(padded.clone(), *args)          # a copy carries no statement: general kernels
    assert O.max_rel_err(tagged.cpu().numpy(), plain.cpu().numpy()) <= 5e-3
    # asynchrony: a long chain of large matrix products first, then the operator on the same stream
    big = torch.randn(8192, 8192, device=gpu_device)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    acc = big
    for _ in range(40):
        acc = (acc @ big) * 1e-4
    queued = time.perf_counter() - t0
    out = ring_rnn_cuda_func(padded, *args)
    returned = time.perf_counter() - t0
    still_busy = not torch.cuda.current_stream().query()
    torch.cuda.synchronize()
    drained = time.perf_counter() - t0
    print(f"[measured] queued {queued * 1e3:.1f} ms, operator returned at {returned * 1e3:.1f} ms, stream drained at "
          f"{drained * 1e3:.1f} ms", flush=True)
    assert still_busy and returned < 0.5 * drained
    assert torch.isfinite(out).all()


@pytest.mark.parametrize("B", [17, 32], ids=["ragged_batch", "whole_tiles"])
@pytest.mark.parametrize("T", [1, 2, 3, 32, 33, 64, 65])
def test_sequence_length_edges_of_the_resident_kernels(T, B, gpu_device):
    """Sequence lengths around the kernels' internal boundaries (first/last step peeling, paired time steps and
    their merged stores at even lengths, gate chunks of 32 steps) with a ragged batch (masked kernels) and with
    whole batch tiles (unmasked kernels), forward and backward."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    k, N = 2, 256
    print(f"[case] sequence edge T={T} B={B}", flush=True)
    p = make_problem(50 + T, B, T, k, N)
    Wa = _t(p["Wa"], gpu_device).requires_grad_(True)
    Wo = _t(p["Wo"], gpu_device).requires_grad_(True)
    r0 = _t(p["r0"], gpu_device).requires_grad_(True)
    h = ring_rnn_cuda_func(_t(p["A"], gpu_device), Wa, -0.1, 0.4, Wo, r0, 0.15, "gelu")
    h.backward(_t(p["G"], gpu_device))
    torch.cuda.synchronize()
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.4, p["Wo"], p["r0"], 0.15, "gelu")
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.4, p["Wo"], ref_hist, p["r0"], 0.15, "gelu")
    assert O.max_rel_err(h.detach().cpu().numpy(), ref_hist) <= TRAJ_TOL
    for key, got in (("grad_Wo", Wo.grad), ("grad_Wa", Wa.grad), ("grad_r_init", r0.grad)):
        assert O.cosine(got.cpu().numpy(), ref[key]) >= 0.999, key
        assert O.max_rel_err(got.cpu().numpy(), ref[key]) <= 2e-2, key


def test_gain_network_model_trains_through_the_operator(gpu_device):
    """The general ring with gain networks (reduced size; tanh, because relu with the model's fixed J0 = -0.1 and
    random weights silences every neuron and all gradients vanish): gain-MLP gradients reach the parameters through
    dL/d action_signal.  Checked against CPU autograd of the torch port with the same parameters."""
    from oracle import torch_port as TP
    from rnn_train_ring_attractor_amd import host
    print("[case] gain-network model N=256 B=64 T=40 tanh", flush=True)
    torch.manual_seed(5)
    N, B, T = 256, 64, 40
    model = host.LeakyRingAttractor(N, activation="tanh", initialization="random")
    av, angle = host.generate_av_integration_data_ultra_fast(B, T)
    r0 = host.create_initial_bump(angle[:, 0], N)

    def loss_of(r_hist, bump):
        return host.cosine_similarity_loss(r_hist, angle.to(r_hist.device)) + 0.2 * host.bump_amplitude_loss(bump)

    # CPU reference: same module parameters, recurrence by the torch port, autograd end to end
    A_cpu = model.action_signal(av)
    bump_cpu = TP.ring_forward(A_cpu, torch.stack([model.Wl, model.Wr]), model.J0, model.J1, model.Wo, r0, 0.15,
                               "tanh").permute(1, 0, 2)
    proj = bump_cpu @ model.W_delta7
    loss_cpu = loss_of(proj / proj.max(dim=2, keepdim=True)[0], bump_cpu)
    loss_cpu.backward()
    want = {n: p.grad.clone() for n, p in model.named_parameters()}
    model.zero_grad()

    model.to(gpu_device)
    r_hist, bump = model(av.to(gpu_device), r0.to(gpu_device))
    loss = loss_of(r_hist, bump)
    loss.backward()
    torch.cuda.synchronize()
    assert abs(float(loss) - float(loss_cpu)) <= 1e-2 * abs(float(loss_cpu))
    for n, p in model.named_parameters():
        got, ref = p.grad.cpu().numpy(), want[n].numpy()
        assert np.isfinite(got).all(), n
        assert O.cosine(got, ref) >= 0.999, n
        assert O.max_rel_err(got, ref) <= 2e-2, n
    # the same objective as chained HIP operators (gain networks, time loop + loss head in one): same loss, and the
    # same gradients for every parameter, the gain networks' included
    model.zero_grad()
    total, _, _, hist = model.loss_pair(av.to(gpu_device), angle.to(gpu_device), r0.to(gpu_device), bump_weight=0.2)
    total.backward()
    torch.cuda.synchronize()
    assert hist.shape == (T, B, N)
    assert abs(float(total) - float(loss_cpu)) <= 1e-2 * abs(float(loss_cpu))
    for n, p in model.named_parameters():
        got, ref = p.grad.cpu().numpy(), want[n].numpy()
        assert O.cosine(got, ref) >= 0.999, n
        assert O.max_rel_err(got, ref) <= 2e-2, n


@pytest.mark.parametrize("N,k,B,T", [(256, 4, 48, 24), (640, 6, 24, 10)], ids=["n256_k4", "n640_k6_step"])
def test_general_ring_with_per_channel_gains(N, k, B, T, gpu_device):
    """host.GeneralizedRingAttractor (train/train_general_ring_attractor.py:22-153 of the reference): one gain
    network per action channel in front of the operator.  Loss and every parameter gradient against CPU autograd
    of the torch port with the same parameters (the port evaluates the gain networks as torch modules)."""
    from oracle import torch_port as TP
    from rnn_train_ring_attractor_amd import host
    print(f"[case] general ring with gains N={N} k={k} B={B} T={T}", flush=True)
    torch.manual_seed(11)
    model = host.GeneralizedRingAttractor(N, action_dim=k, activation="tanh", initialization="random")
    av, angle = host.generate_av_integration_data_ultra_fast(B, T)
    # (an even channel count: relu(av * linspace(-1, 1, k)) then has no identically zero channel)
    action = host.av_to_action_signal_ND(av, action_dim=k, zero_padding=False)
    r0 = host.create_initial_bump(angle[:, 0], N)

    def loss_of(r_hist, bump):
        return host.cosine_similarity_loss(r_hist, angle.to(r_hist.device)) + 0.2 * host.bump_amplitude_loss(bump)

    A_cpu = model.gated_action_signal(action)
    bump_cpu = TP.ring_forward(A_cpu, model.Wa, model.J0, model.J1, model.Wo, r0, 0.15, "tanh").permute(1, 0, 2)
    proj = bump_cpu @ model.W_delta7
    loss_cpu = loss_of(proj / proj.max(dim=2, keepdim=True)[0], bump_cpu)
    loss_cpu.backward()
    want = {n: p.grad.clone() for n, p in model.named_parameters()}
    model.zero_grad()

    model.to(gpu_device)
    r_hist, bump = model(action.to(gpu_device), r0.to(gpu_device))
    assert r_hist.shape == (B, T, N) and bump.shape == (B, T, N)
    loss = loss_of(r_hist, bump)
    loss.backward()
    torch.cuda.synchronize()
    assert abs(float(loss) - float(loss_cpu)) <= 1e-2 * abs(float(loss_cpu))
    assert len(want) == 2 + 4 * k
    for n, p in model.named_parameters():
        got, ref = p.grad.cpu().numpy(), want[n].numpy()
        assert np.isfinite(got).all(), n
        assert O.cosine(got, ref) >= 0.999, n
        assert O.max_rel_err(got, ref) <= 2e-2, n
    # the same objective with time loop and loss head as one operator
    model.zero_grad()
    total, _, _, _ = model.loss_pair(action.to(gpu_device), angle.to(gpu_device), r0.to(gpu_device), bump_weight=0.2)
    total.backward()
    torch.cuda.synchronize()
    assert abs(float(total) - float(loss_cpu)) <= 1e-2 * abs(float(loss_cpu))
    for n, p in model.named_parameters():
        got, ref = p.grad.cpu().numpy(), want[n].numpy()
        assert O.cosine(got, ref) >= 0.999, n
        assert O.max_rel_err(got, ref) <= 2e-2, n


def _gain_model(N, act, dev, seed=5):
    from rnn_train_ring_attractor_amd import host
    torch.manual_seed(seed)
    model = host.LeakyRingAttractor(N, activation=act, initialization="random")
    model.J0, model.J1 = -1.0 / N, 1.0
    return model.to(dev)


def _gain_oracle(model, av, r0, G, act):
    """fp64 oracle of the gain-network model on a batch slice: gates, trajectory, weight gradients and the
    gain-network parameter gradients through dL/d action_signal."""
    from rnn_train_ring_attractor_amd.gain import pack_gain_nets
    c = lambda t: t.detach().cpu().numpy().astype(np.float64)
    params = c(pack_gain_nets([model.gain_l_net, model.gain_r_net]))
    base = np.stack([np.maximum(-c(av), 0.0), np.maximum(c(av), 0.0)], axis=2)
    A = O.gain_forward(base, params)
    Wa = np.stack([c(model.Wl), c(model.Wr)])
    hist, _ = O.forward_dense(A, Wa, model.J0, model.J1, c(model.Wo), c(r0), 0.15, act)
    g = O.backward_dense(c(G), A, Wa, model.J0, model.J1, c(model.Wo), hist, c(r0), 0.15, act)
    gp, _ = O.gain_backward(base, params, g["grad_A"])
    # the same with the kernels' operand rounding made explicit (weight-resident family): relu's derivative flips
    model_g = OB.forward_backward(A, Wa, model.J0, model.J1, c(model.Wo), c(r0), 0.15, act, c(G), folded=True)
    gp_model, _ = O.gain_backward(base, params, model_g["grad_A"])
    return hist, g, gp, model_g, gp_model


def test_gain_network_configuration_at_full_size(gpu_device, default_kernels):
    """The general ring with gain networks at its benchmark size: N=256, B=4096, T=240, relu, two 1 -> 16 -> 1 gain
    networks evaluated by the HIP gain operator, BPTT through the weight-resident kernel with dL/d action_signal.
    A 64-row slice is checked against the fp64 oracle (trajectory, weight gradients, gain-network gradients); the
    full size by bitwise repeatability, slice invariance and additivity over batch shards."""
    from rnn_train_ring_attractor_amd import host
    from rnn_train_ring_attractor_amd.gain import pack_gain_nets
    print("[case] gain-network configuration N=256 B=4096 T=240 relu (full size)", flush=True)
    N, B, T, act = 256, 4096, 240, "relu"
    model = _gain_model(N, act, gpu_device)
    torch.manual_seed(6)
    av, angle = host.generate_av_integration_data_ultra_fast(B, T)
    r0 = host.create_initial_bump(angle[:, 0], N)
    av, r0 = av.to(gpu_device), r0.to(gpu_device)
    G = torch.randn(T, B, N, device=gpu_device, generator=torch.Generator(device=gpu_device).manual_seed(8))
    names = [n for n, _ in model.named_parameters()]

    def run(rows):
        model.zero_grad()
        h = model.forward_history(av[rows].contiguous(), r0[rows].contiguous())
        h.backward(G[:, rows].contiguous())
        return h.detach(), {n: p.grad.clone() for n, p in model.named_parameters()}

    full, again = run(slice(0, B)), run(slice(0, B))
    assert torch.equal(full[0], again[0])
    assert all(torch.equal(full[1][n], again[1][n]) for n in names)
    assert all(torch.isfinite(full[1][n]).all() for n in names)
    sl = slice(2048, 2112)
    part = run(sl)
    assert torch.equal(part[0], full[0][:, sl])
    hist, g, gp, model_g, gp_model = _gain_oracle(model, av[sl], r0[sl], G[:, sl], act)
    c = lambda t: t.cpu().numpy()
    assert O.max_rel_err(c(part[0]), hist) <= TRAJ_TOL
    # relu: the derivative flips at the kink (operands rounded to bf16) leave the cosine; entry-wise bounds are
    # asserted at a realistic batch in test_relu_gradients_against_fp64_at_a_realistic_batch
    assert O.cosine(c(part[1]["Wo"]), g["grad_Wo"]) >= GRAD_COS
    assert O.cosine(c(part[1]["Wl"]), g["grad_Wa"][0]) >= GRAD_COS and O.cosine(c(part[1]["Wr"]), g["grad_Wa"][1]) >= GRAD_COS
    h = 16
    got_l = np.concatenate([c(part[1]["gain_l_net.0.weight"]).ravel(), c(part[1]["gain_l_net.0.bias"]).ravel(),
                            c(part[1]["gain_l_net.2.weight"]).ravel(), c(part[1]["gain_l_net.2.bias"]).ravel()])
    got_r = np.concatenate([c(part[1]["gain_r_net.0.weight"]).ravel(), c(part[1]["gain_r_net.0.bias"]).ravel(),
                            c(part[1]["gain_r_net.2.weight"]).ravel(), c(part[1]["gain_r_net.2.bias"]).ravel()])
    assert got_l.shape == (3 * h + 1,)
    # per-sample dL/dA does not average relu's derivative flips: against fp64 the gain-network gradients are held to
    # the cosine, entry-wise to the rounding-aware model (same operand rounding as the kernels)
    for got, want, want_model in ((got_l, gp[0], gp_model[0]), (got_r, gp[1], gp_model[1])):
        assert O.cosine(got, want) >= 0.995
        assert O.max_rel_err(got, want_model) <= GRAD_TOL
    assert O.max_rel_err(c(part[1]["Wo"]), model_g["grad_Wo"]) <= GRAD_TOL
    assert O.max_rel_err(c(part[1]["Wl"]), model_g["grad_Wa"][0]) <= GRAD_TOL
    lo, hi = run(slice(0, B // 2)), run(slice(B // 2, B))
    for n in names:
        assert O.max_rel_err(c(lo[1][n] + hi[1][n]), c(full[1][n])) <= 2e-4, n


@pytest.mark.parametrize("weights", ["random", "perfect"])
def test_relu_gradients_against_fp64_at_a_realistic_batch(weights, gpu_device, default_kernels):
    """relu weight gradients against the fp64 oracle at B = 1024, T = 120 (122 880 samples per entry).  relu's
    derivative is a step, and rounding the operands to bf16 moves pre-activations across it: with random weights
    single entries differ from fp64 by 3-6 % even at this batch, with bump-sustaining weights (a few neurons carry
    the gradient) by 7-9 %; the cosine holds everywhere (>= 0.9991 measured).  The CPU model that rounds the same
    operands differs from fp64 by the same amounts and agrees with the kernels to 1e-2 and better, so the deviation
    is the operand format's, not a kernel's: the CPU model attributes all of it to the two forward operands (state
    and weights, either of which alone exceeds 2e-2; tests/test_oracle_bf16.py), and the weights cannot be carried
    at higher precision in a compute unit that keeps them resident.  The entry-wise 2e-2 bound is therefore asserted
    against that model; against fp64 the test asserts what was measured on the MI355X plus 20 % (random weights
    3.4e-2 / 5.6e-2, bump-sustaining weights 7.5e-2 / 9.1e-2 for grad_Wo / grad_Wa) so that a regression shows."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print(f"[case] relu gradients vs fp64 at N=256 B=1024 T=120, {weights} weights", flush=True)
    B, T, k, N = 1024, 120, 2, 256
    J0, J1 = -1.0 / N, 1.0
    p = make_problem(31, B, T, k, N, weights=weights)
    if weights == "perfect":                       # scaled so that the bump stays bounded under relu
        p["Wa"], p["Wo"] = p["Wa"] / N, p["Wo"] / N
    Wa = _t(p["Wa"], gpu_device).requires_grad_(True)
    Wo = _t(p["Wo"], gpu_device).requires_grad_(True)
    h = ring_rnn_cuda_func(_t(p["A"], gpu_device), Wa, J0, J1, Wo, _t(p["r0"], gpu_device), 0.15, "relu")
    h.backward(_t(p["G"], gpu_device))
    torch.cuda.synchronize()
    ref, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, "relu")
    g = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref, p["r0"], 0.15, "relu")
    model = OB.forward_backward(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, "relu", p["G"], folded=True)
    gWo, gWa = Wo.grad.cpu().numpy(), Wa.grad.cpu().numpy()
    e_wo, e_wa = O.max_rel_err(gWo, g["grad_Wo"]), O.max_rel_err(gWa, g["grad_Wa"])
    c_wo, c_wa = O.cosine(gWo, g["grad_Wo"]), O.cosine(gWa, g["grad_Wa"])
    m_wo, m_wa = O.max_rel_err(gWo, model["grad_Wo"]), O.max_rel_err(gWa, model["grad_Wa"])
    mm_wo = O.max_rel_err(model["grad_Wo"], g["grad_Wo"])
    print(f"[measured] relu {weights} B=1024 T=120: vs fp64 grad_Wo max-rel {e_wo:.3e} cos {c_wo:.6f}, grad_Wa max-rel "
          f"{e_wa:.3e} cos {c_wa:.6f}; vs rounding model grad_Wo {m_wo:.3e} grad_Wa {m_wa:.3e}; rounding model vs fp64 "
          f"grad_Wo {mm_wo:.3e}", flush=True)
    assert O.max_rel_err(h.detach().cpu().numpy(), ref) <= TRAJ_TOL
    assert c_wo >= GRAD_COS and c_wa >= GRAD_COS
    assert m_wo <= GRAD_TOL and m_wa <= GRAD_TOL
    bound_wo, bound_wa = {"random": (0.041, 0.067), "perfect": (0.090, 0.109)}[weights]
    assert e_wo <= bound_wo and e_wa <= bound_wa


def test_training_driver_reduces_loss(gpu_device):
    """The reference-style driver (same imports and call pattern) trains on the HIP operator."""
    import train_general_ring_no_gain as drv
    print("[case] training driver N=128 B=64 T=60 k=2", flush=True)
    _, hist = drv.run_training(action_dim=2, num_neurons=128, training_steps=40, batch_size=64, seq_len=60,
                               lr=3e-3, activation="gelu", log_every=0, seed=1)
    assert all(np.isfinite(hist))
    assert np.mean(hist[-5:]) < np.mean(hist[:5])
    # the same run with the fused loss head follows the same loss curve (same seed, same data)
    _, hist_fused = drv.run_training(action_dim=2, num_neurons=128, training_steps=40, batch_size=64, seq_len=60,
                                     lr=3e-3, activation="gelu", log_every=0, seed=1, fused_loss=True)
    assert all(np.isfinite(hist_fused))
    assert abs(hist_fused[0] - hist[0]) <= 1e-3 * abs(hist[0])
    assert np.mean(hist_fused[-5:]) < np.mean(hist_fused[:5])
    # and with the fused clip + Adam step in place of clip_grad_norm_ + torch.optim.Adam: the same curve
    _, hist_opt = drv.run_training(action_dim=2, num_neurons=128, training_steps=40, batch_size=64, seq_len=60,
                                   lr=3e-3, activation="gelu", log_every=0, seed=1, fused_optimizer=True)
    assert all(np.isfinite(hist_opt))
    assert abs(hist_opt[0] - hist[0]) <= 1e-6 * abs(hist[0])
    assert np.max(np.abs(np.array(hist_opt[:10]) - np.array(hist[:10]))) <= 1e-2 * abs(hist[0])
    assert np.mean(hist_opt[-5:]) < np.mean(hist_opt[:5])


def test_training_and_evaluation_entry_point(gpu_device):
    """run_training_and_evaluation, the reference script's entry point (train_general_ring_no_gain.py:261-376 there):
    training followed by the single-trial evaluation with both decoders, on the padded 16-channel action signal."""
    import train_general_ring_no_gain as drv
    print("[case] training + evaluation entry point N=128 k=16", flush=True)
    model, hist, res = drv.run_training_and_evaluation(action_dim=16, training_steps=30, num_neurons=128, batch_size=32,
                                                       seq_len=40, lr=3e-3, log_every=0, seed=2)
    assert len(hist) == 30 and all(np.isfinite(hist))
    assert res["cos_activity"].shape == (1, 40, 128) and res["bump_activity"].shape == (1, 40, 128)
    assert res["decoded_pv"].shape == (1, 40) and res["decoded_argmax"].shape == (1, 40)
    assert 0.0 <= res["mean_abs_error_pv"] <= np.pi and 0.0 <= res["mean_abs_error_argmax"] <= np.pi
    # the aligned target starts where the model's default bump sits
    assert abs(float(res["aligned_target"][0, 0]) - np.pi) <= 1e-5


def test_reference_sanity_check_and_gain_model_entry_points(gpu_device):
    """The reference's own acceptance bound (train/train_ring_attractor.py:327-348: fixed cosine weights, N = 360, gelu,
    cosine-similarity loss below 0.5) through the HIP path, and its two gain-model training entry points
    (train.train_ring_attractor / train.train_general_ring_attractor `run_training_and_evaluation`) at a reduced size,
    with the torch loss chain and with the objective as chained HIP operators."""
    import train.train_general_ring_attractor as TG
    import train.train_ring_attractor as TL
    print("[case] sanity check N=360 gelu; gain-model training entry points N=120 B=32 T=40", flush=True)
    assert TL.sanity_check_loss(batch_size=128, seq_len=120) < 0.5
    small = dict(num_neurons=120, training_steps=24, batch_size=32, seq_len=40, lr=3e-3, log_every=0, eval_seq_len=50)
    for fused in (False, True):
        model, hist, ev = TL.run_training_and_evaluation(fused=fused, sanity_check=False, **small)
        assert len(hist) == 24 and all(np.isfinite(hist)) and np.mean(hist[-4:]) < np.mean(hist[:4])
        assert ev["decoded_pv"].shape == (1, 50) and np.isfinite(ev["mean_abs_error_pv"])
        assert [n for n, _ in model.named_parameters()][:3] == ["Wo", "Wl", "Wr"]
        model, hist, ev = TG.run_training_and_evaluation(action_dim=2, fused=fused, **small)
        assert len(hist) == 24 and all(np.isfinite(hist)) and np.mean(hist[-4:]) < np.mean(hist[:4])
        assert ev["cos_activity"].shape == (1, 50, 120) and len(model.gain_nets) == 2
    with pytest.raises(ValueError):
        TG.run_training_and_evaluation(action_dim=3, **small)


def test_reference_signature_entry_points(gpu_device):
    """fwd_cuda / bwd_cuda with the reference's exact C argument lists (null stream, own scratch)."""
    import ctypes
    from rnn_train_ring_attractor_amd import _lib
    lib = _lib.load()
    B, T, k, N = 32, 9, 2, 64
    p = make_problem(14, B, T, k, N)
    A, Wa, Wo, r0, G = (_t(p[n], gpu_device) for n in ("A", "Wa", "Wo", "r0", "G"))
    hist = torch.empty(T, B, N, device=gpu_device)
    torch.cuda.synchronize()
    lib.fwd_cuda(A.data_ptr(), Wa.data_ptr(), -0.1, 0.1, Wo.data_ptr(), r0.data_ptr(), hist.data_ptr(), 0.15,
                 N, k, T, B, 2)
    ref, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, "tanh")
    assert O.max_rel_err(hist.cpu().numpy(), ref) <= TRAJ_TOL
    gWa, gWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
    dummy = torch.empty(1, device=gpu_device, dtype=torch.bfloat16)
    z = ctypes.c_void_p(None)
    lib.bwd_cuda(G.data_ptr(), A.data_ptr(), Wa.data_ptr(), -0.1, 0.1, Wo.data_ptr(), hist.data_ptr(), dummy.data_ptr(),
                 r0.data_ptr(), gWa.data_ptr(), gWo.data_ptr(), 0.15, N, k, T, B, 2, z, z, z, z, z, z, z)
    g = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.1, p["Wo"], ref, p["r0"], 0.15, "tanh")
    assert O.cosine(gWo.cpu().numpy(), g["grad_Wo"]) >= GRAD_COS
    assert O.max_rel_err(gWa.cpu().numpy(), g["grad_Wa"]) <= GRAD_TOL


@pytest.mark.parametrize("B,T,k,N,act", [(256, 33, 2, 256, "gelu"), (96, 21, 5, 512, "tanh"), (48, 13, 3, 1024, "silu")],
                         ids=["n256", "n512_k5", "n1024"])
def test_weight_gradient_time_segments_add_up(B, T, k, N, act, gpu_device, monkeypatch):
    """The weight-gradient kernel cuts long sequences into time segments, one launch each, whose partial sums add up
    (RINGATTR_DW_SEGMENT = K chunks per workgroup and launch).  Tiny segments here (odd lengths, several matrix
    groups, every tiled geometry): the gradients must equal those of one launch to fp32 summation order and meet the
    fp64 oracle; 0 switches the cut off."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print(f"[case] dW segments B={B} T={T} k={k} N={N} {act}", flush=True)
    p = make_problem(77, B, T, k, N, action="dense")
    J0, J1 = -0.05, 0.4

    from rnn_train_ring_attractor_amd import _lib

    def run(segment):
        monkeypatch.setenv("RINGATTR_DW_SEGMENT", str(segment))
        Wa, Wo = _t(p["Wa"], gpu_device).requires_grad_(True), _t(p["Wo"], gpu_device).requires_grad_(True)
        h = ring_rnn_cuda_func(_t(p["A"], gpu_device), Wa, J0, J1, Wo, _t(p["r0"], gpu_device), 0.15, act)
        h.backward(_t(p["G"], gpu_device))
        torch.cuda.synchronize()
        segments = _lib.load().ringattr_dw_segments(N, k, T, B)       # under the environment just set
        return Wa.grad.cpu().numpy(), Wo.grad.cpu().numpy(), segments, _lib.last_kernel_names().get("dw", "")

    one = run(0)
    assert one[2] == 1 and "ring_dw_direct_kernel" in one[3]
    for segment in (1, 3):
        cut = run(segment)
        assert cut[2] >= 2
        assert O.max_rel_err(cut[0], one[0]) <= 1e-5 and O.max_rel_err(cut[1], one[1]) <= 1e-5
    again = run(3)
    assert np.array_equal(again[0], cut[0]) and np.array_equal(again[1], cut[1])    # and it is repeatable bit for bit
    ref, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    g = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref, p["r0"], 0.15, act)
    assert O.max_rel_err(cut[1], g["grad_Wo"]) <= GRAD_TOL and O.max_rel_err(cut[0], g["grad_Wa"]) <= GRAD_TOL
