"""GPU parity: the HIP path (through the operator API and the C ABI) against the fp64 oracle on the
same seeded inputs.  Tolerances (bf16 operands, fp32 accumulation): state trajectories and decoded
angles within 1e-2 (max error over max magnitude); weight gradients cosine >= 0.999 and max error
over max magnitude <= 2e-2."""
import os

import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from oracle import ring_oracle_bf16 as OB
from tests.ring_cases import make_problem

pytestmark = pytest.mark.gpu

# relu's derivative is a step: with random weights ~8 % of the pre-activations sit within bf16 rounding
# of zero and flip it, which alone moves single gradient entries by 3-7 % against fp64 (the CPU model
# that rounds the same operands, oracle/ring_oracle_bf16.py, shows the same figure).  For relu the
# fp64 comparison therefore asserts the cosine only, and the entry-wise bound is asserted against the
# rounding-aware model; smooth activations are held to both.
TRAJ_TOL = 1e-2
GRAD_COS = 0.999
GRAD_TOL = 2e-2
ELEMENTWISE_TRAJ_TOL = 5e-2   # |x - ref| / |ref| on the entries that are at least 10 % of the largest
ELEMENTWISE_GRAD_TOL = 1e-1
MODEL_TOL = 5e-3        # HIP vs the rounding-aware CPU model (same operand rounding, fp64 accumulation)
ACTS = {"relu": 0, "gelu": 1, "tanh": 2, "silu": 3}


def _folded(N, k, A=None):
    """The weight-resident kernels (128 < N <= 256 and two action channels, or more of which the caller states that at
    most two are driven: the Python operator then runs on those two) take Wo as the bf16 rounding of J1 * Wo + J0, the
    generic ones round Wo alone and sum the J0 term in fp32; the rounding model follows the kernel under test."""
    if not (128 < N <= 256) or os.environ.get("RINGATTR_STREAMING") == "1":
        return False
    if k == 2:
        return True
    return _driven_hint(k, A) is not None and os.environ.get("RINGATTR_COMPACT_CHANNELS", "1") != "0"


def _driven_hint(k, A):
    """What a caller that zero-pads (L, R) to k channels knows and tells the operator: channels 0 and 1 are driven."""
    if k <= 2 or A is None:
        return None
    return (0, 1) if np.abs(A[..., 2:]).max() == 0 else None


CASES = [
    # name,            B,   T,   k,  N,  act,   J0,     J1,  action
    ("config0",        64, 120,  2, 120, "tanh", -1 / 120, 1.0, "lr"),
    ("config0_refJ",   64, 120,  2, 120, "tanh", -0.1, 0.1, "lr"),
    ("script_k16",    128, 100, 16, 256, "gelu", -0.1, 0.1, "lr"),
    ("n256_gelu",     256,  40,  2, 256, "gelu", -1 / 256, 1.0, "lr"),
    ("n256_relu",      96,  30,  2, 256, "relu", -1 / 256, 1.0, "lr"),
    ("ragged_silu",    37,   7,  3, 100, "silu", -0.1, 0.1, "dense"),
    ("tiny_k1",         5,   3,  1,  48, "relu", 0.02, 0.5, "dense"),
    ("n512_tanh",      32,  16,  2, 512, "tanh", -0.1, 0.1, "dense"),
    ("n512_odd",       40,   7,  2, 512, "gelu", -0.1, 0.1, "dense"),     # odd length, odd tile count: the four-tile rebuild's edges
    ("n64_one_step",   16,   1,  2,  64, "gelu", -0.1, 0.1, "dense"),
    ("odd_shapes",     17,   9,  5, 130, "gelu", -0.05, 0.2, "spread"),
    ("n64_lr",         32,   9,  2,  64, "tanh", -0.1, 0.1, "lr"),        # zero gates at the start: matrices skipped
    ("n48_dense",      16,   3,  2,  48, "tanh", -0.1, 0.1, "dense"),
    ("n512_k16_pad",   32,   6, 16, 512, "gelu", -0.1, 0.1, "lr"),        # zero-padded channels, widest tiling
    ("k70_wide_action", 20,  4, 70,  96, "tanh", -0.1, 0.1, "dense"),     # more channels than the LDS gate stage holds
    ("n300_k5_spread", 48,   5,  5, 300, "silu", -0.05, 0.2, "spread"),   # widest tiling, several matrix groups
    # wide rings (step-per-launch kernels, NPAD a multiple of 512): the reference's published widths
    ("n1024_gelu",     48,   6,  2, 1024, "gelu", -1 / 1024, 1.0, "lr"),
    ("n2048_k3_tanh",  20,   4,  3, 2048, "tanh", -0.01, 0.1, "dense"),
    ("n700_k16_pad",   32,   5, 16, 700, "silu", -0.05, 0.2, "lr"),       # ragged width, zero-padded channels
    ("n1500_relu",     17,   3,  2, 1500, "relu", -1 / 1500, 1.0, "dense"),
    # the reference's published many-channel rows (assets/REPORT.md:11-12: 32 and 64 channels)
    ("n2048_k32_dense", 16,  2, 32, 2048, "silu", -0.01, 0.1, "dense"),
    ("n1024_k64_dense", 16,  3, 64, 1024, "tanh", -0.01, 0.1, "dense"),
    ("n640_k66_dense",  20,  3, 66, 640, "tanh", -1 / 640, 0.3, "dense"),   # wide ring, more channels than the gate stage holds
]


def _problem(seed, B, T, k, N, action):
    action, _, weights = action.partition("+")
    return make_problem(seed, B, T, k, N, action=action, weights=weights or "random")


def _dev(x, device):
    return torch.tensor(x, device=device)


def _run_op(p, J0, J1, act, device, requires_grad=True):
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    A, r0 = _dev(p["A"], device), _dev(p["r0"], device)
    Wa = _dev(p["Wa"], device).requires_grad_(requires_grad)
    Wo = _dev(p["Wo"], device).requires_grad_(requires_grad)
    hist = ring_rnn_cuda_func(action_signal=A, Wa=Wa, J0=J0, J1=J1, Wo=Wo, r_init=r0, alpha=0.15, activation=act,
                              driven_channels=_driven_hint(p["A"].shape[2], p["A"]))
    return hist, Wa, Wo


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_forward_trajectory_and_decoded_angle(case, gpu_device):
    name, B, T, k, N, act, J0, J1, action = case
    print(f"[case] fwd {name} B={B} T={T} k={k} N={N} {act}", flush=True)
    p = _problem(100, B, T, k, N, action)
    hist, _, _ = _run_op(p, J0, J1, act, gpu_device, requires_grad=False)
    torch.cuda.synchronize()
    got = hist.cpu().numpy().astype(np.float64)
    ref, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    assert got.shape == (T, B, N)
    assert np.isfinite(got).all()
    err = O.max_rel_err(got, ref)
    assert err <= TRAJ_TOL, f"trajectory error {err}"
    ew = O.elementwise_rel_err(got, ref)
    print(f"[measured] fwd {name}: max-norm err {err:.2e}, element-wise (entries >= 10% of max) {ew:.2e}", flush=True)
    assert ew <= ELEMENTWISE_TRAJ_TOL
    model = OB.forward_backward(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act,
                                folded=_folded(N, k, p["A"]))["bump_history"]
    assert O.max_rel_err(got, model) <= MODEL_TOL
    # per-step error must not blow up along the sequence either
    for t in (0, T // 2, T - 1):
        assert O.max_rel_err(got[t], ref[t]) <= TRAJ_TOL


@pytest.mark.parametrize("N,act", [(120, "tanh"), (256, "gelu"), (256, "relu")])
def test_decoded_angles_with_bump_sustaining_weights(N, act, gpu_device):
    """Decoded head direction is only well conditioned while a bump exists, so it is compared on the
    reference's own sanity recipe: cos(d), cos(d +- pi/4) weights (train/train_ring_attractor.py:94-103)."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    B, T = 64, 120
    print(f"[case] decode N={N} {act}", flush=True)
    p = make_problem(500, B, T, 2, N)
    idx = np.arange(N, dtype=np.float64)
    d = 2 * np.pi * (idx[:, None] - idx[None, :]) / N
    Wo = np.cos(d).astype(np.float32)
    Wa = np.stack([np.cos(d + np.pi / 4), np.cos(d - np.pi / 4)]).astype(np.float32)
    hist = ring_rnn_cuda_func(_dev(p["A"], gpu_device), _dev(Wa, gpu_device), -0.1, 0.1, _dev(Wo, gpu_device),
                              _dev(p["r0"], gpu_device), 0.15, act)
    got = hist.cpu().numpy().astype(np.float64)
    ref, _ = O.forward_dense(p["A"], Wa, -0.1, 0.1, Wo, p["r0"], 0.15, act)
    assert O.max_rel_err(got, ref) <= TRAJ_TOL
    dec_got = O.decode_angle_from_population_vector(O.readout(got.transpose(1, 0, 2)))
    dec_ref = O.decode_angle_from_population_vector(O.readout(ref.transpose(1, 0, 2)))
    diff = np.abs(np.angle(np.exp(1j * (dec_got - dec_ref))))
    assert diff.max() <= TRAJ_TOL * 2 * np.pi, f"decoded angle error {diff.max()} rad"
    # and the network does integrate: the reference's own sanity bound on the loss
    assert O.cosine_similarity_loss(O.readout(got.transpose(1, 0, 2)), p["angle"]) < 0.5


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_backward_weight_gradients(case, gpu_device):
    name, B, T, k, N, act, J0, J1, action = case
    print(f"[case] bwd {name} B={B} T={T} k={k} N={N} {act}", flush=True)
    p = _problem(200, B, T, k, N, action)
    hist, Wa, Wo = _run_op(p, J0, J1, act, gpu_device)
    hist.backward(_dev(p["G"], gpu_device))
    torch.cuda.synchronize()
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref_hist, p["r0"], 0.15, act)
    model = OB.forward_backward(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act, p["G"],
                                folded=_folded(N, k, p["A"]))
    gWo, gWa = Wo.grad.cpu().numpy(), Wa.grad.cpu().numpy()
    assert np.isfinite(gWo).all() and np.isfinite(gWa).all()
    assert np.abs(ref["grad_Wo"]).max() > 0, "degenerate case: the reference gradient is identically zero"
    smooth = act != "relu"
    model_tol = MODEL_TOL if smooth else GRAD_TOL      # a few borderline relu kinks also differ fp32 vs fp64
    assert O.cosine(gWo, ref["grad_Wo"]) >= GRAD_COS
    assert O.max_rel_err(gWo, model["grad_Wo"]) <= model_tol
    if smooth:
        assert O.max_rel_err(gWo, ref["grad_Wo"]) <= GRAD_TOL
        ew = O.elementwise_rel_err(gWo, ref["grad_Wo"])
        print(f"[measured] bwd {name}: grad_Wo element-wise (entries >= 10% of max) {ew:.2e}", flush=True)
        assert ew <= ELEMENTWISE_GRAD_TOL
    used = [c for c in range(k) if np.abs(p["A"][..., c]).max() > 0]
    for c in range(k):
        if c in used:
            assert O.cosine(gWa[c], ref["grad_Wa"][c]) >= GRAD_COS, f"Wa[{c}]"
            assert O.max_rel_err(gWa[c], model["grad_Wa"][c]) <= model_tol, f"Wa[{c}]"
            if smooth:
                assert O.max_rel_err(gWa[c], ref["grad_Wa"][c]) <= GRAD_TOL, f"Wa[{c}]"
        else:                       # an action channel that is identically zero has an exactly zero gradient
            assert np.abs(gWa[c]).max() == 0.0


_REBUILD_CASES = ("config0", "n256_gelu", "ragged_silu", "odd_shapes", "n1024_gelu", "n700_k16_pad", "n512_tanh", "n512_odd")


@pytest.mark.parametrize("case", [c for c in CASES if c[0] in _REBUILD_CASES], ids=lambda c: c[0])
def test_backward_without_saved_buffer_rebuilds_it(case, gpu_device):
    """bwd_cuda.bwd called the way the reference operator calls it (dummy re_history, reference workspaces
    absent): F'(re) is rebuilt from bump_history; the result agrees with the saved-buffer path to fp32
    summation-order noise (the two paths evaluate the pre-activation in a different order)."""
    from rnn_train_ring_attractor_amd import bwd_cuda
    name, B, T, k, N, act, J0, J1, action = case
    print(f"[case] bwd-rebuild {name}", flush=True)
    p = _problem(200, B, T, k, N, action)
    hist, Wa, Wo = _run_op(p, J0, J1, act, gpu_device)
    G = _dev(p["G"], gpu_device)
    hist.backward(G)
    gWa = torch.zeros_like(Wa)
    gWo = torch.zeros_like(Wo)
    g0 = torch.zeros(B, N, device=gpu_device)
    dummy = torch.empty(1, device=gpu_device, dtype=torch.bfloat16)
    bwd_cuda.bwd(grad_output=G, A=_dev(p["A"], gpu_device), Wa=Wa.detach(), J0=J0, J1=J1, Wo=Wo.detach(),
                 bump_history=hist.detach(), re_history=dummy, r_init=_dev(p["r0"], gpu_device),
                 grad_Wa=gWa, grad_Wo=gWo, alpha=0.15, activation_type=ACTS[act], grad_r_init=g0)
    torch.cuda.synchronize()
    assert O.max_rel_err(gWa.cpu().numpy(), Wa.grad.cpu().numpy()) <= 1e-3
    assert O.max_rel_err(gWo.cpu().numpy(), Wo.grad.cpu().numpy()) <= 1e-3
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref_hist, p["r0"], 0.15, act)
    assert O.cosine(g0.cpu().numpy(), ref["grad_r_init"]) >= GRAD_COS
    assert O.max_rel_err(g0.cpu().numpy(), ref["grad_r_init"]) <= GRAD_TOL


@pytest.mark.parametrize("B,T,k,N,act,action", [(40, 24, 2, 120, "tanh", "lr"), (48, 20, 2, 256, "gelu", "lr"),
                                                (21, 9, 3, 200, "silu", "dense"), (32, 12, 16, 64, "tanh", "spread"),
                                                (32, 7, 2, 256, "tanh", "dense"), (37, 10, 2, 200, "silu", "dense"),
                                                (64, 66, 2, 256, "relu", "lr"), (24, 6, 3, 700, "silu", "dense"),
                                                (20, 5, 2, 1024, "tanh", "lr"), (18, 4, 4, 1300, "gelu", "spread"),
                                                (1, 3, 2, 256, "gelu", "dense"), (1, 2, 2, 2048, "tanh", "dense"),
                                                (1, 1, 2, 40, "tanh", "dense"), (16, 3, 64, 640, "silu", "dense")],
                         ids=["n120", "n256", "ragged_k3", "k16", "n256_odd_T", "n200_ragged_resident", "n256_relu_T66",
                              "n700_k3_step", "n1024_step", "n1300_k4_step",
                              "one_sample_resident", "one_sample_n2048_step", "one_sample_one_step", "n640_k64_step"])
def test_gradients_of_action_signal_and_initial_state(B, T, k, N, act, action, gpu_device):
    """dL/d action_signal and dL/d r_init, which the reference operator does not return (cpp/ring_rnn_cuda.py:144);
    pinned by the fp64 oracle, whose grad_A / grad_r_init are themselves checked by finite differences."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print(f"[case] grad_A B={B} T={T} k={k} N={N} {act}", flush=True)
    p = _problem(400, B, T, k, N, action)
    # (relu with strong inhibition silences every neuron and all gradients are exactly zero: weak inhibition there)
    J0, J1 = (-1.0 / N, 1.0) if act == "relu" else (-0.05, 0.4)
    A = _dev(p["A"], gpu_device).requires_grad_(True)
    r0 = _dev(p["r0"], gpu_device).requires_grad_(True)
    Wa = _dev(p["Wa"], gpu_device).requires_grad_(True)
    Wo = _dev(p["Wo"], gpu_device).requires_grad_(True)
    hist = ring_rnn_cuda_func(A, Wa, J0, J1, Wo, r0, 0.15, act)
    hist.backward(_dev(p["G"], gpu_device))
    torch.cuda.synchronize()
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref_hist, p["r0"], 0.15, act)
    model = OB.forward_backward(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act, p["G"], folded=_folded(N, k))
    for name, got, want in (("grad_A", A.grad, ref["grad_A"]), ("grad_r_init", r0.grad, ref["grad_r_init"]),
                            ("grad_Wo", Wo.grad, ref["grad_Wo"]), ("grad_Wa", Wa.grad, ref["grad_Wa"])):
        got = got.cpu().numpy()
        assert got.shape == want.shape and np.isfinite(got).all(), name
        assert np.abs(want).max() > 0, name
        if act == "relu":
            # per-sample gradients do not average the derivative flips at the kink (see the note at the top): the
            # fp64 comparison is by cosine, the entry-wise bound is against the rounding-aware model
            assert O.cosine(got, want) >= 0.995, name
            assert O.max_rel_err(got, model[name]) <= GRAD_TOL, name
        else:
            assert O.cosine(got, want) >= GRAD_COS, name
            assert O.max_rel_err(got, want) <= GRAD_TOL, name


def test_gradients_accumulate_and_are_deterministic(gpu_device):
    from rnn_train_ring_attractor_amd import bwd_cuda
    B, T, k, N = 48, 20, 2, 256
    p = make_problem(300, B, T, k, N)
    hist, Wa, Wo = _run_op(p, -0.1, 0.1, "gelu", gpu_device)
    G = _dev(p["G"], gpu_device)
    hist.backward(G)
    outs = []
    for _ in range(2):
        gWa = torch.ones_like(Wa)          # pre-filled: the call must ADD to it
        gWo = torch.full_like(Wo, 2.0)
        bwd_cuda.bwd(grad_output=G, A=_dev(p["A"], gpu_device), Wa=Wa.detach(), J0=-0.1, J1=0.1, Wo=Wo.detach(),
                     bump_history=hist.detach(), r_init=_dev(p["r0"], gpu_device), grad_Wa=gWa, grad_Wo=gWo,
                     alpha=0.15, activation_type=1)
        outs.append((gWa, gWo))
    torch.cuda.synchronize()
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])     # bitwise repeatable
    # accumulation: result = prefill + gradient.  The rebuild path recomputes F' with fp32 row sums of the stored
    # history, the saved path took them over the bf16 operand copy: a difference at operand-rounding level.
    assert O.max_rel_err((outs[0][0] - 1.0).cpu().numpy(), Wa.grad.cpu().numpy()) <= MODEL_TOL
    assert O.max_rel_err((outs[0][1] - 2.0).cpu().numpy(), Wo.grad.cpu().numpy()) <= MODEL_TOL
    # accumulate=False: the buffers are written, whatever they held (here NaN), to exactly the accumulated sums
    gWa = torch.full_like(Wa, float("nan"))
    gWo = torch.full_like(Wo, float("nan"))
    bwd_cuda.bwd(grad_output=G, A=_dev(p["A"], gpu_device), Wa=Wa.detach(), J0=-0.1, J1=0.1, Wo=Wo.detach(),
                 bump_history=hist.detach(), r_init=_dev(p["r0"], gpu_device), grad_Wa=gWa, grad_Wo=gWo,
                 alpha=0.15, activation_type=1, accumulate=False)
    zWa, zWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
    bwd_cuda.bwd(grad_output=G, A=_dev(p["A"], gpu_device), Wa=Wa.detach(), J0=-0.1, J1=0.1, Wo=Wo.detach(),
                 bump_history=hist.detach(), r_init=_dev(p["r0"], gpu_device), grad_Wa=zWa, grad_Wo=zWo,
                 alpha=0.15, activation_type=1)
    torch.cuda.synchronize()
    assert torch.equal(gWa, zWa) and torch.equal(gWo, zWo)


def test_alpha_zero_and_zero_weights_closed_forms(gpu_device):
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    B, T, k, N = 32, 6, 2, 128
    p = make_problem(400, B, T, k, N)
    A, r0 = _dev(p["A"], gpu_device), _dev(p["r0"], gpu_device)
    Wa, Wo = _dev(p["Wa"], gpu_device), _dev(p["Wo"], gpu_device)
    frozen = ring_rnn_cuda_func(A, Wa, -0.1, 0.1, Wo, r0, 0.0, "gelu")
    assert torch.equal(frozen, r0.expand(T, B, N))
    decay = ring_rnn_cuda_func(A, torch.zeros_like(Wa), 0.0, 1.0, torch.zeros_like(Wo), r0, 0.15, "tanh")
    for t in range(T):
        torch.testing.assert_close(decay[t], r0 * 0.85 ** (t + 1), rtol=1e-5, atol=1e-8)


@pytest.mark.parametrize("N", [256, 200], ids=["resident", "streaming"])
def test_saved_buffer_that_was_copied_or_lands_on_a_stale_note(N, gpu_device):
    """The forward leaves a transposed weight copy behind the saved activations and remembers, under the buffer's
    address, what it packed (family, shape, J0, J1, weight tensors).  A backward must trust that copy only on an exact
    match: a clone of the buffer (no note at its address) and a buffer whose address still carries the note of an
    EARLIER forward with another J1 (whose packed Wo would be folded differently) both have to give the bits of the
    backward that consumes the original buffer."""
    from rnn_train_ring_attractor_amd.rnn_cuda import fwd_cuda, bwd_cuda, saved_nbytes
    B, T, k = 48, 12, 2
    print(f"[case] saved-buffer notes N={N} B={B} T={T}", flush=True)
    p = _problem(300, B, T, k, N, "lr")
    A, Wa, Wo, r0, G = (_dev(p[x], gpu_device) for x in ("A", "Wa", "Wo", "r0", "G"))
    nbytes = saved_nbytes(N, k, T, B)

    def forward(J1, saved):
        hist = torch.empty(T, B, N, device=gpu_device)
        fwd_cuda.fwd(A=A, Wa=Wa, J0=-0.05, J1=J1, Wo=Wo, r_init=r0, bump_history=hist, alpha=0.15,
                     activation_type=ACTS["gelu"], saved=saved)
        return hist

    def backward(J1, hist, saved):
        gWa, gWo = torch.empty_like(Wa), torch.empty_like(Wo)
        bwd_cuda.bwd(grad_output=G, A=A, Wa=Wa, J0=-0.05, J1=J1, Wo=Wo, bump_history=hist, r_init=r0, grad_Wa=gWa,
                     grad_Wo=gWo, alpha=0.15, activation_type=ACTS["gelu"], saved=saved, accumulate=False)
        return gWa, gWo

    stale = torch.empty(nbytes, dtype=torch.uint8, device=gpu_device)
    forward(0.9, stale)                                  # leaves a note for J1 = 0.9 under stale's address
    saved = torch.empty(nbytes, dtype=torch.uint8, device=gpu_device)
    hist = forward(0.4, saved)
    want = backward(0.4, hist, saved)
    clone = saved.clone()                                # an address the library has never seen
    got_clone = backward(0.4, hist, clone)
    stale.copy_(saved)                                   # right contents, wrong note
    got_stale = backward(0.4, hist, stale)
    torch.cuda.synchronize()
    for got in (got_clone, got_stale):
        for x, y in zip(got, want):
            assert torch.equal(x, y)
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], -0.05, 0.4, p["Wo"], p["r0"], 0.15, "gelu")
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], -0.05, 0.4, p["Wo"], ref_hist, p["r0"], 0.15, "gelu")
    assert O.max_rel_err(want[1].cpu().numpy(), ref["grad_Wo"]) <= GRAD_TOL


def _self_check_recipe(seed, B, T, k, N):
    """Inputs of the reference's own forward + backward comparison (legacy/bwd_fp32.py:486-507): weights, action
    signal and initial state all ~ N(0, 1), UNSCALED (so gates and states are signed and the state grows by an order
    of magnitude per step), and a random target for an MSE loss (:612-619)."""
    rng = np.random.default_rng(seed)
    return dict(Wa=rng.standard_normal((k, N, N)).astype(np.float32), Wo=rng.standard_normal((N, N)).astype(np.float32),
                A=rng.standard_normal((B, T, k)).astype(np.float32), r0=rng.standard_normal((B, N)).astype(np.float32),
                gt=rng.standard_normal((T, B, N)).astype(np.float32))


SELF_CHECK = [
    # name,                 B,  T,  k,    N, act      (J0 = -0.1, J1 = 0.1 as legacy/bwd_fp32.py:488-489)
    ("reference_recipe",  256,  4, 16,  512, "silu"),   # the reference's own shape (legacy/bwd_fp32.py:587-594 region)
    ("resident_signed",    64,  4,  2,  256, "silu"),   # signed dense gates on the weight-resident kernels
    ("streaming_signed",   64,  5,  3,  200, "silu"),   # ... the persistent streaming kernels
    ("step_signed",        32,  3,  3, 1024, "silu"),   # ... the step-per-launch kernels
]


@pytest.mark.parametrize("case", SELF_CHECK, ids=[c[0] for c in SELF_CHECK])
def test_reference_self_check_recipe(case, gpu_device):
    """The one forward + backward comparison the reference itself holds (legacy/bwd_fp32.py:486-507, 587-660): MSE
    against a random target, gradients of Wa and Wo, on unscaled N(0, 1) weights, signed gates and signed states.
    The trajectory meets the 1e-2 bound against fp64.  The weight gradients are held to cosine >= 0.998 against
    fp64 (the CPU model of the bf16 operands alone reaches 0.99903 for grad_Wa at the reference's shape) and to the
    rounding-aware model (same bf16 operands, fp64 sums): on this recipe the state grows ~10 x per
    step and the Jacobian's norm is ~14, and bf16 operand rounding alone moves the largest gradient entries by
    1e-2 .. 4e-1 of the largest (measured on the CPU model: grad_Wo 0.17, grad_Wa 0.36 at the reference's shape),
    so the 2e-2 max-norm bound is not one a bf16-operand implementation can meet here -- the reference's own WMMA
    path rounds the same operands (cpp/kernels/fwd_1loop_tc_idx.cuh:6-48) and its check is off by default with
    loosened tolerances (legacy/bwd_fp32.py:641-660)."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    name, B, T, k, N, act = case
    J0, J1 = -0.1, 0.1
    print(f"[case] self-check {name} B={B} T={T} k={k} N={N} {act}", flush=True)
    p = _self_check_recipe(7, B, T, k, N)
    A, r0, gt = _dev(p["A"], gpu_device), _dev(p["r0"], gpu_device), _dev(p["gt"], gpu_device)
    Wa, Wo = _dev(p["Wa"], gpu_device).requires_grad_(True), _dev(p["Wo"], gpu_device).requires_grad_(True)
    hist = ring_rnn_cuda_func(A, Wa, J0, J1, Wo, r0, 0.15, act)
    torch.nn.functional.mse_loss(hist, gt).backward()
    torch.cuda.synchronize()
    got = hist.detach().cpu().numpy().astype(np.float64)
    ref, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    assert np.isfinite(got).all()
    terr = O.max_rel_err(got, ref)
    G_ref = (2.0 * (ref - p["gt"]) / ref.size)
    rb = O.backward_dense(G_ref, p["A"], p["Wa"], J0, J1, p["Wo"], ref, p["r0"], 0.15, act)
    G_hip = (2.0 * (got - p["gt"]) / got.size).astype(np.float32)
    model = OB.forward_backward(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act, G_hip, folded=_folded(N, k))
    gWo, gWa = Wo.grad.cpu().numpy(), Wa.grad.cpu().numpy()
    assert np.isfinite(gWo).all() and np.isfinite(gWa).all()
    e_o, e_a = O.max_rel_err(gWo, rb["grad_Wo"]), O.max_rel_err(gWa, rb["grad_Wa"])
    m_o, m_a = O.max_rel_err(gWo, model["grad_Wo"]), O.max_rel_err(gWa, model["grad_Wa"])
    print(f"[measured] self-check {name}: trajectory {terr:.2e}; vs fp64 grad_Wo {e_o:.2e} grad_Wa {e_a:.2e} "
          f"(cos {O.cosine(gWo, rb['grad_Wo']):.5f} {O.cosine(gWa, rb['grad_Wa']):.5f}); vs rounding model "
          f"grad_Wo {m_o:.2e} grad_Wa {m_a:.2e}", flush=True)
    assert terr <= TRAJ_TOL
    for t in range(T):
        assert O.max_rel_err(got[t], ref[t]) <= TRAJ_TOL
    assert O.cosine(gWo, rb["grad_Wo"]) >= 0.998 and O.cosine(gWa, rb["grad_Wa"]) >= 0.998
    assert O.max_rel_err(got, model["bump_history"]) <= MODEL_TOL
    # measured against the model: 1.2e-2 / 2.1e-2 at the reference's shape (fp32 against fp64 sums, amplified as above)
    assert m_o <= 2 * GRAD_TOL and m_a <= 2 * GRAD_TOL


@pytest.mark.parametrize("B,T,k,N,act", [(48, 14, 2, 256, "gelu"), (40, 9, 2, 200, "tanh"), (24, 5, 3, 640, "silu")],
                         ids=["resident", "streaming", "step"])
def test_operator_switches_recompute_and_precise_wo(B, T, k, N, act, gpu_device):
    """The two module-level switches of the Python operator.  RECOMPUTE_IN_BACKWARD: the forward keeps no saved
    record and the backward rebuilds it (gradients agree with the stored-record path to summation-order noise,
    bitwise where the rebuild re-runs the same kernel).  precise_wo: Wo as two bf16 operands through one more action
    matrix with the constant gate J1 -- same output and gradient shapes, gradients of Wa, Wo, the action signal and
    the initial state against the fp64 oracle, and a trajectory at least as close to fp64 as the bf16-Wo one."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda as op
    print(f"[case] operator switches B={B} T={T} k={k} N={N} {act}", flush=True)
    J0, J1 = -0.05, 0.6
    p = _problem(400, B, T, k, N, "dense")
    ref_hist, _ = O.forward_dense(p["A"], p["Wa"], J0, J1, p["Wo"], p["r0"], 0.15, act)
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], J0, J1, p["Wo"], ref_hist, p["r0"], 0.15, act)

    def run(**kw):
        A = _dev(p["A"], gpu_device).requires_grad_(True)
        r0 = _dev(p["r0"], gpu_device).requires_grad_(True)
        Wa, Wo = _dev(p["Wa"], gpu_device).requires_grad_(True), _dev(p["Wo"], gpu_device).requires_grad_(True)
        h = op.ring_rnn_cuda_func(A, Wa, J0, J1, Wo, r0, 0.15, act, **kw)
        h.backward(_dev(p["G"], gpu_device))
        torch.cuda.synchronize()
        return [x.detach().cpu().numpy() for x in (h, Wa.grad, Wo.grad, A.grad, r0.grad)]

    base = run()
    assert op.RECOMPUTE_IN_BACKWARD is False and op.PRECISE_WO is False
    op.RECOMPUTE_IN_BACKWARD = True
    try:
        rec = run()
    finally:
        op.RECOMPUTE_IN_BACKWARD = False
    assert np.array_equal(rec[0], base[0])
    for x, y in zip(rec[1:], base[1:]):
        assert O.max_rel_err(x, y) <= 1e-3
    pre = run(precise_wo=True)
    assert [x.shape for x in pre] == [x.shape for x in base]
    e_pre, e_base = O.max_rel_err(pre[0], ref_hist), O.max_rel_err(base[0], ref_hist)
    print(f"[measured] trajectory vs fp64: bf16 Wo {e_base:.2e}, Wo as hi + lo {e_pre:.2e}", flush=True)
    assert e_pre <= TRAJ_TOL and e_pre <= 1.2 * e_base + 1e-4
    for got, key in zip(pre[1:], ("grad_Wa", "grad_Wo", "grad_A", "grad_r_init")):
        assert O.cosine(got, ref[key]) >= GRAD_COS, key
        assert O.max_rel_err(got, ref[key]) <= GRAD_TOL, key
