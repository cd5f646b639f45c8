"""GPU tests of the N = 512 cluster forward (four compute units of one XCD keep the weights on chip and exchange the
state through L2): parity with the fp64 oracle and the rounding model on a subset of batch rows (rows are independent),
agreement with the streaming kernels, run-to-run reproducibility (a race between cluster members would show as a
difference between two runs), the choice of kernel by shape, and the exit taken when a wait runs out.

RINGATTR_CLUSTER=1 makes the kernel run on every shape it can (whole pairs of batch tiles); left alone it only takes
shapes with at least four pairs per cluster, where it is ahead.  The BPTT on the same clusters runs only under
RINGATTR_CLUSTER_BPTT=1 (it is not ahead of the streaming kernel anywhere); its tests compare it with that kernel on
the same saved record, with the fp64 oracle where the CPU can afford the batch, and run to run."""
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from oracle import ring_oracle_bf16 as OB
from tests.ring_cases import make_problem

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ACTS = {"relu": 0, "gelu": 1, "tanh": 2, "silu": 3}
N, K = 512, 2
TRAJ_TOL = 1e-2
MODEL_TOL = 5e-3
GRAD_COS = 0.999
GRAD_TOL = 2e-2

# name, B, T, act, action: one pair (both halves in phase), two pairs per cluster (the late half's epilogue is awaited by
# the very next staging), four pairs (the full rotation), odd length, a single step, clusters with unequal pair counts
CASES = [
    ("one_pair",          32,  9, "tanh", "dense"),
    ("one_step",          64,  1, "gelu", "dense"),
    ("pairs_over_xcds",  416,  6, "silu", "lr"),       # 13 clusters: XCDs with one and with two
    ("two_per_cluster", 2112,  5, "tanh", "dense"),    # 66 pairs over 33 clusters
    ("four_per_cluster", 8192, 6, "gelu", "lr"),
    ("uneven_rotation", 6400,  7, "tanh", "dense"),    # 200 pairs: clusters with three and with four
]


def _t(x, dev):
    return torch.tensor(x, device=dev)


def _forward(p, act, dev, saved=True):
    from rnn_train_ring_attractor_amd import rnn_cuda
    A, Wa, Wo, r0 = (_t(p[k], dev) for k in ("A", "Wa", "Wo", "r0"))
    B, T = p["A"].shape[:2]
    hist = torch.full((T, B, N), float("nan"), device=dev)
    sv = torch.zeros(rnn_cuda.saved_nbytes(N, K, T, B), dtype=torch.uint8, device=dev) if saved else None
    rnn_cuda._Fwd.fwd(A, Wa, -0.1, 0.1, Wo, r0, hist, 0.15, ACTS[act], saved=sv)
    torch.cuda.synchronize()
    return hist, sv


def _backward(p, act, dev, hist, sv):
    from rnn_train_ring_attractor_amd import rnn_cuda
    A, Wa, Wo, r0, G = (_t(p[k], dev) for k in ("A", "Wa", "Wo", "r0", "G"))
    gWa, gWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
    rnn_cuda._Bwd.bwd(G, A, Wa, -0.1, 0.1, Wo, hist, r_init=r0, grad_Wa=gWa, grad_Wo=gWo, alpha=0.15,
                      activation_type=ACTS[act], saved=sv)
    torch.cuda.synchronize()
    return gWa.cpu().numpy().astype(np.float64), gWo.cpu().numpy().astype(np.float64)


def _rows(B):
    """Batch rows the CPU references are run on: the first and last pair of tiles and one in the middle."""
    pick = sorted(set(list(range(0, min(B, 32))) + list(range(max(0, B // 2 - 8), min(B, B // 2 + 8))) + list(range(max(0, B - 32), B))))
    return np.array(pick)


def _fwd_kernel_name():
    from rnn_train_ring_attractor_amd import _lib
    return _lib.last_kernel_names().get("fwd", "")


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_cluster_forward_against_the_oracle_and_the_streaming_kernels(case, gpu_device, monkeypatch):
    name, B, T, act, action = case
    print(f"[case] cluster fwd {name} B={B} T={T} {act} {action}", flush=True)
    p = make_problem(311, B, T, K, N, action=action)
    monkeypatch.setenv("RINGATTR_CLUSTER", "0")
    h_stream, s_stream = _forward(p, act, gpu_device)
    assert "cluster" not in _fwd_kernel_name()
    monkeypatch.setenv("RINGATTR_CLUSTER", "1")
    h, s = _forward(p, act, gpu_device)
    assert "ring_fwd_cluster8_kernel" in _fwd_kernel_name()
    got = h.cpu().numpy().astype(np.float64)
    assert np.isfinite(got).all()
    rows = _rows(B)
    ref, _ = O.forward_dense(p["A"][rows], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"][rows], 0.15, act)
    err = O.max_rel_err(got[:, rows], ref)
    model = OB.forward_backward(p["A"][rows], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"][rows], 0.15, act, folded=True)["bump_history"]
    merr = O.max_rel_err(got[:, rows], model)
    serr = O.max_rel_err(got, h_stream.cpu().numpy().astype(np.float64))
    print(f"[measured] {name}: vs fp64 {err:.2e}, vs rounding model {merr:.2e}, vs streaming kernels (all rows) {serr:.2e}", flush=True)
    # (the two kernels round Wo differently -- J1 * Wo + J0 folded into one matrix here -- so each is held to the fp64
    # bound and to its own rounding model, and the two to each other only as far as those bounds allow)
    assert err <= TRAJ_TOL and merr <= MODEL_TOL and serr <= TRAJ_TOL
    # the record it leaves is what the streaming backward reads: gradients from either forward agree, and match fp64
    # where the CPU can afford the whole batch
    ga, go = _backward(p, act, gpu_device, h, s)
    ga_s, go_s = _backward(p, act, gpu_device, h_stream, s_stream)
    tol = 6e-2 if act == "relu" else 1e-2   # (relu: derivative flips where the two forwards round a pre-activation apart)
    assert O.max_rel_err(go, go_s) <= tol and O.max_rel_err(ga, ga_s) <= tol
    if B <= 512:
        ref_h, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, act)
        g = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.1, p["Wo"], ref_h, p["r0"], 0.15, act)
        assert O.cosine(go, g["grad_Wo"]) >= GRAD_COS and O.cosine(ga, g["grad_Wa"]) >= GRAD_COS
        assert O.max_rel_err(go, g["grad_Wo"]) <= GRAD_TOL and O.max_rel_err(ga, g["grad_Wa"]) <= GRAD_TOL


def test_cluster_forward_without_a_record_and_rebuilt_record(gpu_device, monkeypatch):
    """Inference (nothing saved) gives the same history; a backward without the record rebuilds it from that history."""
    B, T, act = 8192, 5, "tanh"
    print(f"[case] cluster fwd without record B={B} T={T}", flush=True)
    p = make_problem(312, B, T, K, N, action="lr")
    monkeypatch.setenv("RINGATTR_CLUSTER", "1")
    h_saved, s = _forward(p, act, gpu_device)
    h_plain, _ = _forward(p, act, gpu_device, saved=False)
    assert "ring_fwd_cluster8_kernel" in _fwd_kernel_name()
    assert torch.equal(h_saved, h_plain)
    ga, go = _backward(p, act, gpu_device, h_saved, s)
    ga_r, go_r = _backward(p, act, gpu_device, h_plain, None)
    print(f"[measured] gradients with the forward's record vs a rebuilt one: {O.max_rel_err(go_r, go):.2e}, {O.max_rel_err(ga_r, ga):.2e}", flush=True)
    assert O.max_rel_err(go_r, go) <= 1e-2 and O.max_rel_err(ga_r, ga) <= 1e-2


def test_cluster_forward_is_reproducible_run_to_run(gpu_device, monkeypatch):
    """The members of a cluster synchronize through flags in memory; the arithmetic has one order.  Any run that read an
    operand before it was complete would differ from the others."""
    monkeypatch.setenv("RINGATTR_CLUSTER", "1")
    for (B, T, act) in ((8192, 24, "tanh"), (2112, 12, "gelu"), (96, 30, "silu")):
        print(f"[case] cluster fwd reproducibility B={B} T={T} {act}", flush=True)
        p = make_problem(313, B, T, K, N, action="dense")
        h0, s0 = _forward(p, act, gpu_device)
        for _ in range(5):
            h, s = _forward(p, act, gpu_device)
            assert torch.equal(h, h0) and torch.equal(s, s0)


def test_cluster_forwards_on_two_streams(gpu_device, monkeypatch):
    """Every cluster kernel wants all compute units for its own workgroups.  Two of them launched back to back on two
    streams still both finish with the right result (the second one's workgroups become resident as the first one's
    leave; every wait for a sibling is bounded in any case)."""
    from rnn_train_ring_attractor_amd import rnn_cuda
    monkeypatch.setenv("RINGATTR_CLUSTER", "1")
    B, T, act = 8192, 48, "tanh"
    print(f"[case] two cluster forwards on two streams B={B} T={T}", flush=True)
    p = make_problem(316, B, T, K, N, action="lr")
    A, Wa, Wo, r0 = (_t(p[k], gpu_device) for k in ("A", "Wa", "Wo", "r0"))
    ref, _ = _forward(p, act, gpu_device, saved=False)
    assert "ring_fwd_cluster8_kernel" in _fwd_kernel_name()
    streams = [torch.cuda.Stream(device=gpu_device) for _ in range(2)]
    out = [torch.full((T, B, N), float("nan"), device=gpu_device) for _ in range(2)]
    torch.cuda.synchronize()
    for _ in range(3):
        for st, h in zip(streams, out):
            with torch.cuda.stream(st):
                rnn_cuda._Fwd.fwd(A, Wa, -0.1, 0.1, Wo, r0, h, 0.15, ACTS[act])
        torch.cuda.synchronize()
        assert torch.equal(out[0], ref) and torch.equal(out[1], ref)
    _forward(p, act, gpu_device, saved=False)      # (a member that had given up would be reported by this call)
    assert "ring_fwd_cluster8_kernel" in _fwd_kernel_name()


def test_kernel_choice_by_shape(gpu_device, monkeypatch):
    """Unasked, the cluster kernel takes shapes with at least four batch-tile pairs per cluster; RINGATTR_CLUSTER=0
    keeps it off, and shapes it cannot run (ragged batch, other widths) never see it."""
    monkeypatch.delenv("RINGATTR_CLUSTER", raising=False)
    for (B, T, n, want) in ((8192, 16, 512, True), (4096, 16, 512, False), (8192, 8, 512, False), (8200, 16, 512, False)):
        print(f"[case] kernel choice B={B} T={T} N={n}", flush=True)
        p = make_problem(314, B, T, K, n, action="lr")
        _forward(p, "tanh", gpu_device, saved=False)
        assert ("cluster" in _fwd_kernel_name()) == want, (B, T, n, _fwd_kernel_name())
    monkeypatch.setenv("RINGATTR_CLUSTER", "0")
    p = make_problem(314, 8192, 16, K, 512, action="lr")
    _forward(p, "tanh", gpu_device, saved=False)
    assert "cluster" not in _fwd_kernel_name()


# name, B, T, act, grad_r_init asked for
BPTT_CASES = [
    ("one_pair_odd_length",  32,  9, "tanh", True),
    ("one_pair_even_length", 32,  8, "tanh", False),
    ("one_step",             64,  1, "gelu", True),
    ("pairs_over_xcds",     416,  6, "silu", True),
    ("two_per_cluster",    2112,  5, "tanh", False),
    ("four_per_cluster",   8192,  6, "gelu", True),
    ("uneven_rotation",    6400,  7, "tanh", True),
]


def _backward_full(p, act, dev, hist, sv, want_r_init):
    from rnn_train_ring_attractor_amd import rnn_cuda
    A, Wa, Wo, r0, G = (_t(p[k], dev) for k in ("A", "Wa", "Wo", "r0", "G"))
    gWa, gWo = torch.zeros_like(Wa), torch.zeros_like(Wo)
    gr = torch.full_like(r0, float("nan")) if want_r_init else None
    rnn_cuda._Bwd.bwd(G, A, Wa, -0.1, 0.1, Wo, hist, r_init=r0, grad_Wa=gWa, grad_Wo=gWo, alpha=0.15,
                      activation_type=ACTS[act], saved=sv, grad_r_init=gr)
    torch.cuda.synchronize()
    return gWa.cpu().numpy().astype(np.float64), gWo.cpu().numpy().astype(np.float64), \
        (gr.cpu().numpy().astype(np.float64) if want_r_init else None)


def _bptt_kernel_name():
    from rnn_train_ring_attractor_amd import _lib
    return _lib.last_kernel_names().get("bptt", "")


@pytest.mark.parametrize("case", BPTT_CASES, ids=[c[0] for c in BPTT_CASES])
def test_cluster_bptt_against_the_streaming_kernel_and_the_oracle(case, gpu_device, monkeypatch):
    from rnn_train_ring_attractor_amd import rnn_cuda
    name, B, T, act, want_r_init = case
    print(f"[case] cluster bptt {name} B={B} T={T} {act} grad_r_init={want_r_init}", flush=True)
    p = make_problem(411, B, T, K, N, action="dense")
    monkeypatch.setenv("RINGATTR_CLUSTER", "0")
    hist, sv = _forward(p, act, gpu_device)
    ga_s, go_s, gr_s = _backward_full(p, act, gpu_device, hist, sv, want_r_init)
    assert "cluster" not in _bptt_kernel_name()
    # the cluster kernel's scratch (carry records, held halves, the exchange, the copy of g with its zero tail) starts
    # out as NaN patterns: whatever it read before writing it would show
    plain_workspace = rnn_cuda._workspace
    monkeypatch.setattr(rnn_cuda, "_workspace",
                        lambda nbytes, device, stream: plain_workspace(nbytes, device, stream).fill_(0xFF))
    monkeypatch.setenv("RINGATTR_CLUSTER", "1")
    monkeypatch.setenv("RINGATTR_CLUSTER_BPTT", "1")
    ga, go, gr = _backward_full(p, act, gpu_device, hist, sv, want_r_init)
    assert "ring_bptt_cluster8_kernel" in _bptt_kernel_name()
    ga2, go2, gr2 = _backward_full(p, act, gpu_device, hist, sv, want_r_init)
    assert np.isfinite(ga).all() and np.isfinite(go).all()
    errs = [O.max_rel_err(ga, ga_s), O.max_rel_err(go, go_s)]
    if want_r_init:
        assert np.isfinite(gr).all()
        errs.append(O.max_rel_err(gr, gr_s))
    print(f"[measured] {name}: vs the streaming BPTT " + ", ".join(f"{e:.2e}" for e in errs), flush=True)
    assert max(errs) <= 1e-2
    # one order of arithmetic, flags in memory between the members: a read of an incomplete operand would differ run to run
    assert np.array_equal(ga, ga2) and np.array_equal(go, go2) and (not want_r_init or np.array_equal(gr, gr2))
    if B <= 512:
        ref_h, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, act)
        g = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.1, p["Wo"], ref_h, p["r0"], 0.15, act)
        assert O.cosine(go, g["grad_Wo"]) >= GRAD_COS and O.cosine(ga, g["grad_Wa"]) >= GRAD_COS
        assert O.max_rel_err(go, g["grad_Wo"]) <= GRAD_TOL and O.max_rel_err(ga, g["grad_Wa"]) <= GRAD_TOL
        if want_r_init:
            assert O.max_rel_err(gr, g["grad_r_init"]) <= GRAD_TOL


def test_cluster_bptt_runs_only_where_asked_for(gpu_device, monkeypatch):
    monkeypatch.delenv("RINGATTR_CLUSTER", raising=False)
    monkeypatch.delenv("RINGATTR_CLUSTER_BPTT", raising=False)
    p = make_problem(412, 8192, 16, K, N, action="lr")
    hist, sv = _forward(p, "tanh", gpu_device)
    assert "cluster" in _fwd_kernel_name()
    _backward_full(p, "tanh", gpu_device, hist, sv, False)
    assert "cluster" not in _bptt_kernel_name(), _bptt_kernel_name()
    monkeypatch.setenv("RINGATTR_CLUSTER_BPTT", "1")
    _backward_full(p, "tanh", gpu_device, hist, sv, False)
    assert "ring_bptt_cluster8_kernel" in _bptt_kernel_name()
    monkeypatch.setenv("RINGATTR_CLUSTER", "0")          # the forward's switch turns both off
    _backward_full(p, "tanh", gpu_device, hist, sv, False)
    assert "cluster" not in _bptt_kernel_name()


_GIVE_UP_SCRIPT = r"""
import os, sys
sys.path.insert(0, {root!r})
os.environ["RINGATTR_CLUSTER"] = "1"
os.environ["RINGATTR_CLUSTER_SPIN"] = "-1"      # every cluster member gives up its first wait at once
import numpy as np, torch
from tests.ring_cases import make_problem
from rnn_train_ring_attractor_amd import rnn_cuda, _lib
dev = torch.device("cuda:0")
p = make_problem(315, 64, 6, 2, 512, action="dense")
A, Wa, Wo, r0 = (torch.tensor(p[k], device=dev) for k in ("A", "Wa", "Wo", "r0"))
def fwd():
    hist = torch.full((6, 64, 512), float("nan"), device=dev)
    rnn_cuda._Fwd.fwd(A, Wa, -0.1, 0.1, Wo, r0, hist, 0.15, 2)
    torch.cuda.synchronize()
    return hist
print("[case] cluster forward whose members give up", flush=True)
h = fwd()                                         # the launch itself succeeds; the kernel leaves at its first wait
assert "cluster" in _lib.last_kernel_names()["fwd"], _lib.last_kernel_names()
try:
    fwd()
    print("no error reported")
    sys.exit(1)
except Exception as e:                            # reported once, by the next call
    assert "gave up waiting" in str(e), str(e)
    print("reported:", str(e)[:60], flush=True)
os.environ["RINGATTR_CLUSTER_SPIN"] = "1000000"
h2 = fwd()                                        # from here on the streaming kernels do the work
assert "cluster" not in _lib.last_kernel_names()["fwd"]
os.environ["RINGATTR_CLUSTER"] = "0"
h3 = fwd()
assert torch.isfinite(h2).all() and torch.equal(h2, h3)
print("give-up path ok")
"""


def test_a_wait_that_runs_out_is_reported_once_and_the_streaming_kernels_take_over(gpu_device):
    """The kernel's waits are bounded.  With the bound set to 'at once' from the host every workgroup leaves at its
    start-up handshake (the kernel ends normally); the library reports that on the next call and stops using the
    cluster kernel.  In a process of its own, since that switch is for good."""
    proc = subprocess.run([sys.executable, "-c", _GIVE_UP_SCRIPT.format(root=ROOT)], capture_output=True, text=True, timeout=300,
                          cwd=ROOT)
    print(proc.stdout[-1500:], proc.stderr[-1500:], flush=True)
    assert proc.returncode == 0 and "give-up path ok" in proc.stdout
