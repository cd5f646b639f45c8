"""The operator under HIP graph capture: forward + backward recorded once, replayed on new inputs.

Nothing on the operator path allocates through HIP, synchronises or reads the device back, so a caller may record a
training step into a graph.  Every replay is checked against an eager run on the same inputs (the kernels sum in a
fixed order, so the comparison is bitwise), with eager work and synchronisations between the replays."""
import numpy as np
import pytest
import torch

from tests.ring_cases import make_problem

pytestmark = pytest.mark.gpu

CASES = [
    # name,        B,  T, k,   N, act, environment
    ("resident",  48, 10, 2, 256, "gelu", {}),
    ("streaming", 40, 12, 2, 120, "tanh", {}),
    ("step",      24,  5, 3, 640, "silu", {}),
    # the N = 512 kernels on clusters of compute units: their flags are cleared by a kernel of the captured stream
    ("cluster_forward", 96, 7, 2, 512, "tanh", {"RINGATTR_CLUSTER": "1"}),
    ("cluster_forward_and_bptt", 64, 6, 2, 512, "gelu", {"RINGATTR_CLUSTER": "1", "RINGATTR_CLUSTER_BPTT": "1"}),
]


@pytest.mark.parametrize("case", CASES, ids=[c[0] for c in CASES])
def test_forward_backward_replays_from_a_graph(case, gpu_device, monkeypatch):
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func, _lib
    name, B, T, k, N, act, env = case
    for key in ("RINGATTR_CLUSTER", "RINGATTR_CLUSTER_BPTT"):
        monkeypatch.delenv(key, raising=False)
    for key, val in env.items():
        monkeypatch.setenv(key, val)
    print(f"[case] graph {name} B={B} T={T} k={k} N={N} {act}", flush=True)
    J0, J1 = -0.05, 0.4
    problems = [make_problem(900 + i, B, T, k, N, action="dense") for i in range(3)]

    def dev(x):
        return torch.tensor(x, device=gpu_device)

    p0 = problems[0]
    A, r0, G = dev(p0["A"]), dev(p0["r0"]), dev(p0["G"])
    Wa, Wo = dev(p0["Wa"]).requires_grad_(True), dev(p0["Wo"]).requires_grad_(True)

    def step(A, Wa, Wo, r0, G):
        hist = ring_rnn_cuda_func(A, Wa, J0, J1, Wo, r0, 0.15, act)
        hist.backward(G)
        return hist

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):                       # the allocator and lazily initialised state settle outside the capture
            Wa.grad = Wo.grad = None
            step(A, Wa, Wo, r0, G)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    Wa.grad = Wo.grad = None
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        hist = step(A, Wa, Wo, r0, G)

    for rep, p in enumerate(problems[::-1] + problems[:1]):
        with torch.no_grad():
            for dst, key in ((A, "A"), (r0, "r0"), (G, "G"), (Wa, "Wa"), (Wo, "Wo")):
                dst.copy_(dev(p[key]))
        graph.replay()
        torch.cuda.synchronize()
        got = (hist.detach().clone(), Wa.grad.clone(), Wo.grad.clone())
        # the same inputs through the eager path (its own tensors), with a synchronisation before the next replay
        eWa, eWo = dev(p["Wa"]).requires_grad_(True), dev(p["Wo"]).requires_grad_(True)
        ehist = step(dev(p["A"]), eWa, eWo, dev(p["r0"]), dev(p["G"]))
        torch.cuda.synchronize()
        assert np.isfinite(got[0].cpu().numpy()).all()
        assert torch.equal(got[0], ehist.detach()), f"replay {rep}: history differs from the eager run"
        assert torch.equal(got[1], eWa.grad), f"replay {rep}: grad_Wa differs from the eager run"
        assert torch.equal(got[2], eWo.grad), f"replay {rep}: grad_Wo differs from the eager run"
        assert float(got[1].abs().max()) > 0
    names = _lib.last_kernel_names()
    assert ("cluster" in names.get("fwd", "")) == ("RINGATTR_CLUSTER" in env)
    assert ("cluster" in names.get("bptt", "")) == ("RINGATTR_CLUSTER_BPTT" in env)


def test_device_counted_optimizer_matches_the_host_counted_one(gpu_device):
    """FusedClipAdam(capturable=True) keeps Adam's step number on the device; five steps agree with the variant that
    receives the number from the host, and the counter has advanced once per step."""
    from rnn_train_ring_attractor_amd import FusedClipAdam
    print("[case] counted clip + Adam", flush=True)
    torch.manual_seed(5)
    shapes = [(256, 256), (2, 256, 256), (16,), (5000,)]
    init = [torch.randn(s, device=gpu_device) for s in shapes]
    host = [x.clone().requires_grad_(True) for x in init]
    counted = [x.clone().requires_grad_(True) for x in init]
    opt_h = FusedClipAdam(host, lr=3e-3, betas=(0.9, 0.99), max_norm=1.0)
    opt_c = FusedClipAdam(counted, lr=3e-3, betas=(0.9, 0.99), max_norm=1.0, capturable=True)
    for step in range(5):
        grads = [torch.randn(s, device=gpu_device) * (3.0 if step % 2 == 0 else 0.01) for s in shapes]
        for p, q, g in zip(host, counted, grads):
            p.grad, q.grad = g.clone(), g.clone()
        opt_h.step()
        opt_c.step()
        torch.cuda.synchronize()
        for p, q in zip(host, counted):
            torch.testing.assert_close(q.detach(), p.detach(), rtol=1e-6, atol=1e-8)
    assert int(opt_c.step_counter) == 5


def test_training_driver_replays_its_step_from_a_graph(gpu_device):
    """The driver's graph mode (three eager steps, then one recorded step replayed) follows the eager run with the
    same seed step for step: zero-padded action channels (the compaction and its device-side check are inside the
    recording), fused loss head, backward, device-counted clip + Adam."""
    import train_general_ring_no_gain as drv
    print("[case] training driver under a HIP graph N=256 B=32 T=30 k=16", flush=True)
    kw = dict(action_dim=16, num_neurons=256, training_steps=14, batch_size=32, seq_len=30, lr=3e-3, activation="gelu",
              log_every=0, seed=2, fused_loss=True, fused_optimizer=True)
    _, eager = drv.run_training(**kw)
    _, replayed = drv.run_training(hip_graph=True, **kw)
    assert len(replayed) == 14 and all(np.isfinite(replayed))
    np.testing.assert_allclose(replayed, eager, rtol=1e-5, atol=1e-7)
    assert np.mean(replayed[-4:]) < np.mean(replayed[:4])
    with pytest.raises(ValueError):
        drv.run_training(hip_graph=True, **dict(kw, fused_loss=False))


def test_two_streams_interleaved_give_the_sequential_results(gpu_device):
    """The library keeps no hidden device state between calls: two callers that drive the operator from two streams at
    the same time, their launches interleaved by one host thread and their kernels free to overlap on the device,
    each get the bits a lone run gives (different kernel families on the two streams)."""
    from rnn_train_ring_attractor_amd import ring_rnn_cuda_func
    print("[case] two streams: N=256 B=1024 T=40 gelu beside N=200 B=640 T=30 tanh", flush=True)
    jobs = [(make_problem(71, 1024, 40, 2, 256), "gelu"), (make_problem(72, 640, 30, 2, 200), "tanh")]

    def dev(x):
        return torch.tensor(x, device=gpu_device)

    def run(p, act):
        Wa, Wo = dev(p["Wa"]).requires_grad_(True), dev(p["Wo"]).requires_grad_(True)
        r0 = dev(p["r0"]).requires_grad_(True)
        hist = ring_rnn_cuda_func(dev(p["A"]), Wa, -0.05, 0.4, Wo, r0, 0.15, act)
        hist.backward(dev(p["G"]))
        return [hist.detach(), Wa.grad, Wo.grad, r0.grad]

    alone = [run(p, act) for p, act in jobs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    together = [[], []]
    for rep in range(3):
        for i, (p, act) in enumerate(jobs):
            with torch.cuda.stream(streams[i]):
                together[i].append(run(p, act))
    torch.cuda.synchronize()
    for i in range(2):
        for got in together[i]:
            for x, y in zip(got, alone[i]):
                assert torch.equal(x, y)


def test_explicit_stream_keyword_with_allocator_churn_on_the_current_stream(gpu_device):
    """`stream=` of fwd_cuda.fwd / bwd_cuda.bwd: the work goes to a stream that is NOT torch's current one.  The
    scratch the calls take from torch's caching allocator is freed when they return, long before their kernels have
    run; it must not be handed to allocations on the current stream meanwhile.  The side stream is kept busy so that
    the operator's kernels are still queued while the current stream allocates, fills and frees blocks of exactly the
    scratch sizes; results must equal those of the same calls on the current stream, bit for bit."""
    from rnn_train_ring_attractor_amd import _lib
    from rnn_train_ring_attractor_amd.rnn_cuda import fwd_cuda, bwd_cuda, saved_nbytes
    B, T, k, N = 512, 24, 2, 256
    print(f"[case] explicit stream= B={B} T={T} k={k} N={N} gelu", flush=True)
    p = make_problem(81, B, T, k, N)

    def dev(x):
        return torch.tensor(x, device=gpu_device)

    A, Wa, Wo, r0, G = dev(p["A"]), dev(p["Wa"]), dev(p["Wo"]), dev(p["r0"]), dev(p["G"])
    lib = _lib.load()
    sizes = [int(lib.ringattr_fwd_workspace_bytes(N, k, T, B)), int(lib.ringattr_bwd_workspace_bytes(N, k, T, B, 1))]

    def run(stream, churn):
        hist = torch.empty(T, B, N, device=gpu_device)
        saved = torch.empty(saved_nbytes(N, k, T, B), dtype=torch.uint8, device=gpu_device)
        gWa, gWo = torch.empty_like(Wa), torch.empty_like(Wo)
        fwd_cuda.fwd(A=A, Wa=Wa, J0=-0.05, J1=0.4, Wo=Wo, r_init=r0, bump_history=hist, alpha=0.15,
                     activation_type=1, saved=saved, stream=stream)
        if churn:
            churn()
        bwd_cuda.bwd(grad_output=G, A=A, Wa=Wa, J0=-0.05, J1=0.4, Wo=Wo, bump_history=hist, r_init=r0, grad_Wa=gWa,
                     grad_Wo=gWo, alpha=0.15, activation_type=1, saved=saved, accumulate=False, stream=stream)
        if churn:
            churn()
        return hist, gWa, gWo

    want = run(None, None)
    torch.cuda.synchronize()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    busy = torch.randn(4096, 4096, device=gpu_device)

    def churn():
        # blocks of the scratch sizes, written on the current stream while the side stream still works
        for _ in range(4):
            for nbytes in sizes:
                torch.empty(nbytes, dtype=torch.uint8, device=gpu_device).fill_(0xFF)

    with torch.cuda.stream(side):
        for _ in range(20):
            busy = busy @ busy * 1e-4          # ~tens of milliseconds queued in front of the operator
    got = run(side, churn)
    queued = not side.query()
    torch.cuda.synchronize()
    print(f"[measured] side stream still busy when the calls returned: {queued}", flush=True)
    for x, y in zip(got, want):
        assert torch.equal(x, y)
    # the raw stream handle is accepted as well
    got = run(side.cuda_stream, churn)
    torch.cuda.synchronize()
    for x, y in zip(got, want):
        assert torch.equal(x, y)
