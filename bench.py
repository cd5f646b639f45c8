"""Headline benchmark: fused forward + BPTT of the ring-attractor time loop on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-cpu] [--prewarm-ms MS] [--recompute]

One "step" = one forward + one backward of the operator over one synthetic batch at
N=256, B=4096, T=120, k=2, gelu (inputs resident in HBM before the timed region).

Phases: an untimed PRE-WARM that always runs (steps of the same workload for at least --prewarm-ms of wall time: the
chip's clocks take tens of milliseconds of sustained load to settle and a step is well under a millisecond; its
length is reported under "prewarm"), then exactly --warmup untimed steps, then exactly --steps timed steps between
two torch.cuda.synchronize().

Prints ONE JSON line: sample-steps/s (B*T per fwd+bwd), the roofline of the slowest kernel from HIP events recorded
on the launch stream inside the timed region (around every --event-stride-th launch of each kernel: the two event
records around a launch cost the stream 4-5 us, 23 us per step when every launch is bracketed), and host-CPU baselines (torch port of the reference's per-sample-W_eff
formulation): the reference's own CPU configuration (N=120, B=64, T=120, tanh, fp32) exactly, and the benchmarked
workload at a reduced batch.
"""
import argparse
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA, TFLOP/s
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E, GB/s

HEADLINE = "train_n256_b4096_t120_gelu"
WORKLOADS = {
    # the headline training shape (the default and the only workload the metric is quoted on)
    HEADLINE: dict(N=256, B=4096, T=120, k=2, act="gelu", J0=-1.0 / 256, J1=1.0, mode="train"),
    # the other benchmark shapes, for reference figures (run with --workload; pick --steps to taste)
    "train_n120_b64_t120_tanh": dict(N=120, B=64, T=120, k=2, act="tanh", J0=-1.0 / 120, J1=1.0, mode="train"),
    "infer_n256_b1024_t120_relu": dict(N=256, B=1024, T=120, k=2, act="relu", J0=-1.0 / 256, J1=1.0, mode="infer"),
    "train_n512_b8192_t512_tanh": dict(N=512, B=8192, T=512, k=2, act="tanh", J0=-1.0 / 512, J1=1.0, mode="train"),
    # a wide ring (the reference's kernels take rings up to 2048 neurons), trained at a large batch
    "train_n1024_b2048_t120_tanh": dict(N=1024, B=2048, T=120, k=2, act="tanh", J0=-1.0 / 1024, J1=1.0, mode="train"),
    # the general ring with gain networks: two 1 -> 16 -> 1 MLPs turn the angular velocity into the (L, R) gates and
    # train through dL/d action_signal (model step: MLPs + time loop forward and backward, MLP gradients included)
    "gain_n256_b4096_t240_relu": dict(N=256, B=4096, T=240, k=2, act="relu", J0=-1.0 / 256, J1=1.0, mode="gain"),
    # the reference training script's own defaults: 16 action channels of which two are driven (zero padding)
    "train_n256_b128_t100_k16pad_gelu": dict(N=256, B=128, T=100, k=16, act="gelu", J0=-0.1, J1=0.1, mode="train",
                                             driven=(0, 1)),
}
# the shapes of the reference's published latency table (assets/REPORT.md:5-10): forward, B=256, T=20, 16 dense channels,
# plus its rows with more channels (:11-12) and the widths it could only run on its fp32 kernel (:13-16, k % 16 != 0)
for _n, _k in [(n, 16) for n in (128, 256, 384, 512, 1024, 2048)] + [(2048, 32), (2048, 64)] + \
        [(1024, k) for k in (2, 3, 6, 12)]:
    WORKLOADS[f"report_fwd_n{_n}_b256_t20_k{_k}"] = dict(N=_n, B=256, T=20, k=_k, act="silu", J0=-0.1, J1=0.1,
                                                        mode="infer", action="dense")


def make_inputs(cfg, device):
    """Seeded synthetic inputs of the named shape, generated on the device (nothing is staged from the host):
    weights ~ N(0, 1/N) from torch's device generator; angular-velocity trials (10 % leading zeros,
    U(-0.1*pi, 0.1*pi), zero ratio in {0.2, 0.5, 0.8}), L/R gates = relu(-/+av) and a von Mises (kappa = 4) bump at
    each trial's initial angle from the library's input generator (ringattr_generate_inputs)."""
    import torch
    from rnn_train_ring_attractor_amd import generate_inputs
    N, B, T, k = cfg["N"], cfg["B"], cfg["T"], cfg["k"]
    gen = torch.Generator(device=device).manual_seed(42)
    Wo = torch.randn(N, N, device=device, generator=gen) / N ** 0.5
    Wa = torch.randn(k, N, N, device=device, generator=gen) / N ** 0.5
    av, angle, A, r0 = generate_inputs(42, B, T, N, k, bump="vm", device=device)
    if cfg.get("action") == "dense":
        A = torch.rand(B, T, k, device=device, generator=gen) * (0.3 / k)
    return dict(A=A, Wa=Wa, Wo=Wo, r0=r0, angle=angle, av=av)


def loss_head_grad(hist, angle):
    """d(loss)/d(bump_history) of the training script's loss pair (cosine-similarity loss of the max-normalised
    cosine read-out + 0.2 * bump-amplitude loss; train_general_ring_no_gain.py:324-330 of the reference), computed
    once with torch ops on the GPU, outside the timed region."""
    import math
    import torch
    from rnn_train_ring_attractor_amd import host
    N = hist.shape[-1]
    idx = torch.arange(N, dtype=torch.float32, device=hist.device)
    w_delta7 = torch.cos(2 * math.pi * (idx[:, None] - idx[None, :]) / N)
    h = hist.detach().clone().requires_grad_(True)
    bump = h.permute(1, 0, 2)
    proj = bump @ w_delta7
    out = proj / proj.max(dim=2, keepdim=True)[0]
    (host.cosine_similarity_loss(out, angle) + 0.2 * host.bump_amplitude_loss(bump)).backward()
    return h.grad.contiguous()


def host_cpu():
    """(threads to use, CPU model string, logical CPUs visible).  Threads = OMP_NUM_THREADS when the environment
    sets it (the GPU boxes export this job's CPU share there), otherwise every CPU this process may run on."""
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    try:
        visible = len(os.sched_getaffinity(0))
    except AttributeError:
        visible = os.cpu_count() or 1
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or visible
    return threads, model, visible


def cpu_baseline(N, B, T, k, act, J0, J1, budget_s, note):
    """Torch port of the reference formulation (W_eff per sample + bmm + autograd), fp32, host cores: one warm-up,
    then fwd+bwd iterations until `budget_s` seconds of work (at least 3)."""
    import torch
    from oracle import torch_port as TP
    from tests.ring_cases import make_problem
    threads, model, visible = host_cpu()
    torch.set_num_threads(threads)
    p = make_problem(42, B, T, k, N, bump="vm")
    t = lambda x: torch.tensor(x)
    args = (t(p["A"]), t(p["Wa"]), J0, J1, t(p["Wo"]), t(p["r0"]), 0.15, act)
    G = t(p["G"])
    TP.fwd_bwd_autograd(*args, grad_output=G)          # warm-up
    ts = []
    while len(ts) < 3 or (sum(ts) < budget_s and len(ts) < 200):
        t0 = time.perf_counter()
        TP.fwd_bwd_autograd(*args, grad_output=G)
        ts.append(time.perf_counter() - t0)
    mean = sum(ts) / len(ts)
    return {"value": B * T / mean, "unit": "sample-steps/s", "cores": threads, "cpu_model": model,
            "logical_cpus_visible": visible, "kind": "port",
            "sample": f"N={N} B={B} T={T} {act} fp32, {len(ts)} fwd+bwd iters, {mean * 1e3:.1f} ms each; {note}"}


def measured_traffic(workload, launched):
    """HBM bytes per launch of each kernel, from the committed rocprofv3 counter summary of this workload
    (profiles/<workload>_counters.md carries a line 'TRAFFIC_BYTES_PER_LAUNCH fwd=.. bptt=.. dw=..': FETCH_SIZE and
    WRITE_SIZE per dispatch, each scaled by what the same counter reads for a 1 GiB device copy).  Counter runs cannot
    share a process with the timed region, so the figure is read from there.  The summary also names the kernels it
    was taken from ('TRAFFIC_KERNELS fwd=<kernel>;bptt=<kernel>;...'); `launched` maps the same keys to the kernels
    this run launched (ringattr_last_kernel_name), and a key whose names differ is dropped: a summary that predates a
    kernel change must not pass for a measurement of the new kernel.  Returns (traffic or None, list of notes)."""
    path = os.path.join(ROOT, "profiles", f"{workload}_counters.md")
    try:
        text = open(path).read()
    except OSError:
        return None, ["no counter summary for this workload"]
    m = re.search(r"^TRAFFIC_BYTES_PER_LAUNCH\s+(.*)$", text, re.M)
    if not m:
        return None, ["counter summary has no TRAFFIC_BYTES_PER_LAUNCH line"]
    traffic = {kv.split("=")[0]: float(kv.split("=")[1]) for kv in m.group(1).split()}
    mk = re.search(r"^TRAFFIC_KERNELS\s+(.*)$", text, re.M)
    if not mk:
        return None, ["counter summary names no kernels (TRAFFIC_KERNELS): not used"]
    named = dict(kv.split("=", 1) for kv in mk.group(1).strip().split(";") if "=" in kv)
    notes = []
    for key in list(traffic):
        if key in launched and named.get(key) != launched[key]:
            notes.append(f"{key}: summary is of '{named.get(key)}', this run launched '{launched[key]}': dropped")
            del traffic[key]
    return (traffic or None), notes


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default=HEADLINE, choices=sorted(WORKLOADS))
    ap.add_argument("--prewarm-ms", type=float, default=500.0,
                    help="untimed steps of the workload run for at least this long before --warmup (clock settling)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline legs")
    ap.add_argument("--recompute", action="store_true",
                    help="training workloads: the forward keeps no saved record and the backward recomputes the "
                         "derivative record and operand copy from bump_history first (activation recompute)")
    ap.add_argument("--precise-wo", action="store_true",
                    help="Wo enters the contraction as two bf16 operands (hi + lo), one more matrix per step: the "
                         "accuracy option for long, marginally stable sequences (never the metric's configuration)")
    ap.add_argument("--cluster-bptt", action="store_true",
                    help="N = 512 workloads: run the BPTT on the compute-unit clusters as well (sets "
                         "RINGATTR_CLUSTER_BPTT=1; off by default because it is not faster; never the metric's "
                         "configuration)")
    ap.add_argument("--event-stride", type=int, default=0,
                    help="bracket every n-th launch of each kernel with HIP events inside the timed region "
                         "(0: steps // 4 clamped to 1..8)")
    ap.add_argument("--no-training-step", action="store_true",
                    help="skip the whole-training-step figure that training workloads report beside the metric")
    ap.add_argument("--cpu-sample-batch", type=int, default=128)
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run three 1 GiB device-to-device copies (known HBM traffic) for scaling rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on exactly one GPU (samples are independent, so the batch shards trivially "
                 "over more); use --gpus 1")

    import torch
    from rnn_train_ring_attractor_amd import _lib, ring_rnn_cuda_func
    from rnn_train_ring_attractor_amd import ring_rnn_cuda as _op
    _op.RECOMPUTE_IN_BACKWARD = bool(args.recompute)
    if args.cluster_bptt:
        os.environ["RINGATTR_CLUSTER_BPTT"] = "1"
    _op.PRECISE_WO = bool(args.precise_wo)
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    dev = torch.device("cuda:0")
    cfg = WORKLOADS[args.workload]
    N, B, T, k = cfg["N"], cfg["B"], cfg["T"], cfg["k"]
    x = make_inputs(cfg, dev)
    mode = cfg["mode"]
    train = mode in ("train", "gain")

    if mode == "gain":
        from rnn_train_ring_attractor_amd import host
        torch.manual_seed(7)
        model = host.LeakyRingAttractor(N, activation=cfg["act"], initialization="random").to(dev)
        model.J0, model.J1 = cfg["J0"], cfg["J1"]
        params = [p for p in model.parameters() if p.requires_grad]

        def fwd():
            return model.forward_history(x["av"], x["r0"])

        G = loss_head_grad(fwd(), x["angle"])

        def step():
            for p in params:
                p.grad = None
            fwd().backward(G)
    else:
        Wa, Wo = x["Wa"], x["Wo"]
        if train:
            Wa.requires_grad_(True)
            Wo.requires_grad_(True)

        def fwd():
            return ring_rnn_cuda_func(x["A"], Wa, cfg["J0"], cfg["J1"], Wo, x["r0"], 0.15, cfg["act"],
                                      driven_channels=cfg.get("driven"))

        if train:
            G = loss_head_grad(fwd(), x["angle"])

            def step():
                Wa.grad = None
                Wo.grad = None
                fwd().backward(G)
        else:
            def step():
                with torch.no_grad():
                    fwd()

    # untimed pre-warm: sustained load until the clocks have settled
    t0 = time.perf_counter()
    prewarm_steps = 0
    while (time.perf_counter() - t0) * 1e3 < args.prewarm_ms:
        for _ in range(10):
            step()
        prewarm_steps += 10
        torch.cuda.synchronize()
    prewarm_ms = (time.perf_counter() - t0) * 1e3

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    stride = args.event_stride if args.event_stride > 0 else max(1, min(8, args.steps // 4))
    _lib.profile_enable(stride)
    _lib.profile_read()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    prof = _lib.profile_read()
    _lib.profile_enable(False)
    launched = _lib.last_kernel_names()      # the kernels of the timed region (the training-step leg below launches others)
    training_step = None
    if mode == "train" and k == 2 and N <= 512 and not args.no_training_step:
        # Beside the metric (not part of it): a whole training step around the same time loop -- a fresh batch from the
        # device generator, forward + loss head as one operator, its backward, gradient clipping + Adam.
        from rnn_train_ring_attractor_amd import FusedClipAdam, generate_inputs, ring_rnn_loss_func
        opt = FusedClipAdam([Wa, Wo], lr=1e-4, max_norm=1.0)

        def train_once(i):
            _, angle_i, action_i, r0_i = generate_inputs(1000 + i, B, T, N, k, bump="vm")
            total = ring_rnn_loss_func(action_i, Wa, cfg["J0"], cfg["J1"], Wo, r0_i, 0.15, cfg["act"], angle_i, 0.2)[0]
            Wa.grad = None
            Wo.grad = None
            total.backward()
            opt.step()
            return total

        n_tr = max(20, min(200, args.steps))
        for i in range(10):
            train_once(i)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for i in range(n_tr):
            last = train_once(10 + i)
        torch.cuda.synchronize()
        training_step = {"ms": (time.perf_counter() - t1) / n_tr * 1e3, "steps": n_tr, "final_loss": float(last),
                         "what": "device input generator + forward and loss head as one operator + backward + fused "
                                 "gradient clipping and Adam; reported beside the metric, not part of it"}
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    ms_per_step = dt / args.steps * 1e3
    value = B * T / (dt / args.steps)
    mats = 1 + k
    flops_third = 2.0 * mats * N * N * B * T               # per kernel: fwd, bptt and dW each contract 2*(1+k)*N^2 per sample-step
    kern = {kname: (ms / max(cnt, 1)) for kname, (ms, cnt) in prof.items() if cnt}
    dominant = max(("fwd", "bptt", "dw") if train else ("fwd",), key=lambda n_: kern.get(n_, 0.0))
    dom_ms = kern[dominant]
    achieved = flops_third / (dom_ms * 1e-3) / 1e12
    bytes_per_ss = 12 * N + 8 * k                           # fp32 history write + r_prev/grad_output reads + A
    traffic, traffic_notes = measured_traffic(args.workload + ("_recompute" if args.recompute else ""),
                                              launched)
    out = {
        "metric": ("fwd+bwd sample-steps/s (B*T/s) at N=256,B=4096,T=120; % bf16 MFMA peak"
                   if args.workload == HEADLINE else
                   f"{'fwd+bwd' if train else 'fwd'} sample-steps/s (B*T/s) at N={N},B={B},T={T}"),
        "value": value, "unit": "sample-steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload + ("_recompute" if args.recompute else "") + ("_precise_wo" if args.precise_wo else "") + ("_cluster_bptt" if args.cluster_bptt else ""), "N": N, "B": B, "T": T, "a_dim": k, "activation": cfg["act"],
                   "mode": {"train": "forward + backward", "infer": "forward only (no saved activations)",
                            "gain": "gain MLPs + forward + backward (MLP gradients through dL/d action_signal)"}[mode],
                   "grad_output": "gradient of the cos-sim + 0.2*bump-amplitude loss pair, precomputed" if train else None},
        "prewarm": {"steps": prewarm_steps, "ms": prewarm_ms, "note": "untimed, before --warmup; clock settling"},
        "pct_bf16_mfma_peak": 100.0 * ((3 if train else 1) * 2.0 * mats * N * N * value) / (PEAK_BF16_TFLOPS * 1e12),
        "algorithmic_hbm_gbs": (bytes_per_ss if train else 4 * N + 4 * k) * value / 1e9,
        "roofline": {"bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": (traffic or {}).get(dominant),
                     "flops_per_launch": flops_third, "avg_launch_ms": dom_ms, "event_stride": stride,
                     "algorithmic_bytes_per_launch": (4 * N + 4 * k) * B * T},
        "kernel_ms": kern,
    }
    if training_step:
        out["training_step"] = training_step
    if traffic_notes:
        out["traffic_notes"] = traffic_notes
    if traffic:
        out["traffic_bytes_per_launch"] = traffic
        complete = all(k_ in traffic for k_ in (("fwd", "bptt", "dw") if train else ("fwd",)))
        out["traffic_over_algorithmic"] = sum(traffic.values()) / (bytes_per_ss * B * T) if train and complete else None
    if not args.no_cpu:
        # the reference's CPU configuration exactly (what cpu_baseline means), then this workload at a reduced batch
        out["cpu_baseline"] = cpu_baseline(120, 64, 120, 2, "tanh", -1.0 / 120, 1.0, 8.0,
                                           "the reference's CPU configuration (LeakyRingAttractor no-gain) at its full size")
        sb = min(args.cpu_sample_batch, B)
        out["cpu_baseline_workload"] = cpu_baseline(
            N, sb, T, k, cfg["act"], cfg["J0"], cfg["J1"], 10.0,
            f"this workload at batch {sb} of {B} (the full batch would need B*N^2*4*T bytes of saved W_eff)")
    print(json.dumps(out))


if __name__ == "__main__":
    main()
