"""Headline benchmark: fused forward + BPTT of the ring-attractor time loop on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

Defaults: K = 1000 timed steps after W = 200 warm-up steps (about one second of GPU time): the chip's clocks
take some tens of milliseconds of sustained load to settle, and a step is well under a millisecond.

One "step" = one forward + one backward of the operator over one synthetic batch at
N=256, B=4096, T=120, k=2, gelu (inputs resident in HBM before the timed region).
Prints ONE JSON line: sample-steps/s (B*T per fwd+bwd), the roofline of the slowest kernel from
HIP events recorded on the launch stream inside the timed region, and a host-CPU baseline (torch
port of the reference's per-sample-W_eff formulation) on a bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA, TFLOP/s
PEAK_HBM_GBS = 8000.0          # MI355X HBM3E, GB/s

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (KiB per dispatch, each scaled by what the
# same counter reads for a 1 GiB device copy: x2.000 for FETCH_SIZE, x1.000 for WRITE_SIZE); the summary is
# profiles/train_n256_b4096_t120_gelu_counters.md.  Counter runs cannot share a process with the timed region, so
# the figures are carried here and refreshed whenever a kernel's memory behaviour changes.
MEASURED_TRAFFIC_BYTES = {
    "train_n256_b4096_t120_gelu": {"fwd": (6002 * 2.0 + 983679) * 1024, "bptt": (376734 * 2.0 + 245760) * 1024,
                                   "dw": (256553 * 2.0 + 49152) * 1024},
}

WORKLOADS = {
    # the headline training shape (the default and the only workload the metric is quoted on)
    "train_n256_b4096_t120_gelu": dict(N=256, B=4096, T=120, k=2, act="gelu", J0=-1.0 / 256, J1=1.0, mode="train"),
    # the other benchmark shapes, for reference figures (run with --workload; pick --steps to taste)
    "train_n120_b64_t120_tanh": dict(N=120, B=64, T=120, k=2, act="tanh", J0=-1.0 / 120, J1=1.0, mode="train"),
    "infer_n256_b1024_t120_relu": dict(N=256, B=1024, T=120, k=2, act="relu", J0=-1.0 / 256, J1=1.0, mode="infer"),
    "train_n512_b8192_t512_tanh": dict(N=512, B=8192, T=512, k=2, act="tanh", J0=-1.0 / 512, J1=1.0, mode="train"),
    # the reference training script's own defaults: 16 action channels of which two are driven (zero padding)
    "train_n256_b128_t100_k16pad_gelu": dict(N=256, B=128, T=100, k=16, act="gelu", J0=-0.1, J1=0.1, mode="train"),
}


def make_inputs(cfg, device):
    """Seeded synthetic inputs of the named shape, drawn on the host with the package's own data helpers:
    weights ~ N(0, 1/N); angular-velocity trials (10 % leading zeros, U(-0.1*pi, 0.1*pi), zero ratio in
    {0.2, 0.5, 0.8}); L/R gates = relu(-/+av); Gaussian bump at each trial's initial angle."""
    import math
    import torch
    from rnn_train_ring_attractor_amd import host
    torch.manual_seed(42)
    N, B, T, k = cfg["N"], cfg["B"], cfg["T"], cfg["k"]
    Wo = torch.randn(N, N) / math.sqrt(N)
    Wa = torch.randn(k, N, N) / math.sqrt(N)
    av, angle = host.generate_av_integration_data_ultra_fast(B, T)
    A = host.av_to_action_signal(av) if k == 2 else host.av_to_action_signal_ND(av, k)
    r0 = host.create_initial_bump(angle[:, 0], N)
    to = lambda x: x.float().contiguous().to(device)
    return dict(A=to(A), Wa=to(Wa), Wo=to(Wo), r0=to(r0), angle=to(angle))


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


def cpu_baseline(cfg, sample_B, iters=8):
    """Torch port of the reference formulation (W_eff per sample + bmm + autograd), fp32, host cores."""
    import torch
    from oracle import torch_port as TP
    from tests.ring_cases import make_problem
    threads = int(os.environ.get("OMP_NUM_THREADS", "0")) or min(16, os.cpu_count() or 1)
    torch.set_num_threads(threads)
    p = make_problem(42, sample_B, cfg["T"], cfg["k"], cfg["N"])
    t = lambda x: torch.tensor(x)
    args = (t(p["A"]), t(p["Wa"]), cfg["J0"], cfg["J1"], t(p["Wo"]), t(p["r0"]), 0.15, cfg["act"])
    G = t(p["G"])
    TP.fwd_bwd_autograd(*args, grad_output=G)          # warm-up
    ts = []
    for _ in range(iters):
        t0 = time.perf_counter()
        TP.fwd_bwd_autograd(*args, grad_output=G)
        ts.append(time.perf_counter() - t0)
    mean = sum(ts) / len(ts)
    return {"value": sample_B * cfg["T"] / mean, "unit": "sample-steps/s", "cores": threads, "kind": "port",
            "sample": f"N={cfg['N']} B={sample_B} T={cfg['T']} {cfg['act']} fp32, {iters} fwd+bwd iters, "
                      f"{mean * 1e3:.0f} ms each (full B={cfg['B']} would need B*N^2*4*T bytes of saved W_eff)"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=1000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--workload", default="train_n256_b4096_t120_gelu", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
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
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible; the HIP path has no CPU fallback")
    dev = torch.device("cuda:0")
    cfg = WORKLOADS[args.workload]
    N, B, T, k = cfg["N"], cfg["B"], cfg["T"], cfg["k"]
    x = make_inputs(cfg, dev)
    Wa = x["Wa"].requires_grad_(True)
    Wo = x["Wo"].requires_grad_(True)

    def fwd():
        return ring_rnn_cuda_func(x["A"], Wa, cfg["J0"], cfg["J1"], Wo, x["r0"], 0.15, cfg["act"])

    train = cfg["mode"] == "train"
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

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    _lib.profile_enable(True)
    _lib.profile_read()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    prof = _lib.profile_read()
    _lib.profile_enable(False)
    if args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()

    ms_per_step = dt / args.steps * 1e3
    value = B * T / (dt / args.steps)
    flops_third = 6.0 * N * N * B * T                      # per kernel: fwd, bptt and dW each contract 2*3*N^2 per sample-step
    kern = {kname: (ms / max(cnt, 1)) for kname, (ms, cnt) in prof.items() if cnt}
    dominant = max(("fwd", "bptt", "dw") if train else ("fwd",), key=lambda n_: kern.get(n_, 0.0))
    dom_ms = kern[dominant]
    achieved = flops_third / (dom_ms * 1e-3) / 1e12
    bytes_per_ss = 12 * N + 8 * k                           # fp32 history write + r_prev/grad_output reads + A
    out = {
        "metric": ("fwd+bwd sample-steps/s (B*T/s) at N=256,B=4096,T=120; % bf16 MFMA peak"
                   if args.workload == "train_n256_b4096_t120_gelu" else
                   f"{'fwd+bwd' if train else 'fwd'} sample-steps/s (B*T/s) at N={N},B={B},T={T}"),
        "value": value, "unit": "sample-steps/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "N": N, "B": B, "T": T, "a_dim": k, "activation": cfg["act"],
                   "mode": "forward + backward" if train else "forward only (no saved activations)",
                   "grad_output": "gradient of the cos-sim + 0.2*bump-amplitude loss pair, precomputed" if train else None},
        "pct_bf16_mfma_peak": 100.0 * ((18.0 if train else 6.0) * N * N * value) / (PEAK_BF16_TFLOPS * 1e12),
        "algorithmic_hbm_gbs": (bytes_per_ss if train else 4 * N + 4 * k) * value / 1e9,
        "roofline": {"bound": "mfma", "kernel": dominant, "achieved": achieved, "peak": PEAK_BF16_TFLOPS,
                     "unit": "TFLOP/s", "frac": achieved / PEAK_BF16_TFLOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES.get(args.workload, {}).get(dominant),
                     "flops_per_launch": flops_third, "avg_launch_ms": dom_ms,
                     "algorithmic_bytes_per_launch": {"fwd": (4 * N + 4 * k) * B * T, "bptt": (4 * N + 4 * k) * B * T,
                                                      "dw": (4 * N + 4 * k) * B * T}[dominant]},
        "kernel_ms": kern,
    }
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(cfg, min(args.cpu_sample_batch, B))
    print(json.dumps(out))


if __name__ == "__main__":
    main()
