"""Seeding, tensor comparison and event-timed latency helpers with the call signatures of the reference's
`utils/benchmark.py` (`set_seed` :5-11, `check_tensor_match` :21-56, `measure_latency_cuda` :58-79), so scripts
written against it run on this library.  torch's `cuda` namespace is HIP on ROCm: the events below are HIP events on
the current stream."""
from __future__ import annotations

import random

import numpy as np
import torch


def set_seed(seed=42):
    random.seed(seed)
    np.random.seed(seed)
    torch.manual_seed(seed)
    if torch.cuda.is_available():
        torch.cuda.manual_seed_all(seed)


def check_tensor_match(tsr_impl, tsr_ref, name, rtol=1e-5, atol=1e-8, max_print=1):
    """True when `tsr_impl` is allclose to `tsr_ref`; otherwise prints where and by how much they differ (first and
    last `max_print` mismatching indices, counts, mean and spread of the absolute and relative difference)."""
    if torch.allclose(tsr_impl, tsr_ref, rtol=rtol, atol=atol):
        print(f"{name} match!")
        return True
    diff = (tsr_impl - tsr_ref).abs()
    rdiff = diff / (tsr_ref.abs() + atol)
    bad = torch.nonzero(~torch.isclose(tsr_impl, tsr_ref, rtol=rtol, atol=atol))
    print(f"\n{name} differences: a_tol = {atol}, r_tol = {rtol}")
    print("index                       ref         impl        diff        rdiff")

    def show(rows):
        for idx in rows.tolist():
            i = tuple(idx)
            print(f"[{','.join(map(str, idx))}]: {float(tsr_ref[i]):10.6f} {float(tsr_impl[i]):10.6f} "
                  f"{float(diff[i]):10.6f} {float(rdiff[i]):10.6f}")

    show(bad[:max_print])
    if len(bad) > max_print:
        print("...")
        show(bad[-max_print:])
    print(f"Total mismatched elements: {len(bad)} out of {tsr_impl.numel()} ({100.0 * len(bad) / tsr_impl.numel():.1f}%)")
    print(f"diff: {float(diff.mean()):.6f} ± {float(diff.std()):.6f}")
    print(f"rdiff: {float(rdiff.mean()):.6f} ± {float(rdiff.std()):.6f}")
    return False


def measure_latency_cuda(fn, *args, n_warmup=2, n_iters=20, **kwargs):
    """'mean ± std ms' of `fn(*args, **kwargs)` over `n_iters` event-bracketed calls after `n_warmup` untimed ones."""
    for _ in range(n_warmup):
        fn(*args, **kwargs)
    torch.cuda.synchronize()
    times = []
    for _ in range(n_iters):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        fn(*args, **kwargs)
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end))
    t = torch.tensor(times)
    return f"{t.mean().item():.3f} ± {t.std(unbiased=False).item():.3f} ms"
