"""The torch host helpers (same module paths the reference script imports) against the numpy oracle."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import ring_oracle as O


def test_module_paths_and_star_import_export_the_reference_names():
    ns = {}
    exec("from cpp.ring_rnn_cuda import *", ns)
    for name in ("torch", "ring_rnn_cuda_func", "RingRnnCudaFunc"):
        assert name in ns
    from cpp.rnn_cuda import fwd_cuda, bwd_cuda
    assert hasattr(fwd_cuda, "fwd") and hasattr(bwd_cuda, "bwd")
    import train.train_ring_attractor as T
    for name in ("non_linear", "create_initial_bump", "cosine_similarity_loss", "bump_amplitude_loss",
                 "decode_angle_from_population_vector", "decode_angle_from_argmax", "plot_ring_matrices"):
        assert callable(getattr(T, name))
    from utils.generate_av_integration_data import AVIntegrationDataset  # noqa: F401
    # the training entry points of the three models, each under the reference's module path and name
    import train.train_general_ring_attractor as TG
    import train.train_general_ring_no_gain as TN
    assert callable(T.run_training_and_evaluation) and callable(TG.run_training_and_evaluation)
    assert callable(TN.run_training_and_evaluation)


def test_helpers_match_oracle():
    from rnn_train_ring_attractor_amd import host as H
    rng = np.random.default_rng(0)
    ang = rng.random(5) * 2 * np.pi
    np.testing.assert_allclose(H.create_initial_bump(torch.tensor(ang), 120).numpy(), O.create_initial_bump(ang, 120), atol=1e-12)
    wave = rng.standard_normal((3, 4, 32))
    tgt = rng.random((3, 4)) * 2 * np.pi
    assert abs(float(H.cosine_similarity_loss(torch.tensor(wave), torch.tensor(tgt))) - O.cosine_similarity_loss(wave, tgt)) < 1e-6
    assert abs(float(H.bump_amplitude_loss(torch.tensor(wave))) - O.bump_amplitude_loss(wave)) < 1e-9
    np.testing.assert_allclose(H.decode_angle_from_population_vector(torch.tensor(wave)).numpy(),
                               O.decode_angle_from_population_vector(wave), atol=1e-6)
    np.testing.assert_allclose(H.decode_angle_from_argmax(torch.tensor(wave)).numpy(), O.decode_angle_from_argmax(wave), atol=1e-6)
    av = rng.standard_normal((3, 7)) * 0.2
    np.testing.assert_allclose(H.av_to_action_signal(torch.tensor(av)).numpy(), O.av_to_action_signal(av))
    np.testing.assert_allclose(H.av_to_action_signal_ND(torch.tensor(av), 16).numpy(), O.av_to_action_signal_nd(av, 16))
    np.testing.assert_allclose(H.av_to_action_signal_ND(torch.tensor(av), 5, zero_padding=False).numpy(),
                               O.av_to_action_signal_nd(av, 5, zero_padding=False), atol=1e-7)
    with pytest.raises(ValueError):
        H.non_linear(torch.zeros(2), "sigmoid")


def test_dataset_structure_and_batch_cursor():
    from rnn_train_ring_attractor_amd.host import AVIntegrationDataset
    torch.manual_seed(1)
    ds = AVIntegrationDataset(num_samples=50, seq_len=40, chunk_size=16)
    assert len(ds) == 50 and ds.av_data.shape == (50, 40)
    av, ang = ds.av_data, ds.angle_data
    assert (av[:, :4] == 0).all() and av.abs().max() <= 0.1 * math.pi
    torch.testing.assert_close(ang[:, 1:], (ang[:, :1] + torch.cumsum(av[:, :-1], 1)) % (2 * math.pi))
    nz = (av[:, 4:] != 0).sum(1)
    assert set(nz.tolist()) <= {36 - int(np.float32(36) * np.float32(z)) for z in (0.2, 0.5, 0.8)}
    seen = torch.cat([ds.generate_batch(20)[0] for _ in range(2)])
    assert seen.shape == (40, 40)
    assert abs(ds.get_memory_usage_mb() - 2 * 50 * 40 * 4 / 2 ** 20) < 1e-9
    b3 = ds.generate_batch(20)[0]              # wraps around the 50 samples
    assert b3.shape == (20, 40)
    with pytest.raises(ValueError):
        ds.generate_batch(51)
    with pytest.raises(IndexError):
        ds[50]


def test_general_ring_gain_networks_follow_the_reference_formula():
    """GeneralizedRingAttractor.gated_action_signal on the CPU: action * gain_c(|action|) per channel
    (train/train_general_ring_attractor.py:99-109 of the reference), and the module path the reference uses."""
    import torch
    from train.train_general_ring_attractor import GeneralizedRingAttractor
    torch.manual_seed(3)
    m = GeneralizedRingAttractor(32, action_dim=3, hidden_gain_neurons=8)
    assert [n for n, _ in m.named_parameters()][:2] == ["Wo", "Wa"] and len(m.gain_nets) == 3
    a = torch.randn(5, 7, 3)
    got = m.gated_action_signal(a)
    for c in range(3):
        net = m.gain_nets[c]
        x = a[:, :, c].abs().reshape(-1, 1)
        h = torch.nn.functional.gelu(x @ net[0].weight.t() + net[0].bias)
        gain = torch.nn.functional.softplus(h @ net[2].weight.t() + net[2].bias).reshape(5, 7)
        assert torch.allclose(got[:, :, c], a[:, :, c] * gain, atol=1e-6)
    with torch.no_grad():
        assert GeneralizedRingAttractor(16, action_dim=2, initialization="perfect").Wa.shape == (2, 16, 16)


def test_comparison_helper_reports_mismatches(capsys):
    """utils.benchmark.check_tensor_match (reference utils/benchmark.py:21-56): allclose verdict plus a report."""
    import torch
    from utils.benchmark import check_tensor_match, set_seed
    set_seed(7)
    a = torch.randn(4, 5)
    assert check_tensor_match(a.clone(), a, "same") is True
    b = a.clone()
    b[1, 2] += 0.5
    b[3, 4] -= 0.25
    assert check_tensor_match(b, a, "two off", rtol=1e-5, atol=1e-8) is False
    out = capsys.readouterr().out
    assert "same match!" in out and "Total mismatched elements: 2 out of 20 (10.0%)" in out and "[1,2]" in out and "[3,4]" in out
    set_seed(7)
    assert torch.equal(torch.randn(4, 5), a)


def test_chunked_generator_concatenates_trials():
    """utils.generate_av_integration_data.generate_av_integration_data_chunked: chunking changes nothing but the
    temporaries -- shapes, the leading zero block and angle = cumulative sum of av hold across chunk borders."""
    import torch
    from utils.generate_av_integration_data import generate_av_integration_data_chunked
    torch.manual_seed(0)
    av, ang = generate_av_integration_data_chunked(25, 40, zero_padding_start_ratio=0.1, zero_ratios_in_rest=[0.5],
                                                   chunk_size=10)
    assert av.shape == (25, 40) and ang.shape == (25, 40)
    assert torch.all(av[:, :4] == 0)
    assert float(av.abs().max()) <= 0.1 * 3.141593
    step = torch.remainder(ang[:, 1:] - ang[:, :-1] - av[:, :-1] + 3.141592653589793, 2 * 3.141592653589793) - 3.141592653589793
    assert float(step.abs().max()) <= 1e-4


def test_bench_drops_counter_summaries_of_other_kernels():
    """bench.py pairs its timings with the HBM traffic of a stored rocprofv3 counter summary; the summary names the
    kernels it was taken from, and a slot whose kernel differs from the one the run launched is dropped with a note."""
    import re
    import bench
    path = os.path.join(os.path.dirname(bench.__file__), "profiles", f"{bench.HEADLINE}_counters.md")
    text = open(path).read()
    named = dict(kv.split("=", 1) for kv in re.search(r"^TRAFFIC_KERNELS\s+(.*)$", text, re.M).group(1).split(";"))
    assert {"fwd", "bptt", "dw"} <= set(named)
    traffic, notes = bench.measured_traffic(bench.HEADLINE, dict(named))
    assert notes == [] and traffic["fwd"] > 5e8 and traffic["bptt"] > 5e8 and traffic["dw"] > 2e8
    other = dict(named, fwd="ring_fwd_res256_kernel<1,true,true,true>")
    traffic, notes = bench.measured_traffic(bench.HEADLINE, other)
    assert "fwd" not in traffic and "bptt" in traffic and len(notes) == 1 and "fwd" in notes[0]
    traffic, notes = bench.measured_traffic("no_such_workload", named)
    assert traffic is None and notes
