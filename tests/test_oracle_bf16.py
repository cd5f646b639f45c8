"""Pins the rounding-aware oracle: rounding helpers against library conversions, and the model itself
against the fp64 oracle with rounding switched off."""
import numpy as np
import pytest
import torch

from oracle import ring_oracle as O
from oracle import ring_oracle_bf16 as OB
from tests.ring_cases import make_problem


def test_round_bf16_matches_torch_bfloat16():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(5000) * 10.0 ** rng.integers(-8, 8, 5000),
                        [0.0, -0.0, 1.0, 1.00390625, 1.001953125, 3.0e38, 1e-40]]).astype(np.float32)
    ref = torch.tensor(x).bfloat16().float().numpy()
    np.testing.assert_array_equal(OB.round_bf16(x).astype(np.float32), ref)
    # ties go to even: 1 + 2^-8 is exactly between 1 and 1 + 2^-7
    assert OB.round_bf16(np.float32(1.00390625)) == 1.0
    assert OB.round_bf16(np.float32(1.01171875)) == 1.015625


def test_round_fp16_matches_torch_half():
    x = (np.random.default_rng(1).standard_normal(4000) * 2).astype(np.float32)
    np.testing.assert_array_equal(OB.round_fp16(x).astype(np.float32), torch.tensor(x).half().float().numpy())


@pytest.mark.parametrize("act", ["relu", "gelu", "tanh", "silu"])
def test_without_rounding_it_is_the_fp64_oracle(act):
    p = make_problem(3, 6, 9, 3, 20, action="dense")
    got = OB.forward_backward(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, act, p["G"], rounding=False)
    hist, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, act)
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.1, p["Wo"], hist, p["r0"], 0.15, act)
    np.testing.assert_allclose(got["bump_history"], hist, rtol=0, atol=1e-13)
    for key in ("grad_Wo", "grad_Wa", "grad_r_init", "grad_A"):
        np.testing.assert_allclose(got[key], ref[key], rtol=0, atol=1e-11, err_msg=key)


def test_rounding_moves_smooth_activations_by_less_than_the_parity_tolerances():
    p = make_problem(4, 32, 40, 2, 64)
    got = OB.forward_backward(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, "gelu", p["G"])
    hist, _ = O.forward_dense(p["A"], p["Wa"], -0.1, 0.1, p["Wo"], p["r0"], 0.15, "gelu")
    ref = O.backward_dense(p["G"], p["A"], p["Wa"], -0.1, 0.1, p["Wo"], hist, p["r0"], 0.15, "gelu")
    assert 0 < O.max_rel_err(got["bump_history"], hist) < 1e-2
    assert O.cosine(got["grad_Wo"], ref["grad_Wo"]) > 0.999
    assert 0 < O.max_rel_err(got["grad_Wo"], ref["grad_Wo"]) < 2e-2
