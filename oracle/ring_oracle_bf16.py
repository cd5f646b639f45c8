"""Rounding-aware restatement: the dense-form recurrence and BPTT of ring_oracle.py with the HIP
kernels' reduced-precision points made explicit (everything else stays fp64).

TEST INFRASTRUCTURE ONLY.  It answers one question the fp64 oracle cannot: is a deviation from the
fp64 result explained by rounding the MFMA operands to bf16 (expected, bounded by the tolerances),
or by a defect in a kernel?  A kernel is compared against this model at a tolerance ~10x tighter
than against the fp64 oracle.

Rounding points (same math as ring_oracle.forward_dense / backward_dense, which cite the reference):
  * weights [Wo|Wa]            -> bf16   (MFMA B operand)
  * r_prev, g as contraction operands -> bf16 (MFMA A operand); the leak term, the J0 row sums and
    the state carried between steps stay unrounded
  * alpha * F'(re) kept for the backward -> fp16
  * A_c * g in the weight-gradient contraction -> bf16
Pinned by tests/test_oracle_bf16.py: with rounding switched off it reproduces ring_oracle exactly.
"""
from __future__ import annotations

import numpy as np

from . import ring_oracle as O


def round_bf16(x):
    """Round-to-nearest-even to bfloat16, returned as float64."""
    u = np.asarray(x, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.astype(np.uint32).view(np.float32).astype(np.float64)


def round_fp16(x):
    return np.asarray(x, np.float64).astype(np.float16).astype(np.float64)


def _identity(x):
    return np.asarray(x, np.float64)


DACT_LO, DACT_HI = -0.25, 1.25   # range of the 8-bit F' code; covers F' of all four activations


def round_u8_dact(x):
    """F' stored as an 8-bit code: round((x - lo) * 255 / (hi - lo)), decoded back."""
    scale = 255.0 / (DACT_HI - DACT_LO)
    code = np.clip(np.rint((np.asarray(x, np.float64) - DACT_LO) * scale), 0, 255)
    return code / scale + DACT_LO


ROUNDING_POINTS = ("r", "w", "g", "dact", "ag")


def forward_backward(A, Wa, J0, J1, Wo, r_init, alpha, activation_name, grad_output=None, rounding=True,
                     folded=False, dact="fp16", only=None):
    """Returns dict(bump_history [T,B,N], and, when grad_output is given, grad_Wa, grad_Wo, grad_r_init, grad_A).
    folded: model of the weight-resident kernels, whose bf16 Wo operand is round(J1 * Wo + J0) (formed in fp32), so
    that J0 * sum_j x_j + J1 * (x Wo^T) is one product over the bf16 operand copy of x; otherwise (the streaming
    kernels) Wo is rounded alone, J1 is applied in fp32 and the J0 row sums run over the fp32 values.
    dact: storage format of F', "fp16" or "u8".
    only: None rounds at every point; otherwise the subset of ROUNDING_POINTS to round at, everything else exact --
    "r" the forward's state operand, "w" the weight operands (Wa and Wo, or the folded J1 * Wo + J0), "g" the
    backward's operand, "dact" the stored derivative, "ag" the gated operand of the weight-gradient contraction.
    Used to attribute a deviation from fp64 to the operand that causes it."""
    if only is not None:
        unknown = set(only) - set(ROUNDING_POINTS)
        if unknown:
            raise ValueError(f"unknown rounding points {sorted(unknown)}; choose from {ROUNDING_POINTS}")
    on = (lambda name: rounding and (only is None or name in only))
    rb16_r = round_bf16 if on("r") else _identity
    rb16_w = round_bf16 if on("w") else _identity
    rb16_g = round_bf16 if on("g") else _identity
    rb16_ag = round_bf16 if on("ag") else _identity
    rf16 = (round_u8_dact if dact == "u8" else round_fp16) if on("dact") else _identity
    A = np.asarray(A, np.float64)
    Wa = np.asarray(Wa, np.float64)
    Wo = np.asarray(Wo, np.float64)
    r = np.array(r_init, np.float64)
    B, T, k = A.shape
    N = Wo.shape[0]
    Wob, Wab = rb16_w(Wo), rb16_w(Wa)
    if folded:   # fp32 fused multiply-add, then one rounding to bf16
        if on("w"):
            Wof = round_bf16((Wo * float(np.float32(J1)) + float(np.float32(J0))).astype(np.float32))
        else:
            Wof = Wo * J1 + J0
    hist = np.empty((T, B, N))
    D = np.empty((T, B, N))
    R = np.empty((T, B, N))
    Rfull = np.empty((T, B, N))
    for t in range(T):
        rb = rb16_r(r)
        R[t] = rb
        Rfull[t] = r
        re = rb @ Wof.T if folded else J0 * r.sum(axis=1, keepdims=True) + J1 * (rb @ Wob.T)
        for c in range(k):
            re = re + A[:, t, c:c + 1] * (rb @ Wab[c].T)
        D[t] = rf16(alpha * O.activation_derivative(re, activation_name))   # the kernels save alpha * F'
        r = (1.0 - alpha) * r + alpha * O.activation(re, activation_name)
        hist[t] = r
    out = {"bump_history": hist}
    if grad_output is None:
        return out
    G_out = np.asarray(grad_output, np.float64)
    grad_Wo = np.zeros_like(Wo)
    grad_Wa = np.zeros_like(Wa)
    grad_A = np.zeros((B, T, k))
    carry = np.zeros((B, N))
    for t in range(T - 1, -1, -1):
        G = G_out[t] + carry
        g = D[t] * G
        gb = rb16_g(g)
        if folded:
            carry = (1.0 - alpha) * G + gb @ Wof
        else:
            carry = (1.0 - alpha) * G + J0 * g.sum(axis=1, keepdims=True) + J1 * (gb @ Wob)
        for c in range(k):
            pc = gb @ Wab[c]
            carry = carry + A[:, t, c:c + 1] * pc
            # dL/dA: the per-matrix product dotted with r_prev (the weight-resident kernels read its bf16 copy)
            grad_A[:, t, c] = (pc * (R[t] if folded else Rfull[t])).sum(axis=1)
        grad_Wo += J1 * (gb.T @ R[t])
        for c in range(k):
            grad_Wa[c] += rb16_ag(A[:, t, c:c + 1] * gb).T @ R[t]
    out.update(grad_Wo=grad_Wo, grad_Wa=grad_Wa, grad_r_init=carry, grad_A=grad_A)
    return out
