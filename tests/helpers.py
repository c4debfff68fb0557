"""Shared input builders for the parity tests (seeded on the CPU so that the oracle and
the GPU operator see identical bits)."""
from __future__ import annotations

import math

import torch


def randn(shape, seed, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def lognormal_lengths(total, seed, median=600.0, sigma=1.0, lo=16, hi=4096):
    """Document lengths: lognormal(median, sigma) clipped to [lo, hi], drawn until they
    fill `total`; the last one is truncated to fit, and a truncated tail shorter than
    `lo` is merged into the previous document."""
    g = torch.Generator().manual_seed(seed)
    lens, s = [], 0
    while s < total:
        L = int(round(math.exp(math.log(median) + sigma * torch.randn((), generator=g).item())))
        L = max(lo, min(hi, L))
        L = min(L, total - s)
        if L < lo and lens:
            lens[-1] += L
        else:
            lens.append(L)
        s += L
    return lens


def cu_from_lengths(lens):
    cu = [0]
    for L in lens:
        cu.append(cu[-1] + L)
    return torch.tensor(cu, dtype=torch.int32)


def rel_l2(a, b):
    a, b = a.double(), b.double()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def max_abs(a, b):
    return float((a.double() - b.double()).abs().max())


# (label, quantity, error, tolerance) of every check made through within(): the test session writes them
# out, worst first, when SBA_MARGINS_FILE names a file (see conftest.py), so that the distance of each
# parity check from its tolerance can be tracked from one kernel change to the next.
MARGINS = []


def within(label, quantity, err, tol):
    """assert err <= tol, and remember how close it came."""
    MARGINS.append((label, quantity, float(err), float(tol)))
    assert err <= tol, f"{label}: {quantity} error {err:.3e} exceeds {tol:.1e}"
