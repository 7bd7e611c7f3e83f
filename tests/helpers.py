"""Shared helpers for the parity tests."""
import numpy as np
import torch

from oracle.bounds_oracle import LinearBounds

RTOL = 1e-5     # parity bar: fp32 rel 1e-5 / abs 1e-6
ATOL = 1e-6


def rand_bounds(g, B, L, D, H, ordered=True, sw=0.5, sb=1.0, gap_w=0.05, gap_b=0.3):
    """Random bound object.  ordered=True gives uw >= lw, ub >= lb (what a
    verifier produces); ordered=False draws lw, uw independently, as the
    reference's own op test does (kernel_test/transformer_forward_test_bound.py:746-754)."""
    lw = (torch.rand(B, L, D, H, generator=g) - 0.5) * 2 * sw
    if ordered:
        uw = lw + torch.rand(B, L, D, H, generator=g) * gap_w
    else:
        uw = (torch.rand(B, L, D, H, generator=g) - 0.5) * 2 * sw
    lb = (torch.rand(B, L, H, generator=g) - 0.5) * 2 * sb
    ub = lb + torch.rand(B, L, H, generator=g) * gap_b
    return LinearBounds(lw, lb, uw, ub)


def as_bounds(d):
    return LinearBounds(d["lw"], d["lb"], d["uw"], d["ub"])


def f64(t):
    return t.detach().cpu().double().numpy()


def close(a, b, rtol=RTOL, atol=ATOL):
    a = torch.as_tensor(a).detach().cpu()
    b = torch.as_tensor(b).detach().cpu()
    return torch.allclose(a.double(), b.double(), rtol=rtol, atol=atol)


def worst(a, b):
    a = torch.as_tensor(a).detach().cpu().double()
    b = torch.as_tensor(b).detach().cpu().double()
    err = (a - b).abs()
    return float(err.max()), float((err / (ATOL + RTOL * b.abs())).max())
