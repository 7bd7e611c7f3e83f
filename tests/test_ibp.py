"""Interval bound propagation (the reference's method "ibp"): the oracle's interval operators are
pinned by sampling (CPU); the HIP kernels and the Bounds class in that mode against the oracle (GPU)."""
from types import SimpleNamespace

import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import rand_bounds, close

KINDS = ["relu", "tanh", "exp", "reciprocal", "sqr", "sqrt"]
TRUE = {"relu": torch.relu, "tanh": torch.tanh, "exp": torch.exp, "reciprocal": lambda v: 1.0 / v,
        "sqr": lambda v: v * v, "sqrt": torch.sqrt}


def intervals(g, kind, n=4000):
    l = torch.randn(n, generator=g) * 2
    u = l + torch.rand(n, generator=g) * 3
    if kind in ("reciprocal", "sqrt"):
        l = l.abs() + 0.05
        u = l + torch.rand(n, generator=g) * 3
    return l, u


@pytest.mark.parametrize("kind", KINDS)
def test_oracle_interval_contains_the_image_and_is_tight(kind):
    g = torch.Generator().manual_seed(81)
    l, u = intervals(g, kind)
    lo, hi = O.interval_unary(kind, l, u)
    t = torch.rand(64, l.numel(), generator=g)
    x = l + t * (u - l)
    y = TRUE[kind](x.double())
    assert bool((y >= lo.double() - 1e-6).all()) and bool((y <= hi.double() + 1e-6).all())
    # tight: both ends are attained (at an end point, or at zero for a square that straddles it)
    ends = torch.stack([TRUE[kind](l.double()), TRUE[kind](u.double())])
    attained_lo = torch.minimum(ends.min(0).values, torch.where((l <= 0) & (u >= 0) & (kind == "sqr"), 0.0, 1e30).double())
    assert torch.allclose(lo.double(), attained_lo, rtol=1e-6, atol=1e-7)
    assert torch.allclose(hi.double(), ends.max(0).values, rtol=1e-6, atol=1e-7)


def test_oracle_interval_product_is_the_range_of_the_corners():
    g = torch.Generator().manual_seed(82)
    xl = torch.randn(3000, generator=g); xu = xl + torch.rand(3000, generator=g)
    yl = torch.randn(3000, generator=g); yu = yl + torch.rand(3000, generator=g)
    lo, hi = O.interval_product(xl, xu, yl, yu)
    tx, ty = torch.rand(32, 3000, generator=g), torch.rand(32, 3000, generator=g)
    z = (xl + tx * (xu - xl)) * (yl + ty * (yu - yl))
    assert bool((z >= lo - 1e-6).all()) and bool((z <= hi + 1e-6).all())
    corners = torch.stack([xl * yl, xl * yu, xu * yl, xu * yu])
    assert torch.equal(lo, corners.min(0).values) and torch.equal(hi, corners.max(0).values)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", KINDS)
def test_hip_interval_kernels_match_the_oracle(kind):
    from faith_amd import ops
    g = torch.Generator().manual_seed(83)
    l, u = intervals(g, kind, 5001)
    lo, hi = ops.interval_unary(kind, l.cuda(), u.cuda())
    elo, ehi = O.interval_unary(kind, l, u)
    assert close(lo, elo) and close(hi, ehi)
    yl, yu = intervals(g, "relu", 5001)
    zl, zu = ops.interval_product(l.cuda(), u.cuda(), yl.cuda(), yu.cuda())
    el, eu = O.interval_product(l, u, yl, yu)
    assert torch.equal(zl.cpu(), el) and torch.equal(zu.cpu(), eu)


@pytest.mark.gpu
def test_bounds_class_in_ibp_mode():
    """args.method == "ibp": coefficients truncated to perturbed_words rows (Bounds.py:285-288) and
    zero after every relaxation; intervals follow the oracle through dense -> relu -> dense -> tanh,
    a product, and both dot products."""
    from faith_amd import Bounds
    g = torch.Generator().manual_seed(84)
    args = SimpleNamespace(perturbed_words=2, method="ibp")
    L, H = 5, 16
    lb = torch.randn(1, L, H, generator=g)
    ub = lb + 0.1 * torch.rand(1, L, H, generator=g)
    w = torch.zeros(1, L, 2 * H, H)
    x = Bounds(args, 2.0, 0.01, lw=w.cuda(), lb=lb.cuda(), uw=w.cuda().clone(), ub=ub.cuda())
    assert x.lw.shape == (1, L, 2, H)
    W1 = torch.randn(H, H, generator=g) / 4
    W2 = torch.randn(H, H, generator=g) / 4
    d1 = SimpleNamespace(weight=W1.cuda(), bias=None)
    d2 = SimpleNamespace(weight=W2.cuda(), bias=None)
    y = x.dense(d1).relu().dense(d2).tanh()

    def lin(l, u, W):
        Wp, Wn = W.t().clamp(min=0), W.t().clamp(max=0)
        return l @ Wp + u @ Wn, u @ Wp + l @ Wn
    l1, u1 = lin(lb, ub, W1)
    l1, u1 = O.interval_unary("relu", l1, u1)
    l2, u2 = lin(l1, u1, W2)
    l2, u2 = O.interval_unary("tanh", l2, u2)
    assert float(y.lw.abs().max()) == 0.0 and float(y.uw.abs().max()) == 0.0
    assert close(y.lb, l2, rtol=1e-5, atol=2e-6) and close(y.ub, u2, rtol=1e-5, atol=2e-6)
    # product and dot products of two interval objects
    z = y.multiply(x)
    el, eu = O.interval_product(l2, u2, lb, ub)
    assert close(z.lb, el, rtol=1e-5, atol=2e-6) and close(z.ub, eu, rtol=1e-5, atol=2e-6)
    s = y.dot_product(x)                                     # [1, L, L] scores
    c1 = l2.unsqueeze(2) * lb.unsqueeze(1); c2 = l2.unsqueeze(2) * ub.unsqueeze(1)
    c3 = u2.unsqueeze(2) * lb.unsqueeze(1); c4 = u2.unsqueeze(2) * ub.unsqueeze(1)
    lo = torch.min(torch.min(c1, c2), torch.min(c3, c4)).sum(-1)
    hi = torch.max(torch.max(c1, c2), torch.max(c3, c4)).sum(-1)
    assert s.lw.shape == (1, L, 2, L) and float(s.lw.abs().max()) == 0.0
    assert close(s.lb, lo, rtol=1e-5, atol=1e-5) and close(s.ub, hi, rtol=1e-5, atol=1e-5)
    ctx = s.context(x)                                       # [1, L, H]
    k1 = lo.unsqueeze(-1) * lb.unsqueeze(1); k2 = lo.unsqueeze(-1) * ub.unsqueeze(1)
    k3 = hi.unsqueeze(-1) * lb.unsqueeze(1); k4 = hi.unsqueeze(-1) * ub.unsqueeze(1)
    clo = torch.min(torch.min(k1, k2), torch.min(k3, k4)).sum(2)
    chi = torch.max(torch.max(k1, k2), torch.max(k3, k4)).sum(2)
    assert ctx.lw.shape == (1, L, 2, H)
    assert close(ctx.lb, clo, rtol=1e-5, atol=1e-4) and close(ctx.ub, chi, rtol=1e-5, atol=1e-4)


@pytest.mark.gpu
def test_ibp_pipeline_is_sound_and_looser_than_linear_bounds():
    """A whole encoder layer with method "ibp" through forward.py: the true outputs of sampled
    perturbations (infinity norm, the set ibp's input interval describes) lie inside, and the
    linear-bound method is at least as tight on the same problem."""
    from faith_amd import Bounds, forward as F
    from tests.oracle_bounds import random_layer, to_device, true_layer
    HIDDEN, HEADS, INTER, LENGTH = 32, 4, 64, 6
    g = torch.Generator().manual_seed(85)
    layer = random_layer(g, HIDDEN, HEADS, INTER)
    norm = SimpleNamespace(weight=1.0 + 0.1 * torch.randn(HIDDEN, generator=g), bias=0.05 * torch.randn(HIDDEN, generator=g))
    pooler = SimpleNamespace(weight=torch.randn(HIDDEN, HIDDEN, generator=g) / HIDDEN ** 0.5, bias=0.05 * torch.randn(HIDDEN, generator=g))
    clf = SimpleNamespace(weight=torch.randn(2, HIDDEN, generator=g) / HIDDEN ** 0.5, bias=0.05 * torch.randn(2, generator=g))
    emb = torch.randn(1, LENGTH, HIDDEN, generator=g)
    eps, index, p = 0.002, 2, float("inf")
    glayer, gnorm = to_device(layer, "cuda"), to_device(norm, "cuda")

    def run(args, ibp):
        make = lambda p_, e_, lw, lb, uw, ub: Bounds(args, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
        x = F.bound_input(make, emb.cuda(), index, eps, 1, p, gnorm, "no_var", ibp=ibp)
        _, _, out = F.bound_layer(x, glayer, "no_var", "relu")
        return out.concretize()
    il, iu = run(SimpleNamespace(perturbed_words=1, method="ibp"), True)
    ll, lu = run(SimpleNamespace(perturbed_words=1), False)
    d = torch.sign(torch.randn(64, HIDDEN, generator=g, dtype=torch.float64)) * eps * torch.rand(64, 1, generator=g, dtype=torch.float64)
    x = emb.double().repeat(64, 1, 1)
    x[:, index] += d
    out, _ = true_layer(x, layer, norm, "no_var", pooler, clf)
    for lo, hi in ((il, iu), (ll, lu)):
        assert bool((out >= lo.cpu().double() - 1e-4).all()) and bool((out <= hi.cpu().double() + 1e-4).all())
    assert float((iu - il).mean()) >= float((lu - ll).mean())
