"""Pins oracle/bounds_oracle.py against things that do not share its code:
library routines, closed forms, brute-force loops and soundness sampling.

The reference holds no golden vectors for this path (its only op test draws
random inputs at run time and stores nothing), so these checks are what makes
the oracle trustworthy.  CPU only.
"""
import math

import numpy as np
import pytest
import torch

from oracle import bounds_oracle as O
from oracle import closed_form as C
from tests.helpers import rand_bounds, f64

INF = float("inf")
PS = [1.0, 2.0, INF, 3.0, 1.5]     # 3.0 and 1.5: general dual exponents (1.5 and 3)


def gen(seed):
    return torch.Generator().manual_seed(seed)


# ----------------------------------------------------------------- concretize
@pytest.mark.parametrize("p", PS + [3.0])
@pytest.mark.parametrize("words", [1, 2, 4])
def test_concretize_vs_numpy(p, words):
    x = rand_bounds(gen(1), 2, 3, 8, 5, ordered=False)
    lo, hi = O.concretize(x, p, 0.37, words)
    q = C.dual(p)
    lw, lb, uw, ub = map(f64, x.tensors())
    for b in range(2):
        for l in range(3):
            for j in range(5):
                el, eu = lb[b, l, j], ub[b, l, j]
                n = 8 // words
                for w in range(words):
                    el -= 0.37 * np.linalg.norm(lw[b, l, w * n:(w + 1) * n, j], ord=q)
                    eu += 0.37 * np.linalg.norm(uw[b, l, w * n:(w + 1) * n, j], ord=q)
                assert abs(lo[b, l, j].item() - el) < 1e-5
                assert abs(hi[b, l, j].item() - eu) < 1e-5


def test_concretize_special_cases():
    x = rand_bounds(gen(2), 1, 2, 6, 4)
    zero = O.LinearBounds(torch.zeros_like(x.lw), x.lb, torch.zeros_like(x.uw), x.ub)
    for p in PS:
        lo, hi = O.concretize(zero, p, 0.5, 1)
        assert torch.equal(lo, x.lb) and torch.equal(hi, x.ub)
    # a single non-zero entry per column: every q-norm equals its magnitude
    onehot = torch.zeros_like(x.lw)
    onehot[:, :, 3, :] = -2.5
    x1 = O.LinearBounds(onehot, x.lb, -onehot, x.ub)
    for p in PS:
        lo, hi = O.concretize(x1, p, 0.1, 1)
        assert torch.allclose(lo, x.lb - 0.25) and torch.allclose(hi, x.ub + 0.25)
    # p = inf (q = 1) is additive over blocks: words does not matter
    a = O.concretize(x, INF, 0.3, 1)
    b = O.concretize(x, INF, 0.3, 3)
    assert torch.allclose(a[0], b[0], atol=1e-6) and torch.allclose(a[1], b[1], atol=1e-6)
    # p = 1 (q = inf): two words give max(block0) + max(block1), not the overall max
    c = O.concretize(x, 1.0, 0.3, 2)
    exp = x.lb - 0.3 * (x.lw[:, :, :3].abs().amax(2) + x.lw[:, :, 3:].abs().amax(2))
    assert torch.allclose(c[0], exp, atol=1e-6)


# --------------------------------------------------------------------- linear
def test_linear_vs_brute_force():
    x = rand_bounds(gen(3), 1, 3, 4, 6, ordered=False)
    W = torch.randn(5, 6, generator=gen(4))
    W[0, 0] = 0.0
    bias = torch.randn(5, generator=gen(5))
    y = O.linear(x, W, bias)
    e = C.linear_brute(*(f64(t)[0] for t in (x.lw, x.lb, x.uw, x.ub)), f64(W), f64(bias))
    for got, exp in zip((y.lw, y.lb, y.uw, y.ub), e):
        np.testing.assert_allclose(f64(got)[0], exp, rtol=1e-5, atol=1e-6)


def test_linear_closed_forms():
    x = rand_bounds(gen(6), 1, 4, 5, 7)
    W = torch.randn(3, 7, generator=gen(7))
    # non-negative weights: each side is an ordinary product
    y = O.linear(x, W.abs())
    assert torch.allclose(y.lw, x.lw @ W.abs().t(), atol=1e-6)
    assert torch.allclose(y.uw, x.uw @ W.abs().t(), atol=1e-6)
    # non-positive weights: sides swap
    y = O.linear(x, -W.abs())
    assert torch.allclose(y.lw, x.uw @ (-W.abs()).t(), atol=1e-6)
    assert torch.allclose(y.ub, x.lb @ (-W.abs()).t(), atol=1e-6)
    # degenerate bounds: both sides equal x @ W^T
    pt = O.LinearBounds(x.lw, x.lb, x.lw, x.lb)
    y = O.linear(pt, W)
    assert torch.allclose(y.lw, x.lw @ W.t(), atol=1e-5) and torch.allclose(y.uw, y.lw, atol=1e-6)
    # width identity: uw' - lw' = (uw - lw) @ |W|^T
    y = O.linear(x, W)
    assert torch.allclose(y.uw - y.lw, (x.uw - x.lw) @ W.abs().t(), atol=1e-5)
    assert torch.allclose(y.ub - y.lb, (x.ub - x.lb) @ W.abs().t(), atol=1e-5)
    # bias shifts lb and ub only
    b = torch.randn(3, generator=gen(8))
    yb = O.linear(x, W, b)
    assert torch.equal(yb.lw, y.lw) and torch.allclose(yb.lb, y.lb + b) and torch.allclose(yb.ub, y.ub + b)


# ----------------------------------------------------------------------- relu
@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("words", [1, 2])
@pytest.mark.parametrize("ordered", [True, False])
def test_relu_vs_per_neuron_closed_form(p, words, ordered):
    x = rand_bounds(gen(9), 1, 3, 8, 16, ordered=ordered, sb=2.0)
    y = O.relu(x, p, 0.2, words)
    lw, lb, uw, ub = (f64(t)[0] for t in x.tensors())
    seen = set()
    for l in range(3):
        for j in range(16):
            e = C.relu_neuron(lw[l, :, j], lb[l, j], uw[l, :, j], ub[l, j], p, 0.2, words)
            lo, hi = C.interval(lw[l, :, j], lb[l, j], uw[l, :, j], ub[l, j], p, 0.2, words)
            seen.add("neg" if hi < 0 else "pos" if lo > 0 else "both")
            np.testing.assert_allclose(f64(y.lw)[0, l, :, j], e[0], rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(f64(y.lb)[0, l, j], e[1], rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(f64(y.uw)[0, l, :, j], e[2], rtol=1e-5, atol=1e-6)
            np.testing.assert_allclose(f64(y.ub)[0, l, j], e[3], rtol=1e-5, atol=1e-6)
    assert seen == {"neg", "pos", "both"}


def _sample_delta(g, D, p, eps, n):
    """n perturbations with ||delta||_p <= eps, a good share on the boundary."""
    d = torch.randn(n, D, generator=g, dtype=torch.float64)
    if math.isinf(p):
        d = torch.sign(d) * eps * torch.rand(n, 1, generator=g, dtype=torch.float64).clamp(min=0.5)
        d[: n // 2] = torch.sign(d[: n // 2]) * eps
    else:
        d = d / torch.linalg.vector_norm(d, ord=p, dim=1, keepdim=True) * eps
        d[n // 2:] *= torch.rand(n - n // 2, 1, generator=g, dtype=torch.float64)
    return d


def _eval(w, b, delta):
    """value of w . delta + b for each delta: w [L,D,H], b [L,H] -> [n,L,H]"""
    return torch.einsum("nd,ldh->nlh", delta, w.double()) + b.double()


@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("act", ["relu", "tanh"])
def test_activation_soundness(p, act):
    """For any admissible delta and any pre-activation v between its two bound
    lines, act(v) must lie between the propagated lines."""
    g = gen(10)
    x = rand_bounds(g, 1, 4, 6, 32, ordered=True, sb=1.2, gap_b=0.4)
    x.ub += 0.1      # keeps the lower line under the upper one on the whole ball
    eps = 0.3
    y = getattr(O, act)(x, p, eps, 1)
    fn = torch.relu if act == "relu" else torch.tanh
    delta = _sample_delta(g, 6, p, eps, 400)
    lo_in = _eval(x.lw[0], x.lb[0], delta)
    hi_in = _eval(x.uw[0], x.ub[0], delta)
    assert (lo_in <= hi_in + 1e-9).all()
    lo_out = _eval(y.lw[0], y.lb[0], delta)
    hi_out = _eval(y.uw[0], y.ub[0], delta)
    # tanh: ten bisection steps stop (range / 2^11) short of the tangent point (or of
    # the interval end when the tangent point lies outside it), which lets the
    # reference's line cross the curve by a few 1e-5; that is the algorithm's
    # own slack, not a rounding effect.
    slack = 1e-5 if act == "relu" else 1e-4
    for t in (0.0, 0.3, 1.0):
        v = fn(lo_in + t * (hi_in - lo_in))
        assert (v >= lo_out - slack).all()
        assert (v <= hi_out + slack).all()


def test_relu_branch_invariants():
    x = rand_bounds(gen(11), 1, 2, 4, 64, sb=0.1)
    up = O.LinearBounds(x.lw, x.lb + 10, x.uw, x.ub + 10)      # all active
    y = O.relu(up, 2.0, 0.1)
    for a, b in zip(y.tensors(), up.tensors()):
        assert torch.equal(a, b)
    dn = O.LinearBounds(x.lw, x.lb - 10, x.uw, x.ub - 10)      # all dead
    y = O.relu(dn, 2.0, 0.1)
    for a in y.tensors():
        assert torch.count_nonzero(a) == 0


# ----------------------------------------------------------------------- tanh
@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("words", [1, 2])
def test_tanh_vs_scalar_loop(p, words):
    x = rand_bounds(gen(12), 1, 3, 8, 24, ordered=True, sb=1.5, gap_b=0.6)
    y = O.tanh(x, p, 0.2, words)
    lw, lb, uw, ub = (f64(t)[0] for t in x.tensors())
    seen = set()
    for l in range(3):
        for j in range(24):
            e = C.tanh_neuron(lw[l, :, j], lb[l, j], uw[l, :, j], ub[l, j], p, 0.2, words)
            lo, hi = C.interval(lw[l, :, j], lb[l, j], uw[l, :, j], ub[l, j], p, 0.2, words)
            seen.add("neg" if hi < 0 else "pos" if lo > 0 else "both")
            # fp32 transcendental error is amplified by 1/(u-l) in the chord slope
            tol = dict(rtol=2e-4, atol=2e-5)
            np.testing.assert_allclose(f64(y.lw)[0, l, :, j], e[0], **tol)
            np.testing.assert_allclose(f64(y.lb)[0, l, j], e[1], **tol)
            np.testing.assert_allclose(f64(y.uw)[0, l, :, j], e[2], **tol)
            np.testing.assert_allclose(f64(y.ub)[0, l, j], e[3], **tol)
    assert seen == {"neg", "pos", "both"}


def test_tanh_odd_symmetry():
    """tanh is odd: negating the input bound object (and swapping its sides)
    negates and swaps the output."""
    x = rand_bounds(gen(13), 1, 2, 6, 40, sb=1.5, gap_b=0.5)
    y = O.tanh(x, 2.0, 0.25)
    xm = O.LinearBounds(-x.uw, -x.ub, -x.lw, -x.lb)
    ym = O.tanh(xm, 2.0, 0.25)
    assert torch.allclose(ym.lw, -y.uw, rtol=1e-4, atol=1e-5)
    assert torch.allclose(ym.lb, -y.ub, rtol=1e-4, atol=1e-5)
    assert torch.allclose(ym.uw, -y.lw, rtol=1e-4, atol=1e-5)
    assert torch.allclose(ym.ub, -y.lb, rtol=1e-4, atol=1e-5)


def test_tanh_lines_bound_the_function():
    for lo, hi in [(-2.0, -0.5), (0.2, 3.0), (-1.0, 2.0), (-3.0, 0.1), (-1e-3, 1e-3), (-4, 4)]:
        (kl, xl, yl), (ku, xu, yu) = C.tanh_lines(lo, hi)
        xs = np.linspace(lo, hi, 201)
        # ten bisection steps stop short of the interval end when the true tangent
        # point lies outside [lo, hi]; the line then crosses the curve by ~3e-5
        # (measured: (-3, 0.1) and (-0.26, 1.4)).  Property of the algorithm.
        slack = 1e-4
        assert (kl * (xs - xl) + yl <= np.tanh(xs) + slack).all()
        assert (ku * (xs - xu) + yu >= np.tanh(xs) - slack).all()


def test_tanh_bisection_lands_on_the_tangent_point():
    """Where the true tangent point lies inside the bracket the ten bisection steps (Bounds.py:1063-1097) must end
    next to it: the lower line through (u, tanh u) touches the curve on [l, 0], the upper line through (l, tanh l)
    touches it on [0, u] (gap ~ curvature x (bracket / 2^11)^2), and each stays on its side of the curve.  A
    bisection that moves the wrong end of its bracket ends at l, 0 or u instead: the line then cuts through the
    curve or stands off it by far more."""
    for lo, hi in [(-4.0, 4.0), (-2.0, 3.0), (-3.0, 1.5), (-1.0, 1.2)]:
        (kl, xl, yl), (ku, xu, yu) = C.tanh_lines(lo, hi)
        xs = np.linspace(lo, hi, 20001)
        gap_l = np.tanh(xs) - (kl * (xs - xl) + yl)
        gap_u = (ku * (xs - xu) + yu) - np.tanh(xs)
        # the brackets are [lo, 0] and [0, hi]: 2^-11 of their length after ten steps
        for gap, side, bracket in ((gap_l, xs <= 0, -lo), (gap_u, xs >= 0, hi)):
            assert gap.min() > -1e-4
            assert gap[side].min() < 4 * (bracket / 2048) ** 2 + 1e-6, (lo, hi, gap[side].min())
        # the line's anchor is the tangent point itself: slope = derivative there, to first order in the bracket
        assert abs(kl - (1 - np.tanh(xl) ** 2)) < 4 * (-lo / 2048) + 1e-6
        assert abs(ku - (1 - np.tanh(xu) ** 2)) < 4 * (hi / 2048) + 1e-6
        assert lo < xl < 0 < xu < hi


# ---------------------------------------------------------------- dot product
@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("words", [1, 2])
def test_dot_vs_brute_force(p, words):
    g = gen(14)
    x = rand_bounds(g, 2, 3, 4, 5, ordered=False, sb=1.0)
    y = rand_bounds(g, 2, 2, 4, 5, ordered=False, sb=1.0)
    z = O.dot_product(x, y, p, 0.3, words)
    assert z.lw.shape == (2, 3, 4, 2) and z.lb.shape == (2, 3, 2)
    for t in range(2):
        e = C.dot_brute(*(f64(a)[t] for a in (x.lw, x.lb, x.uw, x.ub, y.lw, y.lb, y.uw, y.ub)),
                        p, 0.3, words)
        for got, exp in zip((z.lw, z.lb, z.uw, z.ub), e):
            np.testing.assert_allclose(f64(got)[t], exp, rtol=1e-5, atol=2e-6)


def test_dot_vs_einsum():
    """Tensor restatement with einsum, the way the reference's TIR experiment
    emulates the weight term (tvm_kernels/TIR_kernel/verify_dot_product_w_tir.py:137-179)."""
    g = gen(15)
    x = rand_bounds(g, 1, 6, 8, 4)
    y = rand_bounds(g, 1, 5, 8, 4)
    z = O.dot_product(x, y, 2.0, 0.1)
    lx, _ = O.concretize(x, 2.0, 0.1)
    ly, uy = O.concretize(y, 2.0, 0.1)
    lx, ly, uy = lx[0], ly[0], uy[0]
    pos, neg = (lambda v: v.clamp(min=0)), (lambda v: v.clamp(max=0))
    lw = (torch.einsum("imk,jk->imj", x.lw[0], pos(ly)) + torch.einsum("imk,jk->imj", x.uw[0], neg(ly))
          + torch.einsum("jmk,ik->imj", y.lw[0], pos(lx)) + torch.einsum("jmk,ik->imj", y.uw[0], neg(lx)))
    uw = (torch.einsum("imk,jk->imj", x.uw[0], pos(uy)) + torch.einsum("imk,jk->imj", x.lw[0], neg(uy))
          + torch.einsum("jmk,ik->imj", y.uw[0], pos(lx)) + torch.einsum("jmk,ik->imj", y.lw[0], neg(lx)))
    assert torch.allclose(z.lw[0], lw, rtol=1e-5, atol=1e-6)
    assert torch.allclose(z.uw[0], uw, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("p", PS)
def test_dot_soundness(p):
    g = gen(16)
    D, d, eps = 5, 6, 0.25
    x = rand_bounds(g, 1, 4, D, d, sb=1.0)
    y = rand_bounds(g, 1, 3, D, d, sb=1.0)
    x.ub += 0.1      # lower line <= upper line on the whole ball
    y.ub += 0.1
    z = O.dot_product(x, y, p, eps)
    delta = _sample_delta(g, D, p, eps, 300)
    xl, xu = _eval(x.lw[0], x.lb[0], delta), _eval(x.uw[0], x.ub[0], delta)
    yl, yu = _eval(y.lw[0], y.lb[0], delta), _eval(y.uw[0], y.ub[0], delta)
    zl = torch.einsum("nd,idj->nij", delta, z.lw[0].double()) + z.lb[0].double()
    zu = torch.einsum("nd,idj->nij", delta, z.uw[0].double()) + z.ub[0].double()
    for tx, ty in [(0, 0), (0, 1), (1, 0), (1, 1), (0.4, 0.7)]:
        xv = xl + tx * (xu - xl)
        yv = yl + ty * (yu - yl)
        prod = torch.einsum("nik,njk->nij", xv, yv)
        assert (prod >= zl - 1e-5).all()
        assert (prod <= zu + 1e-5).all()


def test_dot_interval_shortcut():
    g = gen(17)
    x = rand_bounds(g, 2, 3, 1, 4)
    y = rand_bounds(g, 2, 5, 1, 4)
    z = O.dot_product(x, y, 2.0, 0.1)
    assert z.lb.shape == (2, 3, 5) and torch.count_nonzero(z.lw) == 0
    for t in range(2):
        for i in range(3):
            for j in range(5):
                lo = hi = 0.0
                for k in range(4):
                    c = [a * b for a in (x.lb[t, i, k].item(), x.ub[t, i, k].item())
                         for b in (y.lb[t, j, k].item(), y.ub[t, j, k].item())]
                    lo += min(c); hi += max(c)
                assert abs(z.lb[t, i, j].item() - lo) < 1e-5 and abs(z.ub[t, i, j].item() - hi) < 1e-5


# ----------------------------------------------------------------------- conv
@pytest.mark.parametrize("stride,pad,K", [(1, 1, 3), (2, 0, 3), (1, 0, 1), (2, 2, 5)])
def test_conv_vs_brute_force(stride, pad, K):
    g = gen(18)
    D, Ci, Co, Hh = 3, 2, 4, 7
    lw = torch.randn(1, D, Ci, Hh, Hh, generator=g)
    uw = torch.randn(1, D, Ci, Hh, Hh, generator=g)
    lb = torch.randn(1, Ci, Hh, Hh, generator=g)
    ub = lb + torch.rand(1, Ci, Hh, Hh, generator=g)
    W = torch.randn(Co, Ci, K, K, generator=g)
    W[0, 0, 0, 0] = 0
    bias = torch.randn(Co, generator=g)
    y = O.conv2d(O.LinearBounds(lw, lb, uw, ub), W, bias, stride, pad)
    el, eu = C.conv_brute(f64(lw)[0], f64(uw)[0], f64(W), stride, pad)
    np.testing.assert_allclose(f64(y.lw)[0], el, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(f64(y.uw)[0], eu, rtol=1e-5, atol=1e-5)
    bl, bu = C.conv_brute(f64(lb), f64(ub), f64(W), stride, pad)
    np.testing.assert_allclose(f64(y.lb), bl + f64(bias).reshape(1, -1, 1, 1), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(f64(y.ub), bu + f64(bias).reshape(1, -1, 1, 1), rtol=1e-5, atol=1e-5)


def test_conv_1x1_equals_linear():
    g = gen(19)
    D, Ci, Co, Hh = 4, 6, 5, 3
    lw = torch.randn(1, D, Ci, Hh, Hh, generator=g)
    uw = lw + torch.rand(1, D, Ci, Hh, Hh, generator=g)
    lb = torch.randn(1, Ci, Hh, Hh, generator=g)
    ub = lb + torch.rand(1, Ci, Hh, Hh, generator=g)
    W = torch.randn(Co, Ci, 1, 1, generator=g)
    bias = torch.randn(Co, generator=g)
    y = O.conv2d(O.LinearBounds(lw, lb, uw, ub), W, bias)
    # pixels as the length axis, channels as the hidden axis
    as_lin = O.LinearBounds(lw[0].permute(2, 3, 0, 1).reshape(1, Hh * Hh, D, Ci),
                            lb[0].permute(1, 2, 0).reshape(1, Hh * Hh, Ci),
                            uw[0].permute(2, 3, 0, 1).reshape(1, Hh * Hh, D, Ci),
                            ub[0].permute(1, 2, 0).reshape(1, Hh * Hh, Ci))
    z = O.linear(as_lin, W.view(Co, Ci), bias)
    assert torch.allclose(y.lw[0].permute(2, 3, 0, 1).reshape(1, Hh * Hh, D, Co), z.lw, atol=1e-5)
    assert torch.allclose(y.ub[0].permute(1, 2, 0).reshape(1, Hh * Hh, Co), z.ub, atol=1e-5)


def test_conv_concretize_soundness():
    g = gen(20)
    D, Ci, Co, Hh, eps = 4, 3, 5, 6, 0.2
    lw = torch.randn(1, D, Ci, Hh, Hh, generator=g)
    uw = lw + 0.1 * torch.rand(1, D, Ci, Hh, Hh, generator=g)
    lb = torch.randn(1, Ci, Hh, Hh, generator=g)
    ub = lb + 0.1 + 0.2 * torch.rand(1, Ci, Hh, Hh, generator=g)
    W = torch.randn(Co, Ci, 3, 3, generator=g)
    y = O.conv2d(O.LinearBounds(lw, lb, uw, ub), W, None, 1, 1)
    lo, hi = O.concretize_conv(y, INF, eps)
    delta = _sample_delta(g, D, INF, eps, 100)
    xin_l = torch.einsum("nd,dchw->nchw", delta, lw[0].double()) + lb.double()
    xin_u = torch.einsum("nd,dchw->nchw", delta, uw[0].double()) + ub.double()
    for t in (0.0, 0.5, 1.0):
        v = torch.nn.functional.conv2d(xin_l + t * (xin_u - xin_l), W.double(), None, 1, 1)
        assert (v >= lo.double() - 1e-5).all() and (v <= hi.double() + 1e-5).all()


# -------------------------------------------------------------------- context
@pytest.mark.parametrize("p", PS)
def test_context_vs_brute_force(p):
    """probs . value with the value object transposed by hand in numpy (no torch views)."""
    g = gen(21)
    L, D, dv = 4, 3, 5
    probs = rand_bounds(g, 2, L, D, L, ordered=False)
    value = rand_bounds(g, 2, L, D, dv, ordered=False)
    z = O.context(probs, value, p, 0.2)
    assert z.lw.shape == (2, L, D, dv) and z.lb.shape == (2, L, dv)
    for t in range(2):
        y = [np.ascontiguousarray(f64(a)[t].transpose(2, 1, 0)) for a in (value.lw, value.uw)]     # [dv, D, L]
        yb = [np.ascontiguousarray(f64(a)[t].T) for a in (value.lb, value.ub)]                      # [dv, L]
        e = C.dot_brute(f64(probs.lw)[t], f64(probs.lb)[t], f64(probs.uw)[t], f64(probs.ub)[t],
                        y[0], yb[0], y[1], yb[1], p, 0.2, 1)
        for got, exp in zip((z.lw, z.lb, z.uw, z.ub), e):
            np.testing.assert_allclose(f64(got)[t], exp, rtol=1e-5, atol=2e-6)


# ------------------------------------------------- exp / reciprocal / sqr / sqrt
def _unary_input(kind, g, ordered=True):
    x = rand_bounds(g, 1, 3, 8, 24, ordered=ordered, sw=0.1, sb=1.5, gap_w=0.02, gap_b=0.5)
    if kind in ("reciprocal", "sqrt"):          # strictly positive pre-activations
        x = O.LinearBounds(x.lw, x.lb.abs() + 1.0, x.uw, x.lb.abs() + 1.0 + (x.ub - x.lb))
    return x


@pytest.mark.parametrize("kind", ["exp", "reciprocal", "sqr", "sqrt"])
@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("words", [1, 2])
def test_unary_vs_per_neuron_closed_form(kind, p, words):
    x = _unary_input(kind, gen(22))
    y = getattr(O, kind)(x, p, 0.2, words)
    fn = getattr(C, kind + "_neuron")
    lw, lb, uw, ub = (f64(t)[0] for t in x.tensors())
    for l in range(3):
        for j in range(24):
            e = fn(lw[l, :, j], lb[l, j], uw[l, :, j], ub[l, j], p, 0.2, words)
            tol = dict(rtol=2e-5, atol=1e-5)
            np.testing.assert_allclose(f64(y.lw)[0, l, :, j], e[0], **tol)
            np.testing.assert_allclose(f64(y.lb)[0, l, j], e[1], **tol)
            np.testing.assert_allclose(f64(y.uw)[0, l, :, j], e[2], **tol)
            np.testing.assert_allclose(f64(y.ub)[0, l, j], e[3], **tol)


@pytest.mark.parametrize("kind", ["exp", "reciprocal", "sqr", "sqrt"])
@pytest.mark.parametrize("p", PS)
def test_unary_soundness(kind, p):
    g = gen(23)
    x = _unary_input(kind, g)
    x.ub += 0.1
    eps = 0.3
    y = getattr(O, kind)(x, p, eps, 1)
    fn = {"exp": torch.exp, "reciprocal": torch.reciprocal, "sqr": torch.square, "sqrt": torch.sqrt}[kind]
    delta = _sample_delta(g, 8, p, eps, 300)
    lo_in, hi_in = _eval(x.lw[0], x.lb[0], delta), _eval(x.uw[0], x.ub[0], delta)
    lo_out, hi_out = _eval(y.lw[0], y.lb[0], delta), _eval(y.uw[0], y.ub[0], delta)
    for t in (0.0, 0.4, 1.0):
        v = fn(lo_in + t * (hi_in - lo_in))
        assert (v >= lo_out - 1e-5 * (1 + v.abs())).all()
        assert (v <= hi_out + 1e-5 * (1 + v.abs())).all()


def test_exp_saturates_above_threshold():
    """Above 12 the reference switches exp to its tangent (Bounds.py:984-989)."""
    lw = torch.zeros(1, 1, 2, 3); lb = torch.tensor([[[11.0, 12.5, 20.0]]]); ub = lb + 1.0
    y = O.exp(O.LinearBounds(lw, lb, lw, ub), 2.0, 0.1)
    e12 = math.exp(12.0)
    for j, (lo, hi) in enumerate([(11.0, 12.0), (12.5, 13.5), (20.0, 21.0)]):
        cap = lambda v: math.exp(v) if v < 12 else e12 * (v - 11.0)
        ku = (cap(hi) - cap(lo)) / (hi - lo)
        assert abs(y.ub[0, 0, j].item() - (hi * ku - ku * lo + cap(lo))) / cap(hi) < 1e-5


# ------------------------------------ scale / add / multiply / divide / softmax / layer_norm
def test_scale_and_add_definitions():
    x = rand_bounds(gen(24), 1, 2, 4, 6, ordered=False)
    y = rand_bounds(gen(25), 1, 2, 4, 6, ordered=False)
    s = O.scale(x, 2.5)
    assert torch.equal(s.lw, x.lw * 2.5) and torch.equal(s.ub, x.ub * 2.5)
    s = O.scale(x, -2.0)                                   # negative factor swaps the sides
    assert torch.equal(s.lw, x.uw * -2.0) and torch.equal(s.lb, x.ub * -2.0) and torch.equal(s.uw, x.lw * -2.0)
    W = torch.tensor([1.0, -2.0, 0.0, 0.5, -0.25, 3.0])
    s = O.scale(x, W)
    for j, w in enumerate(W.tolist()):
        a, b = (x.lw, x.uw) if w > 0 else (x.uw, x.lw)
        assert torch.allclose(s.lw[..., j], a[..., j] * w) and torch.allclose(s.uw[..., j], b[..., j] * w)
    z = O.add(x, y)
    assert torch.equal(z.lw, x.lw + y.lw) and torch.equal(z.ub, x.ub + y.ub)
    z = O.add(x, 0.5)
    assert torch.equal(z.lw, x.lw) and torch.equal(z.lb, x.lb + 0.5)


@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("words", [1, 2])
def test_multiply_vs_brute_force(p, words):
    """An elementwise product is a dot product with a reduction of length one."""
    g = gen(26)
    x = rand_bounds(g, 1, 3, 4, 7, ordered=False)
    y = rand_bounds(g, 1, 3, 4, 7, ordered=False)
    z = O.multiply(x, y, p, 0.3, words)
    for l in range(3):
        for j in range(7):
            col = lambda t_: f64(t_)[0, l, :, j].reshape(1, 4, 1)
            sc = lambda t_: f64(t_)[0, l, j].reshape(1, 1)
            e = C.dot_brute(col(x.lw), sc(x.lb), col(x.uw), sc(x.ub), col(y.lw), sc(y.lb), col(y.uw), sc(y.ub),
                            p, 0.3, words)
            np.testing.assert_allclose(f64(z.lw)[0, l, :, j], e[0][0, :, 0], rtol=1e-5, atol=2e-6)
            np.testing.assert_allclose(f64(z.lb)[0, l, j], e[1][0, 0], rtol=1e-5, atol=2e-6)
            np.testing.assert_allclose(f64(z.uw)[0, l, :, j], e[2][0, :, 0], rtol=1e-5, atol=2e-6)
            np.testing.assert_allclose(f64(z.ub)[0, l, j], e[3][0, 0], rtol=1e-5, atol=2e-6)


def _bounded_between(fn, x, y, g, D, p, eps, slack=1e-4):
    delta = _sample_delta(g, D, p, eps, 200)
    lo_in, hi_in = _eval(x.lw[0], x.lb[0], delta), _eval(x.uw[0], x.ub[0], delta)
    lo_out, hi_out = _eval(y.lw[0], y.lb[0], delta), _eval(y.uw[0], y.ub[0], delta)
    for t in (0.0, 0.35, 1.0):
        v = fn(lo_in + t * (hi_in - lo_in))
        assert (v >= lo_out - slack * (1 + v.abs())).all(), float((lo_out - v).max())
        assert (v <= hi_out + slack * (1 + v.abs())).all(), float((v - hi_out).max())


@pytest.mark.parametrize("p", PS)
def test_softmax_soundness(p):
    g = gen(27)
    x = rand_bounds(g, 1, 3, 5, 8, sw=0.1, sb=1.0, gap_w=0.01, gap_b=0.05)
    x.ub += 0.02
    y = O.softmax(x, p, 0.1)
    _bounded_between(lambda v: torch.softmax(v, dim=-1), x, y, g, 5, p, 0.1)
    # the bounds of one row of probabilities must bracket a distribution: sum l <= 1 <= sum u
    lo, hi = O.concretize(y, p, 0.1)
    assert (lo.sum(-1) <= 1 + 1e-5).all() and (hi.sum(-1) >= 1 - 1e-5).all()


@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("mode", ["no_var", "standard"])
def test_layer_norm_soundness(p, mode):
    g = gen(28)
    H = 8
    x = rand_bounds(g, 1, 3, 5, H, sw=0.05, sb=1.0, gap_w=0.005, gap_b=0.02)
    x.ub += 0.01
    weight = torch.randn(H, generator=g)
    bias = torch.randn(H, generator=g)
    y = O.layer_norm(x, weight, bias, mode, p, 0.05)

    def true_ln(v):
        c = v - v.mean(-1, keepdim=True)
        if mode == "standard":
            c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + 1e-12)
        return c * weight.double() + bias.double()
    _bounded_between(true_ln, x, y, g, 5, p, 0.05)
    assert O.layer_norm(x, weight, bias, "no", p, 0.05) is x
