"""CPU oracle for forward linear-bound propagation (TEST INFRASTRUCTURE ONLY).

This module is a checker.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import it; nothing under faith_amd/ does.

It restates, on CPU torch tensors in fp32 and in the same operation order, the
arithmetic of the reference's PyTorch ``Bounds`` class
(reference: Transformer_Verification_Code/Verifiers/Bounds.py).  Each function
names the reference lines it follows.  Tensor convention (Bounds.py:293-297):

    lw, uw : [B, L, D_in, H]    coefficients of the perturbation
    lb, ub : [B, L, H]          constant terms

A neuron (b, l, j) is bounded by  lw[b,l,:,j] . delta + lb[b,l,j]  from below
and  uw[b,l,:,j] . delta + ub[b,l,j]  from above, for ||delta||_p <= eps.

Parity status of each function (what pins it; tests/test_oracle_*.py, tests/test_reference_vectors.py,
tests/test_bounds_reference_vectors.py):
  Every function below except conv is pinned BY EXECUTION OF THE REFERENCE: tests/golden/
  bounds_reference_vectors.npz holds what the reference's own Bounds class returns
  (Verifiers/Bounds.py run once in the build container by tests/golden/make_bounds_golden.py,
  without its six top-level statements that need tvm and nvcc and with nothing in their place)
  for tanh, relu, exp, sqr, sqrt, reciprocal, multiply, divide, softmax, layer_norm (both
  modes), concretize, dot_product, context, matmul, scalar multiply and add, at p in {1, 2, inf}
  with one and two perturbed words, on inputs with every branch and crafted edge neurons
  (l = 0, u = 0, |u| = |l|, a point, a tiny and a wide interval); tests/golden/
  reference_vectors.npz holds the same for relu, matmul, concretize and dot_product from the
  pure-torch files of HandTunedKernels/python_reference_code.  This module reproduces all of
  them at rtol 1e-5 / atol 1e-6, and mutations of the free choices (nine bisection steps,
  another tangent point for exp, [|u| >= |l|], beta_u = u_x) miss them.  In addition:
  concretize   numpy.linalg.norm, one-hot and zero special cases,
               block-sum identity for perturbed_words > 1.
  linear       brute-force triple loop, W>=0 / lw==uw closed forms,
               (uw'-lw') == (uw-lw)@|W| identity.
  relu         independent fp64 per-neuron closed form
               (oracle/closed_form.py), branch invariants, sampled soundness.
  tanh         independent fp64 scalar loop, odd symmetry, sampled
               soundness, and tangency: the lines touch the curve at the
               point the bisection returns, to the resolution of ten halvings.
  exp, reciprocal, sqr, sqrt
               independent fp64 per-neuron closed forms, sampled soundness
               (lower line <= f <= upper line on [l, u]).
  scale, add   one-line tensor identities (checked against their definition).
  multiply     the brute-force McCormick loop with a reduction of length 1.
  divide, softmax, layer_norm
               compositions of the parts above, in the reference's order; sampled soundness
               (the true softmax / layer norm of any admissible input lies between the
               propagated lines).
  dot_product  brute-force five-deep loop on tiny shapes, einsum
               restatement, sampled soundness of the McCormick planes.
  context      the same function on transposed views; the brute-force loop
               fed with explicitly transposed numpy arrays.
  conv         NOT pinned by execution: the reference has NO Python conv bound; semantics
               come from HandTunedKernels/convolution_verification.cu:124-138
               and its launcher :219-239 (two launches: b with batch 1, w with
               batch = D_in), which needs nvcc.  Pinned by brute-force loops,
               1x1 conv == linear, F.conv2d linearity.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

# Bounds.py:27 -- the guard added to denominators.
EPSILON = 1e-12


def dual_norm(p: float) -> float:
    """q with 1/p + 1/q = 1 (Bounds.py:277)."""
    if p == 1:
        return float("inf")
    if math.isinf(p):
        return 1.0
    return 1.0 / (1.0 - 1.0 / p)


@dataclass
class LinearBounds:
    lw: torch.Tensor
    lb: torch.Tensor
    uw: torch.Tensor
    ub: torch.Tensor

    def tensors(self):
        return self.lw, self.lb, self.uw, self.ub


# --------------------------------------------------------------------------
# concretize  (Bounds.py:311-326)
# --------------------------------------------------------------------------
def concretize(x: LinearBounds, p: float, eps: float, words: int = 1):
    """l = lb - eps * sum_blocks ||lw_block||_q,  u = ub + eps * sum_blocks ||uw_block||_q.

    The norm runs over the D_in axis (dim -2), separately for each of the
    ``words`` equal blocks of D_in, and the per-block terms are added to a
    copy of lb / ub one after the other (Bounds.py:319-326).
    """
    q = dual_norm(p)
    d_in = x.lw.shape[-2]
    blk = d_in // words
    lo = x.lb.clone()
    hi = x.ub.clone()
    for i in range(words):
        sl = slice(blk * i, blk * (i + 1))
        lo += -eps * torch.norm(x.lw[..., sl, :], p=q, dim=-2)
        hi += eps * torch.norm(x.uw[..., sl, :], p=q, dim=-2)
    return lo, hi


# --------------------------------------------------------------------------
# linear / dense  (Bounds.py:397-413 ori_matmul 2-D branch, :383-395 add,
#                  :1016-1025 dense)
# --------------------------------------------------------------------------
def linear(x: LinearBounds, weight: torch.Tensor, bias: torch.Tensor | None = None) -> LinearBounds:
    """Sign-split affine propagation through y = x @ weight.T + bias.

    weight is [H_out, H] (nn.Linear layout).  Eight separately rounded fp32
    products, one add each, bias last.
    """
    wt = weight.t()
    w_pos = wt * torch.gt(wt, 0).to(torch.float32)
    w_neg = wt - w_pos
    lw = x.lw.matmul(w_pos) + x.uw.matmul(w_neg)
    lb = x.lb.matmul(w_pos) + x.ub.matmul(w_neg)
    uw = x.lw.matmul(w_neg) + x.uw.matmul(w_pos)
    ub = x.lb.matmul(w_neg) + x.ub.matmul(w_pos)
    if bias is not None:
        lb = lb + bias
        ub = ub + bias
    return LinearBounds(lw, lb, uw, ub)


# --------------------------------------------------------------------------
# helpers shared by the activation relaxations
#   Bounds.new (Bounds.py:348-360) and Bounds.add_linear (:362-381)
# --------------------------------------------------------------------------
def _fresh(x: LinearBounds, p, eps, words):
    lo, hi = concretize(x, p, eps, words)
    is_pos = torch.gt(lo, 0).to(torch.float32)
    is_neg = torch.lt(hi, 0).to(torch.float32)
    is_both = 1 - is_pos - is_neg
    out = LinearBounds(torch.zeros_like(x.lw), torch.zeros_like(x.lb),
                       torch.zeros_like(x.uw), torch.zeros_like(x.ub))
    return lo, hi, is_pos, is_neg, is_both, out


def _add_line(x: LinearBounds, sel, w_out, b_out, side, k, x0, y0):
    """Accumulate the line  k * (v - x0) + y0  applied to the bound of v.

    For ``side == "lower"`` a positive slope takes the lower source bound and
    a non-positive slope the upper one; mirrored for "upper".  0/1 masks are
    multiplied in first, exactly as the reference does (Bounds.py:376-381).
    """
    if side == "lower":
        w_a, b_a, w_b, b_b = x.lw, x.lb, x.uw, x.ub
    else:
        w_a, b_a, w_b, b_b = x.uw, x.ub, x.lw, x.lb
    sel_w = sel.unsqueeze(2)
    up = torch.gt(k, 0).to(torch.float32)
    w_out += sel_w * up.unsqueeze(2) * w_a * k.unsqueeze(2)
    b_out += sel * up * ((b_a - x0) * k + y0)
    down = 1 - up
    w_out += sel_w * down.unsqueeze(2) * w_b * k.unsqueeze(2)
    b_out += sel * down * ((b_b - x0) * k + y0)


# --------------------------------------------------------------------------
# relu  (Bounds.py:921-963)
# --------------------------------------------------------------------------
def relu(x: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    lo, hi, is_pos, is_neg, is_both, out = _fresh(x, p, eps, words)
    zero = torch.zeros_like(lo)
    one = torch.ones_like(lo)
    # dead neurons: the zero line, both sides
    _add_line(x, is_neg, out.lw, out.lb, "lower", zero, 0, 0)
    _add_line(x, is_neg, out.uw, out.ub, "upper", zero, 0, 0)
    # active neurons: identity, both sides
    _add_line(x, is_pos, out.lw, out.lb, "lower", one, 0, 0)
    _add_line(x, is_pos, out.uw, out.ub, "upper", one, 0, 0)
    # straddling neurons: chord from (l, 0) to (u, u) above ...
    k = hi / (hi - lo + EPSILON)
    _add_line(x, is_both, out.uw, out.ub, "upper", k, lo, 0)
    # ... and slope 0 or 1 below, whichever is tighter
    k = torch.gt(torch.abs(hi), torch.abs(lo)).to(torch.float32)
    _add_line(x, is_both, out.lw, out.lb, "lower", k, 0, 0)
    return out


# --------------------------------------------------------------------------
# tanh  (Bounds.py:1027-1103)
# --------------------------------------------------------------------------
def _dtanh(v):
    return 1.0 / torch.cosh(v).pow(2)


def tanh(x: LinearBounds, p: float, eps: float, words: int = 1, iters: int = 10) -> LinearBounds:
    lo, hi, is_pos, is_neg, is_both, out = _fresh(x, p, eps, words)

    # one-signed neurons: tangent at the midpoint on the convex side,
    # chord on the concave side (Bounds.py:1037-1060)
    mid = (lo + hi) / 2
    k_tan = _dtanh(mid)
    _add_line(x, is_neg, out.lw, out.lb, "lower", k_tan, mid, torch.tanh(mid))
    _add_line(x, is_pos, out.uw, out.ub, "upper", k_tan, mid, torch.tanh(mid))
    k_chord = (torch.tanh(hi) - torch.tanh(lo)) / (hi - lo + EPSILON)
    _add_line(x, is_neg, out.uw, out.ub, "upper", k_chord, lo, torch.tanh(lo))
    _add_line(x, is_pos, out.lw, out.lb, "lower", k_chord, lo, torch.tanh(lo))

    # straddling neurons, lower line: tangent point d in [l, 0] whose tangent
    # passes through (u, tanh u); bisection (Bounds.py:1065-1080)
    d = lo / 2
    left = lo
    right = torch.zeros_like(lo)
    for _ in range(iters):
        v = (torch.tanh(hi) - torch.tanh(d)) / (hi - d + EPSILON) - _dtanh(d)
        go = torch.gt(v, 0).to(torch.float32)
        left = d * go + left * (1 - go)
        right = d * (1 - go) + right * go
        d = (d + right) / 2 * go + (d + left) / 2 * (1 - go)
    k = (torch.tanh(d) - torch.tanh(hi)) / (d - hi + EPSILON)
    _add_line(x, is_both, out.lw, out.lb, "lower", k, d, torch.tanh(d))

    # straddling neurons, upper line: tangent point d in [0, u] whose tangent
    # passes through (l, tanh l) (Bounds.py:1082-1097)
    d = hi / 2
    left = torch.zeros_like(lo)
    right = hi
    for _ in range(iters):
        v = (torch.tanh(d) - torch.tanh(lo)) / (d - lo + EPSILON) - _dtanh(d)
        go = torch.gt(v, 0).to(torch.float32)
        left = d * (1 - go) + left * go
        right = d * go + right * (1 - go)
        d = (d + right) / 2 * (1 - go) + (d + left) / 2 * go
    k = (torch.tanh(d) - torch.tanh(lo)) / (d - lo + EPSILON)
    _add_line(x, is_both, out.uw, out.ub, "upper", k, d, torch.tanh(d))
    return out


# --------------------------------------------------------------------------
# further unary relaxations on the same skeleton
# --------------------------------------------------------------------------
EXP_THRESHOLD = 12.0   # Bounds.py:984


def _exp_capped(v):
    """exp below the threshold, its tangent at the threshold above it (Bounds.py:986-989)."""
    thres = torch.tensor(EXP_THRESHOLD)
    below = torch.lt(v, thres).to(torch.float32)
    return below * torch.exp(torch.min(v, thres)) + (1 - below) * (torch.exp(thres) * (v - thres + 1))


def exp(x: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.exp (Bounds.py:970-1003): tangent below (at min(mid, l + 0.99)), chord above."""
    lo, hi = concretize(x, p, eps, words)
    thres = torch.tensor(EXP_THRESHOLD)
    m = torch.min((lo + hi) / 2, lo + 0.99)
    kl = torch.exp(torch.min(m, thres))
    lw = x.lw * kl.unsqueeze(2)
    lb = kl * (x.lb - m + 1)
    ku = (_exp_capped(hi) - _exp_capped(lo)) / (hi - lo + EPSILON)
    uw = x.uw * ku.unsqueeze(2)
    ub = x.ub * ku - ku * lo + _exp_capped(lo)
    return LinearBounds(lw, lb, uw, ub)


def reciprocal(x: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.reciprocal (Bounds.py:1136-1161); needs l >= 1e-12 everywhere."""
    lo, hi = concretize(x, p, eps, words)
    assert torch.min(lo) >= EPSILON
    m = (lo + hi) / 2
    kl = -1 / m.pow(2)
    lw = x.uw * kl.unsqueeze(2)
    lb = x.ub * kl + 2 / m
    ku = -1.0 / (lo * hi)
    uw = x.lw * ku.unsqueeze(2)
    ub = x.lb * ku - ku * lo + 1 / lo
    return LinearBounds(lw, lb, uw, ub)


def sqr(x: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.sqr (Bounds.py:860-890): chord above; tangent below for one-signed neurons, zero
    for straddling ones."""
    lo, hi, is_pos, is_neg, _is_both, out = _fresh(x, p, eps, words)
    _add_line(x, torch.ones_like(lo), out.uw, out.ub, "upper", hi + lo, lo, lo.pow(2))
    m = torch.max((lo + hi) / 2, 2 * hi)
    _add_line(x, is_neg, out.lw, out.lb, "lower", 2 * m, m, m.pow(2))
    m = torch.min((lo + hi) / 2, 2 * lo)
    _add_line(x, is_pos, out.lw, out.lb, "lower", 2 * m, m, m.pow(2))
    return out


def sqrt(x: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.sqrt (Bounds.py:892-919): chord below, tangent at the midpoint above; needs l > 0."""
    lo, hi, _p, _n, _b, out = _fresh(x, p, eps, words)
    assert torch.min(lo) > 0
    one = torch.ones_like(lo)
    k = (torch.sqrt(hi) - torch.sqrt(lo)) / (hi - lo + EPSILON)
    _add_line(x, one, out.lw, out.lb, "lower", k, lo, torch.sqrt(lo))
    m = (lo + hi) / 2
    k = 0.5 / torch.sqrt(m)
    _add_line(x, one, out.uw, out.ub, "upper", k, m, torch.sqrt(m))
    return out


# --------------------------------------------------------------------------
# elementwise algebra and the composites built from it
# --------------------------------------------------------------------------
def scale(x: LinearBounds, W) -> LinearBounds:
    """Bounds.multiply with a float (Bounds.py:595-607) or a tensor [H] (:653-664)."""
    if isinstance(W, float):
        if W > 0:
            return LinearBounds(x.lw * W, x.lb * W, x.uw * W, x.ub * W)
        return LinearBounds(x.uw * W, x.ub * W, x.lw * W, x.lb * W)
    w_pos = W * torch.gt(W, 0).to(torch.float32)
    w_neg = W - w_pos
    return LinearBounds(x.lw * w_pos + x.uw * w_neg, x.lb * w_pos + x.ub * w_neg,
                        x.lw * w_neg + x.uw * w_pos, x.lb * w_neg + x.ub * w_pos)


def add(x: LinearBounds, delta) -> LinearBounds:
    """Bounds.add (Bounds.py:383-395)."""
    if isinstance(delta, LinearBounds):
        return LinearBounds(x.lw + delta.lw, x.lb + delta.lb, x.uw + delta.uw, x.ub + delta.ub)
    return LinearBounds(x.lw, x.lb + delta, x.uw, x.ub + delta)


def multiply(x: LinearBounds, y: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.multiply with a Bounds argument (Bounds.py:608-651): McCormick planes
    a_l = l_y, a_u = u_y, b = l_x (both sides), pushed through x and y by sign."""
    lx, _ux = concretize(x, p, eps, words)
    ly, uy = concretize(y, p, eps, words)
    out = LinearBounds(torch.zeros_like(x.lw), torch.zeros_like(x.lb), torch.zeros_like(x.uw), torch.zeros_like(x.ub))
    every = torch.ones_like(lx)
    _add_line(x, every, out.lw, out.lb, "lower", ly, 0, -ly * lx)
    _add_line(y, every, out.lw, out.lb, "lower", lx, 0, 0)
    _add_line(x, every, out.uw, out.ub, "upper", uy, 0, -uy * lx)
    _add_line(y, every, out.uw, out.ub, "upper", lx, 0, 0)
    return out


def divide(x: LinearBounds, y: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.divide (Bounds.py:825-830)."""
    return multiply(x, reciprocal(y, p, eps, words), p, eps, words)


def softmax(x: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.softmax (Bounds.py:1005-1014): exp, then division by the (repeated) sum over H."""
    e = exp(x, p, eps, words)
    H = x.lw.shape[-1]
    total = LinearBounds(torch.sum(e.lw, dim=-1, keepdim=True).repeat(1, 1, 1, H),
                         torch.sum(e.lb, dim=-1, keepdim=True).repeat(1, 1, H),
                         torch.sum(e.uw, dim=-1, keepdim=True).repeat(1, 1, 1, H),
                         torch.sum(e.ub, dim=-1, keepdim=True).repeat(1, 1, H))
    return divide(e, total, p, eps, words)


def layer_norm(x: LinearBounds, weight: torch.Tensor, bias: torch.Tensor, mode: str,
               p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.layer_norm (Bounds.py:1111-1131); mode in {"no", "no_var", "standard"}."""
    if mode == "no":
        return x
    H = x.lw.shape[-1]
    w_avg = torch.ones(H, H) * (1.0 / H)
    minus_mu = add(x, scale(linear(x, w_avg), -1.0))
    if mode == "standard":
        variance = linear(sqr(minus_mu, p, eps, words), w_avg)
        normalized = divide(minus_mu, sqrt(add(variance, EPSILON), p, eps, words), p, eps, words)
    else:
        assert mode == "no_var"
        normalized = minus_mu
    return add(scale(normalized, weight), bias)


# --------------------------------------------------------------------------
# dot product  (Bounds.py:666-688 get_bounds_xy, :710-823 ori_dot_product)
# --------------------------------------------------------------------------
def dot_product(x: LinearBounds, y: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """McCormick bounds of z[i, j] = sum_k x[i, k] * y[j, k]  (Q . K^T).

    x: [B, Lx, D, d], y: [B, Ly, D, d]  ->  z: lw, uw [B, Lx, D, Ly], lb, ub [B, Lx, Ly].
    Planes (Bounds.py:680-688):  x*y >= a_l*x + b_l*y - a_l*b_l  with
    a_l = l_y, b_l = l_x, and  x*y <= a_u*x + b_u*y - a_u*b_u  with
    a_u = u_y, b_u = l_x.
    Accumulation order follows Bounds.py:761-818: gamma first, then the
    x-terms (positive part, negative part), then the y-terms.
    """
    B, Lx, D, d = x.lw.shape
    Ly = y.lw.shape[1]
    if D == 1:
        # interval shortcut (Bounds.py:711-721)
        l1, u1 = x.lb.unsqueeze(-2), x.ub.unsqueeze(-2)
        l2, u2 = y.lb.unsqueeze(1), y.ub.unsqueeze(1)
        c1, c2, c3, c4 = l1 * l2, l1 * u2, u1 * l2, u1 * u2
        lo = torch.min(torch.min(c1, c2), torch.min(c3, c4)).sum(-1)
        hi = torch.max(torch.max(c1, c2), torch.max(c3, c4)).sum(-1)
        w = lo.unsqueeze(-2) * 0
        return LinearBounds(w, lo, w, hi)

    l_x, _u_x = concretize(x, p, eps, words)
    l_y, u_y = concretize(y, p, eps, words)
    lw = torch.zeros(B, Lx, D, Ly)
    uw = torch.zeros(B, Lx, D, Ly)
    lb = torch.zeros(B, Lx, Ly)
    ub = torch.zeros(B, Lx, Ly)

    def part(v, cmp):
        return v * cmp(v, 0).to(torch.float32)

    for t in range(B):
        a_l, a_u, b_lu = l_y[t], u_y[t], l_x[t]          # [Ly,d], [Ly,d], [Lx,d]
        # gamma = -alpha * beta, summed over k (Bounds.py:682, 686, 761-762)
        lb[t] += torch.sum(-(a_l.unsqueeze(0) * b_lu.unsqueeze(1)), dim=-1)
        ub[t] += torch.sum(-(a_u.unsqueeze(0) * b_lu.unsqueeze(1)), dim=-1)

        def x_term_w(dst, src, coef, cmp):      # add_w_alpha, Bounds.py:764-770
            dst[t] += src[t].matmul(part(coef, cmp).t())              # [Lx,D,d]@[d,Ly]

        def x_term_b(dst, src, coef, cmp):      # add_b_alpha, Bounds.py:772-778
            dst[t] += src[t].matmul(part(coef, cmp).t())              # [Lx,d]@[d,Ly]

        def y_term_w(dst, src, coef, cmp):      # add_w_beta, Bounds.py:780-787
            dst[t] += src[t].matmul(part(coef, cmp).t()).transpose(0, 2)   # [Ly,D,Lx] -> [Lx,D,Ly]

        def y_term_b(dst, src, coef, cmp):      # add_b_beta, Bounds.py:789-796
            dst[t] += src[t].matmul(part(coef, cmp).t()).transpose(0, 1)   # [Ly,Lx] -> [Lx,Ly]

        x_term_w(lw, x.lw, a_l, torch.gt)
        x_term_w(lw, x.uw, a_l, torch.lt)
        y_term_w(lw, y.lw, b_lu, torch.gt)
        y_term_w(lw, y.uw, b_lu, torch.lt)
        x_term_b(lb, x.lb, a_l, torch.gt)
        x_term_b(lb, x.ub, a_l, torch.lt)
        y_term_b(lb, y.lb, b_lu, torch.gt)
        y_term_b(lb, y.ub, b_lu, torch.lt)

        x_term_w(uw, x.uw, a_u, torch.gt)
        x_term_w(uw, x.lw, a_u, torch.lt)
        y_term_w(uw, y.uw, b_lu, torch.gt)
        y_term_w(uw, y.lw, b_lu, torch.lt)
        x_term_b(ub, x.ub, a_u, torch.gt)
        x_term_b(ub, x.lb, a_u, torch.lt)
        y_term_b(ub, y.ub, b_lu, torch.gt)
        y_term_b(ub, y.lb, b_lu, torch.lt)
    return LinearBounds(lw, lb, uw, ub)


def transpose_bounds(v: LinearBounds) -> LinearBounds:
    """Bounds.t (Bounds.py:335-346): swap the length and the hidden axis (views, no copy)."""
    return LinearBounds(v.lw.transpose(1, 3), v.lb.transpose(1, 2), v.uw.transpose(1, 3), v.ub.transpose(1, 2))


def context(probs: LinearBounds, value: LinearBounds, p: float, eps: float, words: int = 1) -> LinearBounds:
    """Bounds.context (Bounds.py:843-850): z[i, j] = sum_k probs[i, k] * value[k, j].

    probs: lw [B, L, D, L], lb [B, L, L];  value: lw [B, L, D, dim_out], lb [B, L, dim_out]
    -> lw [B, L, D, dim_out], lb [B, L, dim_out].  It is the dot product of probs with the
    transposed value bounds.
    """
    return dot_product(probs, transpose_bounds(value), p, eps, words)


# --------------------------------------------------------------------------
# convolution  (HandTunedKernels/convolution_verification.cu:124-138, :219-239)
# --------------------------------------------------------------------------
def conv2d(x: LinearBounds, weight: torch.Tensor, bias: torch.Tensor | None = None,
           stride: int = 1, padding: int = 0) -> LinearBounds:
    """Sign-split propagation through a 2-D convolution.

    x.lw, x.uw: [1, D_in, C_in, Hh, Ww] (D_in acts as the conv batch, as in the
    reference launcher's second launch), x.lb, x.ub: [1, C_in, Hh, Ww].
    weight: [C_out, C_in, K, K].  A positive tap multiplies the same-side
    bound, a non-positive tap the opposite one.  Bias (not present in the
    reference kernel) is added to lb / ub only.
    """
    w_pos = weight * torch.gt(weight, 0).to(torch.float32)
    w_neg = weight - w_pos

    def cv(t, w):
        return F.conv2d(t, w, None, stride, padding)

    lw_in, uw_in = x.lw[0], x.uw[0]
    lw = (cv(lw_in, w_pos) + cv(uw_in, w_neg)).unsqueeze(0)
    uw = (cv(uw_in, w_pos) + cv(lw_in, w_neg)).unsqueeze(0)
    lb = cv(x.lb, w_pos) + cv(x.ub, w_neg)
    ub = cv(x.ub, w_pos) + cv(x.lb, w_neg)
    if bias is not None:
        lb = lb + bias.view(1, -1, 1, 1)
        ub = ub + bias.view(1, -1, 1, 1)
    return LinearBounds(lw, lb, uw, ub)


def concretize_conv(x: LinearBounds, p: float, eps: float):
    """Concretize conv-shaped bounds: the norm runs over D_in (dim 1 of lw)."""
    q = dual_norm(p)
    lo = x.lb - eps * torch.norm(x.lw, p=q, dim=1)
    hi = x.ub + eps * torch.norm(x.uw, p=q, dim=1)
    return lo, hi


# --------------------------------------------------------------------------
# interval bound propagation  (method "ibp": the `if self.ibp` branches)
# --------------------------------------------------------------------------
def interval_unary(kind: str, l: torch.Tensor, u: torch.Tensor):
    """Image of the concrete interval [l, u] under a monotone operator, and sqr
    (Bounds.py:924-926 relu, :1030-1032 tanh, :973-975 exp, :1139-1143 reciprocal,
    :896-898 sqrt, :863-866 sqr).  Coefficients are zero in this mode."""
    if kind == "relu":
        zero = torch.tensor(0.0)
        return torch.max(l, zero), torch.max(u, zero)
    if kind == "tanh":
        return torch.tanh(l), torch.tanh(u)
    if kind == "exp":
        return torch.exp(l), torch.exp(u)
    if kind == "reciprocal":
        return 1.0 / u, 1.0 / l
    if kind == "sqrt":
        return torch.sqrt(l), torch.sqrt(u)
    if kind == "sqr":
        both = 1 - torch.gt(l, 0).to(torch.float32) - torch.lt(u, 0).to(torch.float32)
        lb = torch.min(l * l, u * u)
        lb = lb - both * lb                      # the lower bound is zero when the interval holds zero
        return lb, torch.max(l * l, u * u)
    raise ValueError(kind)


def interval_product(xl, xu, yl, yu):
    """Interval of x * y from the four corner products (get_bounds_xy, Bounds.py:667-676)."""
    p1, p2, p3, p4 = xl * yl, xl * yu, xu * yl, xu * yu
    return (torch.min(p1, torch.min(p2, torch.min(p3, p4))), torch.max(p1, torch.max(p2, torch.max(p3, p4))))
