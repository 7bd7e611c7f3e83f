"""Independent fp64 restatements used to PIN oracle/bounds_oracle.py
(TEST INFRASTRUCTURE ONLY -- same import rule as bounds_oracle.py).

Everything here is written per neuron from the mathematics (what line bounds
what function on which interval), with plain Python / numpy loops, so that a
slip in the tensorised oracle (a swapped source, a wrong sign, a transposed
index) shows up as a disagreement.  Nothing here shares code with the oracle.
"""
from __future__ import annotations

import math

import numpy as np

TINY = 1e-12   # Bounds.py:27


def qnorm(v: np.ndarray, q: float) -> float:
    v = np.abs(np.asarray(v, dtype=np.float64))
    if math.isinf(q):
        return float(v.max()) if v.size else 0.0
    if q == 1:
        return float(v.sum())
    return float((v ** q).sum() ** (1.0 / q))


def dual(p: float) -> float:
    if p == 1:
        return math.inf
    if math.isinf(p):
        return 1.0
    return p / (p - 1.0)


def interval(lw_col, lb, uw_col, ub, p, eps, words=1):
    """Concrete [l, u] of one neuron from its coefficient columns (Bounds.py:311-326)."""
    q = dual(p)
    n = len(lw_col) // words
    lo, hi = float(lb), float(ub)
    for i in range(words):
        lo -= eps * qnorm(lw_col[i * n:(i + 1) * n], q)
        hi += eps * qnorm(uw_col[i * n:(i + 1) * n], q)
    return lo, hi


def _apply(side, k, x0, y0, lw_col, lb, uw_col, ub):
    """Line k*(v-x0)+y0 applied to a bounded v; returns (w_col, b) (Bounds.py:362-381)."""
    if (side == "lower") == (k > 0):
        w, b = lw_col, lb
    else:
        w, b = uw_col, ub
    return np.asarray(w, dtype=np.float64) * k, (float(b) - x0) * k + y0


def relu_lines(lo, hi):
    """(k, x0, y0) of the lower and the upper line of ReLU on [lo, hi] (Bounds.py:921-963)."""
    if hi < 0:                       # dead: the zero line
        return (0.0, 0.0, 0.0), (0.0, 0.0, 0.0)
    if lo > 0:                       # active: identity
        return (1.0, 0.0, 0.0), (1.0, 0.0, 0.0)
    upper = (hi / (hi - lo + TINY), lo, 0.0)          # chord from (lo, 0) to (hi, hi)
    lower = (1.0 if abs(hi) > abs(lo) else 0.0, 0.0, 0.0)
    return lower, upper


def lines_applied(lower, upper, lw_col, lb, uw_col, ub):
    lw2, lb2 = _apply("lower", *lower, lw_col, lb, uw_col, ub)
    uw2, ub2 = _apply("upper", *upper, lw_col, lb, uw_col, ub)
    return lw2, lb2, uw2, ub2


def relu_neuron(lw_col, lb, uw_col, ub, p, eps, words=1):
    """(lw', lb', uw', ub') of one neuron through ReLU."""
    lo, hi = interval(lw_col, lb, uw_col, ub, p, eps, words)
    return lines_applied(*relu_lines(lo, hi), lw_col, lb, uw_col, ub)


def _sech2(v):
    c = math.cosh(v)
    return 1.0 / (c * c)


def tanh_lines(lo, hi, iters=10):
    """Slopes / anchor points (k, x0, y0) of the lower and upper lines of tanh
    on [lo, hi]  (Bounds.py:1027-1097)."""
    if hi < 0 or lo > 0:
        m = 0.5 * (lo + hi)
        tangent = (_sech2(m), m, math.tanh(m))
        chord = ((math.tanh(hi) - math.tanh(lo)) / (hi - lo + TINY), lo, math.tanh(lo))
        return (tangent, chord) if hi < 0 else (chord, tangent)
    # lower line: tangent at d in [lo, 0] through (hi, tanh hi)
    d, a, b = lo / 2, lo, 0.0
    for _ in range(iters):
        v = (math.tanh(hi) - math.tanh(d)) / (hi - d + TINY) - _sech2(d)
        if v > 0:
            a = d
            d = (d + b) / 2
        else:
            b = d
            d = (d + a) / 2
    lower = ((math.tanh(d) - math.tanh(hi)) / (d - hi + TINY), d, math.tanh(d))
    # upper line: tangent at d in [0, hi] through (lo, tanh lo)
    d, a, b = hi / 2, 0.0, hi
    for _ in range(iters):
        v = (math.tanh(d) - math.tanh(lo)) / (d - lo + TINY) - _sech2(d)
        if v > 0:
            b = d
            d = (d + a) / 2
        else:
            a = d
            d = (d + b) / 2
    upper = ((math.tanh(d) - math.tanh(lo)) / (d - lo + TINY), d, math.tanh(d))
    return lower, upper


def tanh_neuron(lw_col, lb, uw_col, ub, p, eps, words=1, iters=10):
    lo, hi = interval(lw_col, lb, uw_col, ub, p, eps, words)
    return lines_applied(*tanh_lines(lo, hi, iters), lw_col, lb, uw_col, ub)


def _exp_capped(v, thres=12.0):
    return math.exp(v) if v < thres else math.exp(thres) * (v - thres + 1.0)


def exp_neuron(lw_col, lb, uw_col, ub, p, eps, words=1):
    return exp_outputs(*interval(lw_col, lb, uw_col, ub, p, eps, words), lw_col, lb, uw_col, ub)


def exp_outputs(lo, hi, lw_col, lb, uw_col, ub):
    """Bounds.py:970-1003.  Lower: tangent of exp at m = min(mid, lo + 0.99); upper: chord."""
    m = min(0.5 * (lo + hi), lo + 0.99)
    kl = math.exp(min(m, 12.0))
    ku = (_exp_capped(hi) - _exp_capped(lo)) / (hi - lo + TINY)
    lw = np.asarray(lw_col, float) * kl
    uw = np.asarray(uw_col, float) * ku
    return lw, kl * (float(lb) - m + 1.0), uw, float(ub) * ku - ku * lo + _exp_capped(lo)


def reciprocal_neuron(lw_col, lb, uw_col, ub, p, eps, words=1):
    return reciprocal_outputs(*interval(lw_col, lb, uw_col, ub, p, eps, words), lw_col, lb, uw_col, ub)


def reciprocal_outputs(lo, hi, lw_col, lb, uw_col, ub):
    """Bounds.py:1136-1161 for a positive interval.  1/x is convex and decreasing: the tangent at
    the midpoint bounds it from below and takes the UPPER input bound (negative slope), the chord
    bounds it from above and takes the LOWER input bound."""
    m = 0.5 * (lo + hi)
    kl = -1.0 / (m * m)
    ku = -1.0 / (lo * hi)
    return (np.asarray(uw_col, float) * kl, float(ub) * kl + 2.0 / m,
            np.asarray(lw_col, float) * ku, float(lb) * ku - ku * lo + 1.0 / lo)


def sqr_lines(lo, hi):
    """Bounds.py:860-890: (lower, upper) lines of x^2 on [lo, hi]."""
    upper = (hi + lo, lo, lo * lo)                       # chord through (lo, lo^2), (hi, hi^2)
    if hi < 0:
        m = max(0.5 * (lo + hi), 2 * hi)
        lower = (2 * m, m, m * m)
    elif lo > 0:
        m = min(0.5 * (lo + hi), 2 * lo)
        lower = (2 * m, m, m * m)
    else:
        lower = (0.0, 0.0, 0.0)
    return lower, upper


def sqrt_lines(lo, hi):
    """Bounds.py:892-919: chord below, tangent at the midpoint above."""
    m = 0.5 * (lo + hi)
    lower = ((math.sqrt(hi) - math.sqrt(lo)) / (hi - lo + TINY), lo, math.sqrt(lo))
    upper = (0.5 / math.sqrt(m), m, math.sqrt(m))
    return lower, upper


def sqr_neuron(lw_col, lb, uw_col, ub, p, eps, words=1):
    lo, hi = interval(lw_col, lb, uw_col, ub, p, eps, words)
    return lines_applied(*sqr_lines(lo, hi), lw_col, lb, uw_col, ub)


def sqrt_neuron(lw_col, lb, uw_col, ub, p, eps, words=1):
    lo, hi = interval(lw_col, lb, uw_col, ub, p, eps, words)
    return lines_applied(*sqrt_lines(lo, hi), lw_col, lb, uw_col, ub)


def outputs_from_interval(kind, lo, hi, lw_col, lb, uw_col, ub):
    """(lw', lb', uw', ub') of one neuron of relaxation `kind`, given its concrete interval."""
    if kind == "exp":
        return exp_outputs(lo, hi, lw_col, lb, uw_col, ub)
    if kind == "reciprocal":
        return reciprocal_outputs(lo, hi, lw_col, lb, uw_col, ub)
    lines = {"relu": relu_lines, "tanh": tanh_lines, "sqr": sqr_lines, "sqrt": sqrt_lines}[kind]
    return lines_applied(*lines(lo, hi), lw_col, lb, uw_col, ub)


def linear_brute(lw, lb, uw, ub, W, bias=None):
    """Triple-loop sign-split affine map; arrays [L, D, H], [L, H], W [N, H]."""
    L, D, H = lw.shape
    N = W.shape[0]
    lw2 = np.zeros((L, D, N)); uw2 = np.zeros((L, D, N))
    lb2 = np.zeros((L, N)); ub2 = np.zeros((L, N))
    for n in range(N):
        for h in range(H):
            w = float(W[n, h])
            if w > 0:
                lw2[:, :, n] += w * lw[:, :, h]; uw2[:, :, n] += w * uw[:, :, h]
                lb2[:, n] += w * lb[:, h];       ub2[:, n] += w * ub[:, h]
            else:
                lw2[:, :, n] += w * uw[:, :, h]; uw2[:, :, n] += w * lw[:, :, h]
                lb2[:, n] += w * ub[:, h];       ub2[:, n] += w * lb[:, h]
        if bias is not None:
            lb2[:, n] += float(bias[n]); ub2[:, n] += float(bias[n])
    return lw2, lb2, uw2, ub2


def dot_brute(xlw, xlb, xuw, xub, ylw, ylb, yuw, yub, p, eps, words=1):
    """Five-deep loop McCormick bounds for one head.

    x*: [Lx, D, d] / [Lx, d];  y*: [Ly, D, d] / [Ly, d].
    For every scalar product x[i,k]*y[j,k] with x in [lx, ux], y in [ly, uy]:
        lower plane  ly*x + lx*y - lx*ly      (tight at the corner (lx, ly))
        upper plane  uy*x + lx*y - lx*uy      (tight at the corner (lx, uy))
    (Bounds.py:680-688), then each plane is pushed through the linear bounds
    of x and y by the sign of its coefficient.
    """
    Lx, D, d = xlw.shape
    Ly = ylw.shape[0]
    lw = np.zeros((Lx, D, Ly)); uw = np.zeros((Lx, D, Ly))
    lb = np.zeros((Lx, Ly)); ub = np.zeros((Lx, Ly))
    for i in range(Lx):
        for j in range(Ly):
            for k in range(d):
                lx, _ = interval(xlw[i, :, k], xlb[i, k], xuw[i, :, k], xub[i, k], p, eps, words)
                ly, uy = interval(ylw[j, :, k], ylb[j, k], yuw[j, :, k], yub[j, k], p, eps, words)
                # lower plane: coefficient of x is ly, of y is lx
                for (cx, cy, w_out, b_out, lower) in ((ly, lx, lw, lb, True), (uy, lx, uw, ub, False)):
                    b_out[i, j] += -cx * cy
                    if cx != 0:
                        take_low = (cx > 0) == lower
                        b_out[i, j] += cx * (xlb[i, k] if take_low else xub[i, k])
                        for m in range(D):
                            w_out[i, m, j] += cx * (xlw[i, m, k] if take_low else xuw[i, m, k])
                    if cy != 0:
                        take_low = (cy > 0) == lower
                        b_out[i, j] += cy * (ylb[j, k] if take_low else yub[j, k])
                        for m in range(D):
                            w_out[i, m, j] += cy * (ylw[j, m, k] if take_low else yuw[j, m, k])
    return lw, lb, uw, ub


def conv_brute(xl, xu, W, stride, pad):
    """Direct sign-split convolution; xl, xu: [N, C, H, W]; W: [Co, Ci, K, K]."""
    N, C, H, Wd = xl.shape
    Co, Ci, K, _ = W.shape
    Ho = (H + 2 * pad - K) // stride + 1
    Wo = (Wd + 2 * pad - K) // stride + 1
    yl = np.zeros((N, Co, Ho, Wo)); yu = np.zeros((N, Co, Ho, Wo))
    for co in range(Co):
        for ci in range(Ci):
            for kh in range(K):
                for kw in range(K):
                    w = float(W[co, ci, kh, kw])
                    for oh in range(Ho):
                        ih = oh * stride - pad + kh
                        if ih < 0 or ih >= H:
                            continue
                        for ow in range(Wo):
                            iw = ow * stride - pad + kw
                            if iw < 0 or iw >= Wd:
                                continue
                            a, b = xl[:, ci, ih, iw], xu[:, ci, ih, iw]
                            if w > 0:
                                yl[:, co, oh, ow] += w * a; yu[:, co, oh, ow] += w * b
                            else:
                                yl[:, co, oh, ow] += w * b; yu[:, co, oh, ow] += w * a
    return yl, yu
