"""Tensor-level wrappers over the C ABI.

Each function checks device / dtype / contiguity / shape on the host, allocates
the outputs with torch (device memory plumbing only) and passes raw pointers
plus the current HIP stream to libfaith_amd.so.  No arithmetic happens here.
"""
from __future__ import annotations

import math
import struct

import torch

from . import _lib, autotune
from ._lib import LAYOUT_NATURAL, LAYOUT_TRANSPOSED, Q_1, Q_2, Q_INF  # noqa: F401


def q_code(p: float) -> int:
    """Dual-norm selector for perturbation norm p (q = 1 / (1 - 1/p))."""
    if p == 1:
        return Q_INF
    if p == 2:
        return Q_2
    if math.isinf(p) or p >= 10:      # the reference treats p >= 10 as infinity
        return Q_1
    if p > 1:
        # any other norm: the bits of the dual exponent travel in the int argument
        return struct.unpack("i", struct.pack("f", 1.0 / (1.0 - 1.0 / p)))[0]
    raise ValueError(f"p={p}: the perturbation norm must be >= 1")


_F32 = torch.float32


def _check(name, t, shape=None):
    # one expression for the tensor that is fine (a small launch is bound by its host side); the
    # detailed tests below only run to name what is wrong
    try:
        if t.is_cuda and t.dtype is _F32 and t.is_contiguous() and (shape is None or t.shape == shape):
            return t
    except AttributeError:
        pass
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name}: expected a tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise ValueError(f"{name}: must live on the GPU (got {t.device}); there is no CPU path")
    if t.dtype != torch.float32:
        raise TypeError(f"{name}: must be float32, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name}: must be contiguous")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise ValueError(f"{name}: expected shape {tuple(shape)}, got {tuple(t.shape)}")
    return t


def _ptr(t):
    return None if t is None else t.data_ptr()


def _stream(t):
    # the raw handle of torch's current stream on the tensor's device; the public
    # torch.cuda.current_stream() builds a Stream object on every call (about 4 us)
    idx = t.device.index
    return torch._C._cuda_getCurrentRawStream(torch.cuda.current_device() if idx is None else idx)


# ------------------------------------------------------------------------------------------
# Result buffers.  By default every call allocates its results (torch's caching allocator).  The reference
# has the caller own all results and scratch (Bounds.py:1270-1277); a caller that runs the same sequence of
# operators again and again -- one propagation per bisection step, per position, per sentence -- can do the
# same here with a Workspace: inside `with ops.workspace(ws):` the i-th result buffer requested during the
# pass is the i-th buffer the workspace holds (allocated on the first pass, reused when shape and device
# match), so a repeated pass allocates nothing.  What a pass returned is overwritten by the next one.
# ------------------------------------------------------------------------------------------
class Workspace:
    """Persistent result and scratch buffers of one repeated sequence of operator calls."""

    def __init__(self):
        self.buffers = []
        self.cursor = 0
        self.allocations = 0

    def reset(self):
        self.cursor = 0

    def take(self, shape, device):
        i = self.cursor
        self.cursor += 1
        if i < len(self.buffers):
            t = self.buffers[i]
            if t.shape == shape and t.device == device:
                return t
        t = torch.empty(shape, device=device, dtype=torch.float32)
        self.allocations += 1
        if i < len(self.buffers):
            self.buffers[i] = t
        else:
            self.buffers.append(t)
        return t

    def bytes(self):
        return sum(t.numel() * 4 for t in self.buffers)

    def scope(self):
        """Context manager: the operator calls inside take their buffers from this workspace, from its start."""
        return workspace(self)


_WORKSPACE = None


class workspace:
    """Context manager: result buffers of the calls inside come from `ws`, in call order, from its start."""

    def __init__(self, ws):
        self.ws = ws

    def __enter__(self):
        global _WORKSPACE
        self.previous = _WORKSPACE
        if self.ws is not None:
            self.ws.reset()
        _WORKSPACE = self.ws
        return self.ws

    def __exit__(self, *exc):
        global _WORKSPACE
        _WORKSPACE = self.previous
        return False


def _empty(*shape, device):
    if _WORKSPACE is not None:
        return _WORKSPACE.take(torch.Size(shape), device)
    return torch.empty(shape, device=device, dtype=torch.float32)


def _empty_like(t):
    if _WORKSPACE is not None:
        return _WORKSPACE.take(t.shape, t.device)
    return torch.empty_like(t)


class _NoGuard:
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


class _Tuned:
    """Device guard plus the tuning-table entry of this (operator, shape), set for the one launch."""

    def __init__(self, guard, knobs):
        self.guard, self.knobs = guard, knobs

    def __enter__(self):
        self.guard.__enter__()
        for k, v in self.knobs.items():
            _lib.call("faith_tune_set", k, v)
        return self

    def __exit__(self, *exc):
        for k in self.knobs:
            _lib.call("faith_tune_set", k, 0)
        return self.guard.__exit__(*exc)


def _on(device, op=None, shape=None):
    """Device guard for the launch; free when the tensor already lives on the current device.
    With a tuning table in use (autotune.use) the entry for (op, shape) is applied around the launch."""
    if device.index is None or device.index == torch.cuda.current_device():
        guard = _NO_GUARD
    else:
        guard = torch.cuda.device(device)
    if op is not None and autotune._ACTIVE is not None:
        knobs = autotune._ACTIVE.lookup(op, shape)
        if knobs:
            return _Tuned(guard, knobs)
    return guard


def _wb_shapes(lw, lb, layout):
    if lw.dim() != 4 or lb.dim() != 3:
        raise ValueError(f"lw must be 4-D and lb 3-D, got {tuple(lw.shape)} and {tuple(lb.shape)}")
    B, L = lw.shape[0], lw.shape[1]
    if layout == LAYOUT_NATURAL:
        D, H = lw.shape[2], lw.shape[3]
    else:
        H, D = lw.shape[2], lw.shape[3]
    if tuple(lb.shape) != (B, L, H):
        raise ValueError(f"lb shape {tuple(lb.shape)} does not match lw shape {tuple(lw.shape)}")
    return B, L, D, H


def concretize(lw, lb, uw, ub, p, eps, words=1, layout=LAYOUT_NATURAL):
    """Concrete interval [l, u] of every neuron.  Shapes as Bounds.concretize."""
    B, L, D, H = _wb_shapes(lw, lb, layout)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    l = _empty_like(lb)
    u = _empty_like(ub)
    with _on(lw.device, "concretize", (B * L, D, H)):
        _lib.call("faith_concretize", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(l), _ptr(u),
                  B * L, D, H, float(eps), q_code(p), int(words), layout, _stream(lw))
    return l, u


_UNARY = {"relu": _lib.OP_RELU, "tanh": _lib.OP_TANH, "exp": _lib.OP_EXP, "reciprocal": _lib.OP_RECIPROCAL,
          "sqr": _lib.OP_SQR, "sqrt": _lib.OP_SQRT}


def _activation(entry, lw, lb, uw, ub, p, eps, words, layout, return_interval, out=None):
    B, L, D, H = _wb_shapes(lw, lb, layout)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    if out is None:
        olw, olb, ouw, oub = (_empty_like(lw), _empty_like(lb),
                              _empty_like(uw), _empty_like(ub))
    else:
        olw, olb, ouw, oub = out
        _check("out lw", olw, lw.shape); _check("out uw", ouw, lw.shape)
        _check("out lb", olb, lb.shape); _check("out ub", oub, lb.shape)
    l = _empty_like(lb) if return_interval else None
    u = _empty_like(ub) if return_interval else None
    with _on(lw.device, "act", (B * L, D, H)):
        if entry in _UNARY:
            _lib.call("faith_unary_verification", _UNARY[entry], _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(olb),
                      _ptr(oub), _ptr(olw), _ptr(ouw), _ptr(l), _ptr(u), B * L, D, H, float(eps), q_code(p),
                      int(words), layout, _stream(lw))
        else:
            _lib.call(entry, _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw),
                      _ptr(l), _ptr(u), B * L, D, H, float(eps), q_code(p), int(words), layout, _stream(lw))
    if return_interval:
        return olw, olb, ouw, oub, l, u
    return olw, olb, ouw, oub


def relu(lw, lb, uw, ub, p, eps, words=1, layout=LAYOUT_NATURAL, return_interval=False, out=None):
    """ReLU relaxation; returns (lw', lb', uw', ub'[, l, u])."""
    return _activation("faith_relu_verification", lw, lb, uw, ub, p, eps, words, layout, return_interval, out)


def tanh(lw, lb, uw, ub, p, eps, words=1, layout=LAYOUT_NATURAL, return_interval=False, out=None):
    """tanh relaxation; returns (lw', lb', uw', ub'[, l, u])."""
    return _activation("faith_tanh_verification", lw, lb, uw, ub, p, eps, words, layout, return_interval, out)


def exp(lw, lb, uw, ub, p, eps, words=1, layout=LAYOUT_NATURAL, return_interval=False, out=None):
    """exp relaxation (tangent below, chord above, capped at 12 as in the reference)."""
    return _activation("exp", lw, lb, uw, ub, p, eps, words, layout, return_interval, out)


def reciprocal(lw, lb, uw, ub, p, eps, words=1, layout=LAYOUT_NATURAL, return_interval=False, out=None):
    """1/x relaxation; the concrete lower bound must be positive."""
    return _activation("reciprocal", lw, lb, uw, ub, p, eps, words, layout, return_interval, out)


def sqr(lw, lb, uw, ub, p, eps, words=1, layout=LAYOUT_NATURAL, return_interval=False, out=None):
    """x^2 relaxation."""
    return _activation("sqr", lw, lb, uw, ub, p, eps, words, layout, return_interval, out)


def sqrt(lw, lb, uw, ub, p, eps, words=1, layout=LAYOUT_NATURAL, return_interval=False, out=None):
    """sqrt relaxation; the concrete lower bound must be positive."""
    return _activation("sqrt", lw, lb, uw, ub, p, eps, words, layout, return_interval, out)


def multiply(x, y, p, eps, words=1, out=None):
    """Product of two bound objects of one shape; x, y: (lw, lb, uw, ub)."""
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    B, L, D, H = _wb_shapes(xlw, xlb, LAYOUT_NATURAL)
    for n, t, s_ in (("x.lw", xlw, None), ("x.uw", xuw, xlw.shape), ("x.lb", xlb, None), ("x.ub", xub, xlb.shape),
                     ("y.lw", ylw, xlw.shape), ("y.uw", yuw, xlw.shape), ("y.lb", ylb, xlb.shape),
                     ("y.ub", yub, xlb.shape)):
        _check(n, t, s_)
    if out is None:
        out = (_empty_like(xlw), _empty_like(xlb), _empty_like(xlw), _empty_like(xlb))
    zlw, zlb, zuw, zub = out
    _check("out lw", zlw, xlw.shape); _check("out uw", zuw, xlw.shape)
    _check("out lb", zlb, xlb.shape); _check("out ub", zub, xlb.shape)
    with _on(xlw.device):
        _lib.call("faith_multiply_verification", _ptr(xlb), _ptr(xub), _ptr(xlw), _ptr(xuw), _ptr(ylb), _ptr(yub),
                  _ptr(ylw), _ptr(yuw), _ptr(zlb), _ptr(zub), _ptr(zlw), _ptr(zuw), B * L, D, H, float(eps),
                  q_code(p), int(words), _stream(xlw))
    return zlw, zlb, zuw, zub


def _object(lw, lb, uw, ub, what="x"):
    """Checks the four tensors of one bound object; returns (rows_w, rows_b, H)."""
    _check(f"{what}.lw", lw); _check(f"{what}.uw", uw, lw.shape); _check(f"{what}.lb", lb); _check(f"{what}.ub", ub, lb.shape)
    H = lw.shape[-1]
    if lb.shape[-1] != H:
        raise ValueError(f"{what}: lw {tuple(lw.shape)} and lb {tuple(lb.shape)} disagree in the last axis")
    return lw.numel() // H, lb.numel() // H, H


def affine(x, scale=None, other=None, shift=None):
    """Bounds.multiply by a float or a per-neuron tensor, Bounds.add with another object and / or a
    per-neuron tensor (which moves the constant terms only) -- any combination, one launch.
    x, other: (lw, lb, uw, ub)."""
    lw, lb, uw, ub = x
    rows_w, rows_b, H = _object(lw, lb, uw, ub)
    vec, scalar = None, 1.0
    if isinstance(scale, torch.Tensor):
        _check("scale", scale, (H,))
        vec = scale
    elif scale is not None:
        scalar = float(scale)
    if other is not None:
        _check("other.lw", other[0], lw.shape); _check("other.uw", other[2], lw.shape)
        _check("other.lb", other[1], lb.shape); _check("other.ub", other[3], lb.shape)
        alw, alb, auw, aub = other
    else:
        alw = alb = auw = aub = None
    if shift is not None:
        if not isinstance(shift, torch.Tensor):
            shift = torch.full((H,), float(shift), device=lb.device, dtype=torch.float32)
        _check("shift", shift, (H,))
    olb, oub = _empty_like(lb), _empty_like(ub)
    if scale is None and other is None:
        # a shift moves the constant terms only: the coefficient tensors are shared, as in the reference
        olw, ouw, rows_w = lw, uw, 0
    else:
        olw, ouw = _empty_like(lw), _empty_like(uw)
    with _on(lw.device):
        _lib.call("faith_affine_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(vec), scalar,
                  _ptr(alb), _ptr(aub), _ptr(alw), _ptr(auw), _ptr(shift), _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw),
                  rows_w, rows_b, H, _stream(lw))
    return olw, olb, ouw, oub


def scale(lw, lb, uw, ub, W):
    """Bounds.multiply with a float or a per-neuron tensor W [H] (sign-split elementwise scaling)."""
    return affine((lw, lb, uw, ub), scale=W)


def add(x, y):
    """Bounds.add with a Bounds argument: elementwise sum of two objects."""
    return affine(x, other=y)


def shift(lw, lb, uw, ub, delta):
    """Bounds.add with a float or a tensor [H]: moves the constant terms only."""
    return affine((lw, lb, uw, ub), shift=delta)


def rowsum(lw, lb, uw, ub):
    """Sum over the last axis, written to every position of that axis, for all four tensors
    (the sum / repeat pair of Bounds.softmax)."""
    rows_w, rows_b, H = _object(lw, lb, uw, ub)
    olw, olb, ouw, oub = _empty_like(lw), _empty_like(lb), _empty_like(uw), _empty_like(ub)
    with _on(lw.device):
        _lib.call("faith_rowsum_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(olb), _ptr(oub), _ptr(olw),
                  _ptr(ouw), rows_w, rows_b, H, _stream(lw))
    return olw, olb, ouw, oub


def rowmean(lw, lb, uw, ub):
    """Mean over the last axis, written to every position of that axis: matmul with the H x H matrix of 1 / H."""
    rows_w, rows_b, H = _object(lw, lb, uw, ub)
    olw, olb, ouw, oub = _empty_like(lw), _empty_like(lb), _empty_like(uw), _empty_like(ub)
    with _on(lw.device):
        _lib.call("faith_rowmean_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(olb), _ptr(oub), _ptr(olw),
                  _ptr(ouw), rows_w, rows_b, H, _stream(lw))
    return olw, olb, ouw, oub


def layer_norm(lw, lb, uw, ub, weight=None, bias=None, other=None):
    """Mean subtraction along the last axis, then per-neuron weight (split by sign) and bias:
    Bounds.layer_norm in mode "no_var"; with weight = bias = None its first step in mode "standard".
    other: (lw, lb, uw, ub) of a second object added first (the residual connection), same launch."""
    rows_w, rows_b, H = _object(lw, lb, uw, ub)
    if weight is not None:
        _check("weight", weight, (H,))
    if bias is not None:
        _check("bias", bias, (H,))
    if other is not None:
        _check("other.lw", other[0], lw.shape); _check("other.uw", other[2], lw.shape)
        _check("other.lb", other[1], lb.shape); _check("other.ub", other[3], lb.shape)
        alw, alb, auw, aub = other
    else:
        alw = alb = auw = aub = None
    olw, olb, ouw, oub = _empty_like(lw), _empty_like(lb), _empty_like(uw), _empty_like(ub)
    with _on(lw.device):
        _lib.call("faith_layer_norm_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(alb), _ptr(aub),
                  _ptr(alw), _ptr(auw), _ptr(weight), _ptr(bias), _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw),
                  rows_w, rows_b, H, _stream(lw))
    return olw, olb, ouw, oub


def spread_positions(t, positions, length):
    """[B, P, ...] -> [B, length, ...]: row positions[b, i] of batch element b holds t[b, i], every other row
    is zero (a position outside 0 ... length-1 names no row).  positions: int64 [B, P] on t's device, distinct
    within a batch element.  One launch that writes the whole result; nothing is computed and nothing waits for
    the device."""
    _check("t", t)
    B, P = positions.shape
    if t.shape[:2] != (B, P):
        raise ValueError(f"t {tuple(t.shape)} does not start with positions' shape {(B, P)}")
    if not (positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous()):
        raise ValueError("positions: expected a contiguous int64 GPU tensor")
    out = _empty(B, length, *t.shape[2:], device=t.device)
    with _on(t.device):
        _lib.call("faith_rows_spread", _ptr(t), _ptr(positions), _ptr(out), B, length, P, t.numel() // (B * P), _stream(t))
    return out


def zeros(*shape, device):
    """A result buffer (the caller's persistent one inside a workspace scope) filled with zeros."""
    return _empty(*shape, device=device).zero_()


def softmax_fits(dim_in, dim_out):
    """True if softmax() takes a [dim_in, dim_out] slab in one launch (16-byte aligned tensors assumed)."""
    return bool(_lib.lib.faith_softmax_fits(int(dim_in), int(dim_out)))


def softmax(lw, lb, uw, ub, p, eps, words=1, return_sum_bound=False, scale=1.0):
    """Bounds.softmax over the last axis in one launch: exp, sum, reciprocal and product on a slab that stays
    in registers.  Returns (lw', lb', uw', ub'[, l_sum]); l_sum [B, L] is the concrete lower bound of the sum,
    which must be >= 1e-12 for the result to mean anything (the reference asserts it).  scale > 0 multiplies
    the object first (Bounds.multiply with a float), in the same launch.  Raises FaithError
    (FAITH_ERR_UNSUPPORTED) when the slab does not fit: see softmax_fits."""
    B, L, D, H = _wb_shapes(lw, lb, LAYOUT_NATURAL)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    olw, olb, ouw, oub = _empty_like(lw), _empty_like(lb), _empty_like(uw), _empty_like(ub)
    l_sum = _empty(B, L, device=lw.device) if return_sum_bound else None
    with _on(lw.device):
        _lib.call("faith_softmax_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(olb), _ptr(oub),
                  _ptr(olw), _ptr(ouw), _ptr(l_sum), float(scale), B * L, D, H, float(eps), q_code(p), int(words),
                  _stream(lw))
    if return_sum_bound:
        return olw, olb, ouw, oub, l_sum
    return olw, olb, ouw, oub


def interval_unary(kind, l, u):
    """Interval bound propagation through relu / tanh / exp / reciprocal / sqr / sqrt: the interval of the
    image of [l, u], elementwise.  Returns (lb, ub)."""
    if kind not in _UNARY:
        raise ValueError(f"unknown operator {kind!r}")
    _check("l", l); _check("u", u, l.shape)
    olb, oub = _empty_like(l), _empty_like(u)
    with _on(l.device):
        _lib.call("faith_interval_unary", _UNARY[kind], _ptr(l), _ptr(u), _ptr(olb), _ptr(oub), l.numel(), _stream(l))
    return olb, oub


def interval_product(xl, xu, yl, yu):
    """Interval of the elementwise product of [xl, xu] and [yl, yu].  Returns (lb, ub)."""
    _check("xl", xl); _check("xu", xu, xl.shape); _check("yl", yl, xl.shape); _check("yu", yu, xl.shape)
    zl, zu = _empty_like(xl), _empty_like(xl)
    with _on(xl.device):
        _lib.call("faith_interval_product", _ptr(xl), _ptr(xu), _ptr(yl), _ptr(yu), _ptr(zl), _ptr(zu), xl.numel(),
                  _stream(xl))
    return zl, zu


def linear(lw, lb, uw, ub, weight, bias=None, out=None):
    """Sign-split propagation through y = x @ weight.T + bias.  weight: [H_out, H]."""
    B, L, D, H = _wb_shapes(lw, lb, LAYOUT_NATURAL)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    _check("weight", weight)
    if weight.dim() != 2 or weight.shape[1] != H:
        raise ValueError(f"weight must be [H_out, {H}], got {tuple(weight.shape)}")
    N = weight.shape[0]
    if bias is not None:
        _check("bias", bias, (N,))
    if out is None:
        olw = _empty(B, L, D, N, device=lw.device)
        ouw = _empty_like(olw)
        olb = _empty(B, L, N, device=lw.device)
        oub = _empty_like(olb)
    else:
        olw, olb, ouw, oub = out
        _check("out lw", olw, (B, L, D, N)); _check("out uw", ouw, (B, L, D, N))
        _check("out lb", olb, (B, L, N)); _check("out ub", oub, (B, L, N))
    if autotune._ACTIVE is not None:
        generated = autotune._ACTIVE.generated("linear", (B * L * D, H, N))
        if generated is not None:
            # a variant compiled by the tuner for this shape takes the coefficient rows; the constant rows stay with
            # the library's exact-accumulation kernel
            with _on(lw.device):
                autotune.load_generated(generated).coefficients(lw, uw, weight, olw, ouw, _stream(lw))
                _lib.call("faith_matmul_rows_verification", _ptr(lb), _ptr(ub), None, None, _ptr(weight), _ptr(bias),
                          _ptr(olb), _ptr(oub), None, None, 0, B * L, H, N, _stream(lw))
            return olw, olb, ouw, oub
    with _on(lw.device, "linear", (B * L * D, H, weight.shape[0])):
        _lib.call("faith_matmul_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(weight), _ptr(bias),
                  _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw), B, L, D, H, N, _stream(lw))
    return olw, olb, ouw, oub


def linear_relu_fits(rows, D, H, N, words=1):
    """Whether linear_relu takes a layer [N, H] on objects of `rows` = batch * length positions with dim_in D:
    0 no, 1 yes but the separate launches are faster, 2 yes and it is the faster choice."""
    return int(_lib.lib.faith_matmul_relu_fits(rows, D, H, N, words))


def linear_relu(lw, lb, uw, ub, weight, bias, p, eps, words=1):
    """relu(linear(x)) in one pass over the coefficients (`dense(x).relu()`); returns (lw', lb', uw', ub').
    Raises FaithError (ERR_UNSUPPORTED) for shapes linear_relu_fits refuses."""
    B, L, D, H = _wb_shapes(lw, lb, LAYOUT_NATURAL)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    _check("weight", weight)
    if weight.dim() != 2 or weight.shape[1] != H:
        raise ValueError(f"weight must be [H_out, {H}], got {tuple(weight.shape)}")
    N = weight.shape[0]
    if bias is not None:
        _check("bias", bias, (N,))
    olw = _empty(B, L, D, N, device=lw.device)
    ouw = _empty_like(olw)
    olb = _empty(B, L, N, device=lw.device)
    oub = _empty_like(olb)
    with _on(lw.device):
        _lib.call("faith_matmul_relu_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(weight), _ptr(bias),
                  _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw), B, L, D, H, N, float(eps), q_code(p), int(words), _stream(lw))
    return olw, olb, ouw, oub


def linear_layer_norm_fits(rows, D, H, N, res_words=0):
    """Whether linear_layer_norm takes a layer [N, H] on objects of `rows` = batch * length positions with dim_in D
    (res_words > 0: the added object holds that many positions per batch element only): 0 no, 1 yes but the
    separate launches are faster (too few tiles to fill the device), 2 yes and it is the faster choice."""
    return int(_lib.lib.faith_matmul_layer_norm_fits(rows, D, H, N, res_words))


def linear_layer_norm(lw, lb, uw, ub, weight, bias, norm_weight=None, norm_bias=None, other=None, positions=None):
    """layer_norm(linear(x) + other) without the variance, one pass over the coefficients
    (`dense(x).add(other).layer_norm(normalizer, "no_var")`).  other: (lw, lb, uw, ub) of the added object; with
    `positions` (int64 [B, P] on the device) its coefficients are [B, P, D, N], the rows of those positions only.
    Raises FaithError (ERR_UNSUPPORTED) for shapes linear_layer_norm_fits refuses."""
    B, L, D, H = _wb_shapes(lw, lb, LAYOUT_NATURAL)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    _check("weight", weight)
    if weight.dim() != 2 or weight.shape[1] != H:
        raise ValueError(f"weight must be [H_out, {H}], got {tuple(weight.shape)}")
    N = weight.shape[0]
    if bias is not None:
        _check("bias", bias, (N,))
    if norm_weight is not None:
        _check("norm_weight", norm_weight, (N,))
    if norm_bias is not None:
        _check("norm_bias", norm_bias, (N,))
    words = 0
    if other is not None:
        alw, alb, auw, aub = other
        if positions is not None:
            if positions.dtype != torch.int64 or not positions.is_cuda or not positions.is_contiguous() or \
                    positions.dim() != 2 or positions.shape[0] != B:
                raise ValueError(f"positions must be a contiguous int64 [{B}, P] tensor on the device")
            words = positions.shape[1]
            _check("other.lw", alw, (B, words, D, N)); _check("other.uw", auw, (B, words, D, N))
        else:
            _check("other.lw", alw, (B, L, D, N)); _check("other.uw", auw, (B, L, D, N))
        _check("other.lb", alb, (B, L, N)); _check("other.ub", aub, (B, L, N))
    else:
        if positions is not None:
            raise ValueError("positions without an added object")
        alw = alb = auw = aub = None
    olw = _empty(B, L, D, N, device=lw.device)
    ouw = _empty_like(olw)
    olb = _empty(B, L, N, device=lw.device)
    oub = _empty_like(olb)
    with _on(lw.device):
        _lib.call("faith_matmul_layer_norm_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(weight), _ptr(bias),
                  _ptr(alb), _ptr(aub), _ptr(alw), _ptr(auw), _ptr(positions), words, _ptr(norm_weight), _ptr(norm_bias),
                  _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw), B, L, D, H, N, _stream(lw))
    return olw, olb, ouw, oub


def linear_concretize(lw, lb, uw, ub, weight, bias, p, eps, words=1, out=None):
    """linear() and concretize() of its result through one entry point (one launch for small problems).
    Returns (lw', lb', uw', ub', l, u).  `out`: the six result tensors, owned by the caller as in the
    reference's interface (Bounds.py:1270-1277); a small layer is bound by its host side, and six
    allocations are a third of it."""
    B, L, D, H = _wb_shapes(lw, lb, LAYOUT_NATURAL)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    _check("weight", weight)
    if weight.dim() != 2 or weight.shape[1] != H:
        raise ValueError(f"weight must be [H_out, {H}], got {tuple(weight.shape)}")
    N = weight.shape[0]
    if bias is not None:
        _check("bias", bias, (N,))
    if out is None:
        olw = _empty(B, L, D, N, device=lw.device)
        ouw = _empty_like(olw)
        olb = _empty(B, L, N, device=lw.device)
        oub = _empty_like(olb)
        l = _empty_like(olb)
        u = _empty_like(olb)
    else:
        olw, olb, ouw, oub, l, u = out
        _check("out lw", olw, (B, L, D, N)); _check("out uw", ouw, (B, L, D, N))
        for name, t in (("out lb", olb), ("out ub", oub), ("out l", l), ("out u", u)):
            _check(name, t, (B, L, N))
    with _on(lw.device, "linear", (B * L * D, H, N)):
        _lib.call("faith_matmul_concretize_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(weight),
                  _ptr(bias), _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw), _ptr(l), _ptr(u), B, L, D, H, N,
                  float(eps), q_code(p), int(words), _stream(lw))
    return olw, olb, ouw, oub, l, u


class BoundCall:
    """An entry point with its arguments converted once: calling the object launches again with the same device
    pointers, sizes and stream -- for a caller that repeats one small launch (a bisection step on the same
    buffers), where shape checks, twelve data_ptr() calls and the stream lookup are most of the host time.  The
    tensors are kept alive by the object; their contents may change between calls, their addresses must not."""

    __slots__ = ("name", "results", "_fn", "_args", "_keep")

    def __init__(self, name, args, keep, results):
        self.name, self.results = name, results
        self._fn = _lib._ENTRY[name]
        self._args = tuple(args)
        self._keep = keep

    def __call__(self, stream=None):
        """stream: a raw HIP stream handle (e.g. torch.cuda.current_stream().cuda_stream) to launch on instead of
        the stream that was current when the call was bound -- a bound call does not follow torch's stream
        context by itself (looking it up is part of what binding saves)."""
        rc = self._fn(*self._args) if stream is None else self._fn(*self._args[:-1], stream)
        if rc:
            raise _lib.FaithError(self.name, rc, _lib.lib.faith_last_error().decode())
        return self.results


def bind_linear_concretize(lw, lb, uw, ub, weight, bias, p, eps, words=1, out=None):
    """linear_concretize() as a BoundCall on torch's current stream: the checks run here, once; every call of the
    returned object is one trip through the C ABI into the same six result tensors (`.results`)."""
    results = linear_concretize(lw, lb, uw, ub, weight, bias, p, eps, words, out=out)      # checks, and a first launch
    olw, olb, ouw, oub, l, u = results
    B, L, D, H = _wb_shapes(lw, lb, LAYOUT_NATURAL)
    args = (_ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(weight), _ptr(bias), _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw),
            _ptr(l), _ptr(u), B, L, D, H, weight.shape[0], float(eps), q_code(p), int(words), _stream(lw))
    return BoundCall("faith_matmul_concretize_verification", args, (lw, lb, uw, ub, weight, bias) + tuple(results), results)


def linear_group(lw, lb, uw, ub, weights, biases=None):
    """Several affine layers of one shape on the same bound object (query, key, value of an attention block):
    one launch where that pays, the same results as linear() per layer.  weights: list of [H_out, H];
    biases: list of [H_out] or None entries, or None.  Returns a list of (lw', lb', uw', ub')."""
    import ctypes
    B, L, D, H = _wb_shapes(lw, lb, LAYOUT_NATURAL)
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    n = len(weights)
    if not 1 <= n <= 3:
        raise ValueError(f"{n} layers: between one and three share a launch")
    N = weights[0].shape[0]
    biases = list(biases) if biases is not None else [None] * n
    for i, (W, b) in enumerate(zip(weights, biases)):
        _check(f"weight {i}", W, (N, H))
        if b is not None:
            _check(f"bias {i}", b, (N,))
    outs = [(_empty(B, L, D, N, device=lw.device),
             _empty(B, L, N, device=lw.device),
             _empty(B, L, D, N, device=lw.device),
             _empty(B, L, N, device=lw.device)) for _ in range(n)]
    arr = ctypes.c_void_p * n
    ptrs = lambda ts: arr(*[_ptr(t) for t in ts])
    a_w, a_b = ptrs(weights), ptrs(biases)
    a_lb, a_ub = ptrs([o[1] for o in outs]), ptrs([o[3] for o in outs])
    a_lw, a_uw = ptrs([o[0] for o in outs]), ptrs([o[2] for o in outs])
    with _on(lw.device):
        _lib.call("faith_matmul_group_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), n,
                  ctypes.addressof(a_w), ctypes.addressof(a_b), ctypes.addressof(a_lb), ctypes.addressof(a_ub),
                  ctypes.addressof(a_lw), ctypes.addressof(a_uw), B, L, D, H, N, _stream(lw))
    return outs


def linear_rows(lw, lb, uw, ub, weights, biases=None):
    """linear() / linear_group() for an object whose coefficient rows and constant rows are counted separately:
    lw, uw [..., H] (any leading axes) and lb, ub [..., H] (any other leading axes) -- an object that keeps the
    coefficients of a few positions only.  weights: list of one to three [H_out, H] of one shape; biases: list
    of [H_out] or None entries, or None.  One launch where linear_group would take one.  Returns a list of
    (lw' [..., H_out], lb' [..., H_out], uw', ub')."""
    import ctypes
    rows_w, rows_b, H = _object(lw, lb, uw, ub)
    n = len(weights)
    if not 1 <= n <= 3:
        raise ValueError(f"{n} layers: between one and three share a launch")
    N = weights[0].shape[0]
    biases = list(biases) if biases is not None else [None] * n
    for i, (W, b) in enumerate(zip(weights, biases)):
        _check(f"weight {i}", W, (N, H))
        if b is not None:
            _check(f"bias {i}", b, (N,))
    dev = lw.device
    outs = [(_empty(*lw.shape[:-1], N, device=dev), _empty(*lb.shape[:-1], N, device=dev),
             _empty(*lw.shape[:-1], N, device=dev), _empty(*lb.shape[:-1], N, device=dev)) for _ in range(n)]
    with _on(dev):
        if n == 1:
            o = outs[0]
            _lib.call("faith_matmul_rows_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(weights[0]),
                      _ptr(biases[0]), _ptr(o[1]), _ptr(o[3]), _ptr(o[0]), _ptr(o[2]), rows_w, rows_b, H, N, _stream(lw))
        else:
            arr = ctypes.c_void_p * n
            ptrs = lambda ts: arr(*[_ptr(t) for t in ts])
            a_w, a_b = ptrs(weights), ptrs(biases)
            a_lb, a_ub = ptrs([o[1] for o in outs]), ptrs([o[3] for o in outs])
            a_lw, a_uw = ptrs([o[0] for o in outs]), ptrs([o[2] for o in outs])
            _lib.call("faith_matmul_group_rows_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), n,
                      ctypes.addressof(a_w), ctypes.addressof(a_b), ctypes.addressof(a_lb), ctypes.addressof(a_ub),
                      ctypes.addressof(a_lw), ctypes.addressof(a_uw), rows_w, rows_b, H, N, _stream(lw))
    return outs


def dot_product_qk(x, y, p, eps, words=1, return_intervals=False, out=None):
    """McCormick bounds of x . y^T.  x, y: (lw, lb, uw, ub) tuples with
    lw [B, Lx|Ly, D, d]; returns (lw [B, Lx, D, Ly], lb [B, Lx, Ly], uw, ub)."""
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    B, Lx, D, d = _wb_shapes(xlw, xlb, LAYOUT_NATURAL)
    B2, Ly, D2, d2 = _wb_shapes(ylw, ylb, LAYOUT_NATURAL)
    if (B2, D2, d2) != (B, D, d):
        raise ValueError(f"x {tuple(xlw.shape)} and y {tuple(ylw.shape)} disagree in batch, dim_in or dim_out")
    for n, t, s in (("x.lw", xlw, None), ("x.uw", xuw, xlw.shape), ("x.lb", xlb, None), ("x.ub", xub, xlb.shape),
                    ("y.lw", ylw, None), ("y.uw", yuw, ylw.shape), ("y.lb", ylb, None), ("y.ub", yub, ylb.shape)):
        _check(n, t, s)
    dev = xlw.device
    x_l = _empty_like(xlb); x_u = _empty_like(xlb) if return_intervals else None     # nothing reads x_u
    y_l = _empty_like(ylb); y_u = _empty_like(ylb)
    if out is None:
        zlw = _empty(B, Lx, D, Ly, device=dev)
        zuw = _empty_like(zlw)
        zlb = _empty(B, Lx, Ly, device=dev)
        zub = _empty_like(zlb)
    else:
        zlw, zlb, zuw, zub = out
        _check("out lw", zlw, (B, Lx, D, Ly)); _check("out uw", zuw, (B, Lx, D, Ly))
        _check("out lb", zlb, (B, Lx, Ly)); _check("out ub", zub, (B, Lx, Ly))
    with _on(dev, "dot_qk", (B, Lx, Ly, D, d)):
        _lib.call("faith_dot_product_verification_QK", _ptr(x_l), _ptr(y_l), _ptr(x_u), _ptr(y_u),
                  _ptr(xlb), _ptr(xub), _ptr(ylb), _ptr(yub), _ptr(xlw), _ptr(xuw), _ptr(ylw), _ptr(yuw),
                  _ptr(zlb), _ptr(zub), _ptr(zlw), _ptr(zuw), B, Lx, Ly, d, D, float(eps), q_code(p), int(words),
                  LAYOUT_NATURAL, _stream(xlw))
    if return_intervals:
        return zlw, zlb, zuw, zub, (x_l, x_u, y_l, y_u)
    return zlw, zlb, zuw, zub


def dot_product_v(x, y, p, eps, words=1, return_intervals=False, out=None):
    """McCormick bounds of the attention context x . y (probabilities times values).

    x: (lw [B, Lx, D, Lk], lb [B, Lx, Lk], uw, ub);  y: the VALUE bounds in their natural layout
    (lw [B, Lk, D, dv], lb [B, Lk, dv], uw, ub) -- no transposed copy is needed.
    Returns (lw [B, Lx, D, dv], lb [B, Lx, dv], uw, ub)."""
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    B, Lx, D, Lk = _wb_shapes(xlw, xlb, LAYOUT_NATURAL)
    B2, Lk2, D2, dv = _wb_shapes(ylw, ylb, LAYOUT_NATURAL)
    if (B2, Lk2, D2) != (B, Lk, D):
        raise ValueError(f"x {tuple(xlw.shape)} and y {tuple(ylw.shape)} disagree in batch, key length or dim_in")
    for n, t, s in (("x.lw", xlw, None), ("x.uw", xuw, xlw.shape), ("x.lb", xlb, None), ("x.ub", xub, xlb.shape),
                    ("y.lw", ylw, None), ("y.uw", yuw, ylw.shape), ("y.lb", ylb, None), ("y.ub", yub, ylb.shape)):
        _check(n, t, s)
    dev = xlw.device
    x_l = _empty_like(xlb); x_u = _empty_like(xlb) if return_intervals else None     # nothing reads x_u
    y_l = _empty_like(ylb); y_u = _empty_like(ylb)
    if out is None:
        zlw = _empty(B, Lx, D, dv, device=dev)
        zuw = _empty_like(zlw)
        zlb = _empty(B, Lx, dv, device=dev)
        zub = _empty_like(zlb)
    else:
        zlw, zlb, zuw, zub = out
        _check("out lw", zlw, (B, Lx, D, dv)); _check("out uw", zuw, (B, Lx, D, dv))
        _check("out lb", zlb, (B, Lx, dv)); _check("out ub", zub, (B, Lx, dv))
    with _on(dev, "dot_v", (B, Lx, dv, D, Lk)):
        _lib.call("faith_dot_product_verification_V", _ptr(x_l), _ptr(y_l), _ptr(x_u), _ptr(y_u),
                  _ptr(xlb), _ptr(xub), _ptr(ylb), _ptr(yub), _ptr(xlw), _ptr(xuw), _ptr(ylw), _ptr(yuw),
                  _ptr(zlb), _ptr(zub), _ptr(zlw), _ptr(zuw), B, Lx, Lk, dv, D, float(eps), q_code(p), int(words),
                  LAYOUT_NATURAL, _stream(xlw))
    if return_intervals:
        return zlw, zlb, zuw, zub, (x_l, x_u, y_l, y_u)
    return zlw, zlb, zuw, zub


def attention_scores(x, y, heads, p, eps, words=1):
    """Scores of all heads from query / key bounds as the dense layers leave them.

    x, y: (lw [B, L, D, heads*size], lb [B, L, heads*size], uw, ub).  Same result as folding both with
    transpose_for_scores (VerifierForward.py:208-229) and dot_product_qk, without the eight permuted
    copies: returns (lw [B*heads, Lx, D, Ly], lb [B*heads, Lx, Ly], uw, ub)."""
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    B, Lx, D, H = _wb_shapes(xlw, xlb, LAYOUT_NATURAL)
    B2, Ly, D2, H2 = _wb_shapes(ylw, ylb, LAYOUT_NATURAL)
    if (B2, D2, H2) != (B, D, H):
        raise ValueError(f"x {tuple(xlw.shape)} and y {tuple(ylw.shape)} must be [B, L, dim_in, heads*size] alike")
    if heads <= 0 or H % heads:
        raise ValueError(f"{heads} heads do not divide a row of {H}")
    for n, t, s in (("x.lw", xlw, None), ("x.uw", xuw, xlw.shape), ("x.lb", xlb, None), ("x.ub", xub, xlb.shape),
                    ("y.lw", ylw, None), ("y.uw", yuw, ylw.shape), ("y.lb", ylb, None), ("y.ub", yub, ylb.shape)):
        _check(n, t, s)
    dev = xlw.device
    x_l = _empty_like(xlb); x_u = None                                               # nothing reads x_u
    y_l = _empty_like(ylb); y_u = _empty_like(ylb)
    zlw = _empty(B * heads, Lx, D, Ly, device=dev)
    zuw = _empty_like(zlw)
    zlb = _empty(B * heads, Lx, Ly, device=dev)
    zub = _empty_like(zlb)
    with _on(dev, "dot_qk", (B * heads, Lx, Ly, D, H // heads)):
        _lib.call("faith_attention_scores", _ptr(x_l), _ptr(y_l), _ptr(x_u), _ptr(y_u),
                  _ptr(xlb), _ptr(xub), _ptr(ylb), _ptr(yub), _ptr(xlw), _ptr(xuw), _ptr(ylw), _ptr(yuw),
                  _ptr(zlb), _ptr(zub), _ptr(zlw), _ptr(zuw), B, heads, Lx, Ly, H // heads, D, float(eps), q_code(p),
                  int(words), _stream(xlw))
    return zlw, zlb, zuw, zub


def _positions_of(t, positions):
    if t.dim() != 3:
        raise ValueError(f"expected [B, L, H], got {tuple(t.shape)}")
    _check("t", t)
    B, L, H = t.shape
    if positions.dtype != torch.int64 or positions.dim() != 2 or positions.shape[0] != B or positions.device != t.device \
            or not positions.is_contiguous():
        raise ValueError(f"positions must be a contiguous int64 tensor [{B}, P] on {t.device}")
    return B, L, positions.shape[1], H


def gather_positions(a, b, positions):
    """a, b [B, L, H] -> two tensors [B, P, H]: row positions[b, i] of batch element b (zero where the position lies
    outside the sentence).  One launch for the pair; data movement only, nothing waits for the device."""
    B, L, P, H = _positions_of(a, positions)
    _check("b", b, a.shape)
    oa, ob = _empty(B, P, H, device=a.device), _empty(B, P, H, device=a.device)
    with _on(a.device):
        _lib.call("faith_rows_gather", _ptr(a), _ptr(b), _ptr(positions), _ptr(oa), _ptr(ob), B, L, P, H, _stream(a))
    return oa, ob


def put_positions(a, b, positions, rows_a, rows_b):
    """Copies of a, b [B, L, H] with row positions[b, i] of batch element b replaced by rows_a[b, i], rows_b[b, i]
    ([B, P, H]).  One launch for the pair."""
    B, L, P, H = _positions_of(a, positions)
    _check("b", b, a.shape); _check("rows_a", rows_a, (B, P, H)); _check("rows_b", rows_b, (B, P, H))
    oa, ob = _empty_like(a), _empty_like(b)
    with _on(a.device):
        _lib.call("faith_rows_put", _ptr(a), _ptr(b), _ptr(rows_a), _ptr(rows_b), _ptr(positions), _ptr(oa), _ptr(ob),
                  B, L, P, H, _stream(a))
    return oa, ob


# ------------------------------------------------------------------------------------------
# The layer driver's own device work (input coefficients, recorded preconditions, verdict): one launch each.
# ------------------------------------------------------------------------------------------
_POSITIONS = {}


def positions_tensor(groups, device):
    """int64 [len(groups), P] on the device for host-side lists of positions.  The same few tuples come back for
    every step of a bisection and every query of a sentence, so the tensors are kept (bounded) and a repeated
    query uploads nothing."""
    key = (str(device), tuple(tuple(int(v) for v in g) for g in groups))
    t = _POSITIONS.get(key)
    if t is None:
        if len(_POSITIONS) >= 4096:
            _POSITIONS.clear()
        t = torch.as_tensor(key[1], dtype=torch.int64, device=device).reshape(len(key[1]), -1)
        _POSITIONS[key] = t
    return t


def input_coefficients(batch, rows, words, dim, device, positions=None, scales=None, scale=1.0, out=None):
    """Coefficients of the input object (VerifierForward.py:127-156) [batch, rows, dim * words, dim], written whole by
    one launch: scale * identity (scales[b] * identity with a tensor `scales` [batch]) in block i of the row that
    holds perturbed word i -- row i when positions is None (an object that keeps those rows only: rows == words),
    row positions[b, i] otherwise (int64 [batch, words] on the device) -- and zero elsewhere."""
    device = torch.device(device)
    if device.type != "cuda":
        raise ValueError(f"input_coefficients: must live on the GPU (got {device}); there is no CPU path")
    shape = (batch, rows, dim * words, dim)
    w = _empty(*shape, device=device) if out is None else _check("out", out, shape)
    if positions is not None:
        if not (positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous()
                and tuple(positions.shape) == (batch, words)):
            raise ValueError(f"positions: expected a contiguous int64 GPU tensor of shape {(batch, words)}")
    elif rows != words:
        raise ValueError(f"input_coefficients: without positions the object has one row per word ({rows} != {words})")
    if scales is not None:
        _check("scales", scales, (batch,))
    with _on(w.device):
        _lib.call("faith_input_coefficients", _ptr(w), _ptr(positions), _ptr(scales), float(scale), batch, rows, words,
                  dim, int(positions is None), _stream(w))
    return w


def _flags(name, t, batch):
    if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype in (torch.bool, torch.uint8) and t.is_contiguous()
            and tuple(t.shape) == (batch,)):
        raise ValueError(f"{name}: expected a contiguous bool / uint8 GPU tensor of shape ({batch},)")
    return t


def flag_below(l, flags, bound, strict):
    """flags[b] |= any(l[b] fails `> bound` (strict) / `>= bound`): the preconditions of Bounds.sqrt and
    Bounds.reciprocal (Bounds.py:892, :1147) recorded per batch element; nothing waits for the device."""
    _check("l", l)
    batch = flags.shape[0]
    _flags("flags", flags, batch)
    if l.numel() % batch:
        raise ValueError(f"l: {l.numel()} values do not split over {batch} batch elements")
    with _on(l.device):
        _lib.call("faith_flag_below", _ptr(l), _ptr(flags), batch, l.numel() // batch, float(bound), int(bool(strict)),
                  _stream(l))


_VERDICTS = {}


def verdict(l, u, flags, label, host=False):
    """safe[b] = (l[b, 0, ...] > 0 if label == 0 else u[b, 0, ...] < 0) and not flags[b]
    (VerifierForward.py:311-314 per batch element; flags may be None).  host = False: a bool tensor on the device,
    nothing waits.  host = True: the kernel writes into pinned host memory, the stream is waited for and a list
    of Python bools comes back -- one launch and no copy where reading a device tensor costs a copy kernel."""
    _check("l", l)
    _check("u", u, l.shape)
    batch = l.shape[0]
    if flags is not None:
        _flags("flags", flags, batch)
    if host:
        key = (str(l.device), batch)
        safe = _VERDICTS.get(key)
        if safe is None:
            safe = _VERDICTS[key] = torch.empty(batch, dtype=torch.bool, pin_memory=True)
    else:
        safe = torch.empty(batch, dtype=torch.bool, device=l.device)
    with _on(l.device):
        _lib.call("faith_verdict", _ptr(l), _ptr(u), _ptr(flags), _ptr(safe), batch, l.numel() // batch, int(label),
                  _stream(l))
        if host:
            torch.cuda.current_stream(l.device).synchronize()
            return safe.tolist()
    return safe


def concretize_positions(lw, lb, uw, ub, positions, p, eps, words=1):
    """Concrete interval [B, L, H] of an object whose coefficients lw, uw [B, P, D, H] exist at `positions` [B, P] only
    (lb, ub [B, L, H]): the constants where there are no coefficients, lb - eps ||lw||, ub + eps ||uw|| at the
    positions.  One launch."""
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb); _check("ub", ub, lb.shape)
    if lw.dim() != 4 or lb.dim() != 3:
        raise ValueError(f"lw {tuple(lw.shape)} must be [B, P, dim_in, H] and lb {tuple(lb.shape)} [B, L, H]")
    B, P, D, H = lw.shape
    if lb.shape[0] != B or lb.shape[2] != H:
        raise ValueError(f"lw {tuple(lw.shape)} and lb {tuple(lb.shape)} disagree in batch or width")
    L = lb.shape[1]
    if not (positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous()
            and tuple(positions.shape) == (B, P)):
        raise ValueError(f"positions: expected a contiguous int64 GPU tensor of shape {(B, P)}")
    l, u = _empty_like(lb), _empty_like(ub)
    with _on(lw.device):
        _lib.call("faith_concretize_rows", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(positions), _ptr(l), _ptr(u),
                  B, L, P, D, H, float(eps), q_code(p), int(words), _stream(lw))
    return l, u


def attention_scores_compact_fits(length, n_positions, head_size, dim_in):
    """True if attention_scores_compact takes operands of this shape (16-byte aligned tensors assumed)."""
    return (dim_in > 1 and length % 4 == 0 and head_size % 4 == 0
            and 8 * n_positions * 128 + 16 * head_size * length <= 160 * 1024)


def attention_scores_compact(x, y, x_l, y_l, y_u, positions, heads):
    """attention_scores for a query and a key whose coefficients vanish outside `positions` [B, P] (int64, on the
    device), with only those coefficient rows in memory:

    x, y: (lw [B, P, D, heads*size], lb [B, L, heads*size], uw, ub); x_l, y_l, y_u [B, L, heads*size]: the
    concrete lower bound of x and both bounds of y (concretize of the P rows, the constants elsewhere).
    Returns what attention_scores returns for the operands with the zeros written out.  Raises FaithError
    (FAITH_ERR_UNSUPPORTED) for shapes the kernel does not take: see attention_scores_compact_fits."""
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    _check("x.lw", xlw); _check("x.uw", xuw, xlw.shape); _check("y.lw", ylw, xlw.shape); _check("y.uw", yuw, xlw.shape)
    _check("x.lb", xlb); _check("x.ub", xub, xlb.shape); _check("y.lb", ylb, xlb.shape); _check("y.ub", yub, xlb.shape)
    _check("x_l", x_l, xlb.shape); _check("y_l", y_l, xlb.shape); _check("y_u", y_u, xlb.shape)
    if xlw.dim() != 4 or xlb.dim() != 3:
        raise ValueError(f"x.lw {tuple(xlw.shape)} must be [B, P, dim_in, heads*size] and x.lb {tuple(xlb.shape)} [B, L, heads*size]")
    B, P, D, H = xlw.shape
    L = xlb.shape[1]
    if xlb.shape[0] != B or xlb.shape[2] != H:
        raise ValueError(f"x.lw {tuple(xlw.shape)} and x.lb {tuple(xlb.shape)} disagree in batch or width")
    if heads <= 0 or H % heads:
        raise ValueError(f"{heads} heads do not divide a row of {H}")
    if positions.dtype != torch.int64 or tuple(positions.shape) != (B, P) or positions.device != xlw.device \
            or not positions.is_contiguous():
        raise ValueError(f"positions must be a contiguous int64 tensor [{B}, {P}] on {xlw.device}")
    dev = xlw.device
    zlw = _empty(B * heads, L, D, L, device=dev)
    zuw = _empty_like(zlw)
    zlb = _empty(B * heads, L, L, device=dev)
    zub = _empty_like(zlb)
    with _on(dev):
        _lib.call("faith_attention_scores_compact", _ptr(x_l), _ptr(y_l), _ptr(y_u), _ptr(xlb), _ptr(xub), _ptr(ylb),
                  _ptr(yub), _ptr(xlw), _ptr(xuw), _ptr(ylw), _ptr(yuw), positions.data_ptr(), _ptr(zlb), _ptr(zub),
                  _ptr(zlw), _ptr(zuw), B, heads, L, P, H // heads, D, _stream(xlw))
    return zlw, zlb, zuw, zub


def attention_context(x, y, p, eps, words=1):
    """Context of all heads: probabilities x (lw [B*heads, Lx, D, Lk], lb [B*heads, Lx, Lk], uw, ub) times the
    value bounds y as the dense layer leaves them (lw [B, Lk, D, heads*size], lb [B, Lk, heads*size], uw, ub).

    Same result as transpose_for_scores on y, dot_product_v and transpose_back
    (VerifierForward.py:208-229, :253-263) without the permuted copies: returns
    (lw [B, Lx, D, heads*size], lb [B, Lx, heads*size], uw, ub)."""
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    BH, Lx, D, Lk = _wb_shapes(xlw, xlb, LAYOUT_NATURAL)
    B, Lk2, D2, H = _wb_shapes(ylw, ylb, LAYOUT_NATURAL)
    if (Lk2, D2) != (Lk, D):
        raise ValueError(f"x {tuple(xlw.shape)} and y {tuple(ylw.shape)} disagree in key length or dim_in")
    if BH % B or H % (BH // B):
        raise ValueError(f"x has {BH} (batch, head) pairs; y has batch {B} and rows of {H}")
    heads = BH // B
    for n, t, s in (("x.lw", xlw, None), ("x.uw", xuw, xlw.shape), ("x.lb", xlb, None), ("x.ub", xub, xlb.shape),
                    ("y.lw", ylw, None), ("y.uw", yuw, ylw.shape), ("y.lb", ylb, None), ("y.ub", yub, ylb.shape)):
        _check(n, t, s)
    dev = xlw.device
    x_l = _empty_like(xlb); x_u = None                                               # nothing reads x_u
    y_l = _empty_like(ylb); y_u = _empty_like(ylb)
    zlw = _empty(B, Lx, D, H, device=dev)
    zuw = _empty_like(zlw)
    zlb = _empty(B, Lx, H, device=dev)
    zub = _empty_like(zlb)
    with _on(dev, "dot_v", (BH, Lx, H // heads, D, Lk)):
        _lib.call("faith_attention_context", _ptr(x_l), _ptr(y_l), _ptr(x_u), _ptr(y_u),
                  _ptr(xlb), _ptr(xub), _ptr(ylb), _ptr(yub), _ptr(xlw), _ptr(xuw), _ptr(ylw), _ptr(yuw),
                  _ptr(zlb), _ptr(zub), _ptr(zlw), _ptr(zuw), B, heads, Lx, Lk, H // heads, D, float(eps), q_code(p),
                  int(words), _stream(xlw))
    return zlw, zlb, zuw, zub


def attention_context_compact_fits(length_k, head_size, dim_in):
    """True if attention_context_compact takes a value operand of this shape (16-byte aligned tensors assumed)."""
    return dim_in > 1 and length_k <= 80 and head_size % 4 == 0


def attention_context_compact(x, y, y_l, y_u, positions, p, eps, words=1):
    """attention_context for a value object whose coefficients vanish outside `positions` [B, P] (int64, on the
    device), with only those coefficient rows in memory: y = (lw [B, P, D, heads*size], lb [B, Lk, heads*size], uw, ub);
    y_l, y_u [B, Lk, heads*size] its concrete bounds; x: the probabilities as for attention_context.  Returns what
    attention_context returns for the value object with the zeros written out.  Raises FaithError
    (FAITH_ERR_UNSUPPORTED) for shapes the kernel does not take: see attention_context_compact_fits."""
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    BH, Lx, D, Lk = _wb_shapes(xlw, xlb, LAYOUT_NATURAL)
    for n, t, s in (("x.lw", xlw, None), ("x.uw", xuw, xlw.shape), ("x.lb", xlb, None), ("x.ub", xub, xlb.shape),
                    ("y.lw", ylw, None), ("y.uw", yuw, ylw.shape), ("y.lb", ylb, None), ("y.ub", yub, ylb.shape),
                    ("y_l", y_l, ylb.shape), ("y_u", y_u, ylb.shape)):
        _check(n, t, s)
    if ylw.dim() != 4 or ylb.dim() != 3:
        raise ValueError(f"y.lw {tuple(ylw.shape)} must be [B, P, dim_in, heads*size] and y.lb {tuple(ylb.shape)} [B, Lk, heads*size]")
    B, P, D2, H = ylw.shape
    if tuple(ylb.shape) != (B, Lk, H) or D2 != D:
        raise ValueError(f"x {tuple(xlw.shape)}, y.lw {tuple(ylw.shape)} and y.lb {tuple(ylb.shape)} disagree in batch, key length, dim_in or width")
    if BH % B or H % (BH // B):
        raise ValueError(f"x has {BH} (batch, head) pairs; y has batch {B} and rows of {H}")
    if positions.dtype != torch.int64 or tuple(positions.shape) != (B, P) or positions.device != xlw.device \
            or not positions.is_contiguous():
        raise ValueError(f"positions must be a contiguous int64 tensor [{B}, {P}] on {xlw.device}")
    heads = BH // B
    dev = xlw.device
    x_l = _empty_like(xlb)                                                            # nothing reads x_u
    zlw = _empty(B, Lx, D, H, device=dev)
    zuw = _empty_like(zlw)
    zlb = _empty(B, Lx, H, device=dev)
    zub = _empty_like(zlb)
    with _on(dev):
        _lib.call("faith_attention_context_compact", _ptr(x_l), None, _ptr(y_l), _ptr(y_u),
                  _ptr(xlb), _ptr(xub), _ptr(ylb), _ptr(yub), _ptr(xlw), _ptr(xuw), _ptr(ylw), _ptr(yuw),
                  positions.data_ptr(), _ptr(zlb), _ptr(zub), _ptr(zlw), _ptr(zuw), B, heads, Lx, Lk, P, H // heads, D,
                  float(eps), q_code(p), int(words), _stream(xlw))
    return zlw, zlb, zuw, zub


def conv2d(lw, lb, uw, ub, weight, bias=None, stride=1, padding=0, out=None):
    """Sign-split propagation through a 2-D convolution.
    lw, uw: [1, D_in, C_in, H, W]; lb, ub: [1, C_in, H, W]; weight: [C_out, C_in, K, K]."""
    if lw.dim() != 5 or lb.dim() != 4 or lw.shape[0] != 1 or lb.shape[0] != 1:
        raise ValueError(f"expected lw [1,D,C,H,W] and lb [1,C,H,W], got {tuple(lw.shape)}, {tuple(lb.shape)}")
    _, D, C, Hh, Ww = lw.shape
    _check("lw", lw); _check("uw", uw, lw.shape); _check("lb", lb, (1, C, Hh, Ww)); _check("ub", ub, lb.shape)
    _check("weight", weight)
    if weight.dim() != 4 or weight.shape[1] != C or weight.shape[2] != weight.shape[3]:
        raise ValueError(f"weight must be [C_out, {C}, K, K], got {tuple(weight.shape)}")
    Co, _, K, _ = weight.shape
    if bias is not None:
        _check("bias", bias, (Co,))
    Ho = (Hh + 2 * padding - K) // stride + 1
    Wo = (Ww + 2 * padding - K) // stride + 1
    if Ho <= 0 or Wo <= 0:
        raise ValueError("convolution output would be empty")
    if out is None:
        olw = _empty(1, D, Co, Ho, Wo, device=lw.device)
        ouw = _empty_like(olw)
        olb = _empty(1, Co, Ho, Wo, device=lw.device)
        oub = _empty_like(olb)
    else:
        olw, olb, ouw, oub = out
        _check("out lw", olw, (1, D, Co, Ho, Wo)); _check("out uw", ouw, (1, D, Co, Ho, Wo))
        _check("out lb", olb, (1, Co, Ho, Wo)); _check("out ub", oub, (1, Co, Ho, Wo))
    with _on(lw.device):
        _lib.call("faith_convolution_verification", _ptr(lb), _ptr(ub), _ptr(lw), _ptr(uw), _ptr(weight),
                  _ptr(bias), _ptr(olb), _ptr(oub), _ptr(olw), _ptr(ouw), 1, Hh, Ww, C, Co, K, int(stride),
                  int(padding), D, _stream(lw))
    return olw, olb, ouw, oub


def concretize_conv(lw, lb, uw, ub, p, eps):
    """Concretize conv-shaped bounds (norm over D_in): lw [1, D, C, H, W] -> l, u [1, C, H, W]."""
    _, D, C, Hh, Ww = lw.shape
    l, u = concretize(lw.view(1, 1, D, C * Hh * Ww), lb.view(1, 1, C * Hh * Ww),
                      uw.view(1, 1, D, C * Hh * Ww), ub.view(1, 1, C * Hh * Ww), p, eps, 1)
    return l.view(1, C, Hh, Ww), u.view(1, C, Hh, Ww)
