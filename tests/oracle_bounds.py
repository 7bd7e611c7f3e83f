"""A bound object with the reference's method names whose arithmetic is the CPU oracle.
Lets the layer-level propagation code (faith_amd/forward.py) run on the checker."""
from types import SimpleNamespace

import torch

from oracle import bounds_oracle as O


class OracleBounds:
    def __init__(self, p, eps, lw, lb, uw, ub, words=1):
        self.p, self.eps, self.words = p, eps, words
        self.lw, self.lb, self.uw, self.ub = lw, lb, uw, ub
        self.update_shape()

    def update_shape(self):
        self.batch_size, self.length, self.dim_in, self.dim_out = self.lw.shape[:4]

    def _x(self):
        return O.LinearBounds(self.lw, self.lb, self.uw, self.ub)

    def _w(self, y):
        return OracleBounds(self.p, self.eps, y.lw, y.lb, y.uw, y.ub, self.words)

    def concretize(self):
        return O.concretize(self._x(), self.p, self.eps, self.words)

    def dense(self, layer):
        return self._w(O.linear(self._x(), layer.weight, getattr(layer, "bias", None)))

    def matmul(self, W):
        return self._w(O.linear(self._x(), W))

    def add(self, delta):
        return self._w(O.add(self._x(), delta._x() if isinstance(delta, OracleBounds) else delta))

    def multiply(self, W):
        if isinstance(W, OracleBounds):
            return self._w(O.multiply(self._x(), W._x(), self.p, self.eps, self.words))
        return self._w(O.scale(self._x(), W))

    def act(self, name):
        return getattr(self, name)()

    def dot_product(self, other):
        return self._w(O.dot_product(self._x(), other._x(), self.p, self.eps, self.words))

    def context(self, value):
        return self._w(O.context(self._x(), value._x(), self.p, self.eps, self.words))

    def layer_norm(self, normalizer, mode):
        return self._w(O.layer_norm(self._x(), normalizer.weight, normalizer.bias, mode, self.p, self.eps, self.words))


for _name in ("relu", "tanh", "exp", "sqr", "sqrt", "reciprocal", "softmax"):
    def _method(self, _n=_name):
        return self._w(getattr(O, _n)(self._x(), self.p, self.eps, self.words))
    setattr(OracleBounds, _name, _method)


from faith_amd.workloads import random_layer, to_device  # noqa: E402,F401  (synthetic layers are shared with bench.py)


def true_layer(x, layer, embed_norm, mode, pooler, classifier):
    """The network itself (float64), for soundness checks: x [n, L, H] -> (layer output, margin)."""
    def ln(v, n):
        c = v - v.mean(-1, keepdim=True)
        if mode == "standard":
            c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + 1e-12)
        return c * n.weight.double() + n.bias.double()

    def lin(v, l):
        return v @ l.weight.double().t() + l.bias.double()
    h = ln(x, embed_norm)
    a = layer.attention.self
    n, L, H = h.shape
    split = lambda t: t.reshape(n, L, a.num_attention_heads, a.attention_head_size).permute(0, 2, 1, 3)
    q, k, v = split(lin(h, a.query)), split(lin(h, a.key)), split(lin(h, a.value))
    probs = torch.softmax(q @ k.transpose(-1, -2) / a.attention_head_size ** 0.5, dim=-1)
    ctx = (probs @ v).permute(0, 2, 1, 3).reshape(n, L, H)
    att = ln(lin(ctx, layer.attention.output.dense) + h, layer.attention.output.LayerNorm)
    out = ln(lin(torch.relu(lin(att, layer.intermediate.dense)), layer.output.dense) + att, layer.output.LayerNorm)
    pooled = torch.tanh(lin(out[:, :1], pooler))
    logits = lin(pooled, classifier)
    return out, logits[..., 0] - logits[..., 1]
