"""Seeded synthetic inputs of the five benchmark configurations.

Shared by the parity tests and bench.py so that the CPU checker and the HIP
path see identical tensors.  Everything is generated on the CPU in fp32 with
``torch.Generator().manual_seed(1000 + cfg)``, drawing (per bound object)
lw, the uw gap, lb, the ub gap, and then the layer's W and bias.
"""
from __future__ import annotations

import math
from types import SimpleNamespace

import torch

INF = float("inf")


def _bounds(g, shape_w, shape_b, sw, sgap, sb, sbgap):
    lw = torch.randn(*shape_w, generator=g) * sw
    uw = lw + (torch.randn(*shape_w, generator=g) * sgap).abs()
    lb = torch.randn(*shape_b, generator=g) * sb
    ub = lb + (torch.randn(*shape_b, generator=g) * sbgap).abs()
    return dict(lw=lw, lb=lb, uw=uw, ub=ub)


def make_config(cfg: int, scale: float = 1.0) -> dict:
    """Inputs of configuration ``cfg`` (0..4).

    ``scale`` < 1 shrinks the length axis L (for conv: the D_in axis) so that
    the CPU checker finishes quickly; 1.0 is the full benchmark size.
    """
    g = torch.Generator().manual_seed(1000 + cfg)

    def sc(v, lo=1):
        return max(lo, int(round(v * scale)))

    if cfg == 0:     # small linear + concretize(p=inf)
        L = sc(16)
        x = _bounds(g, (1, L, 64, 64), (1, L, 64), 0.1, 0.01, 1.0, 0.1)
        W = torch.randn(64, 64, generator=g) / 8
        b = torch.randn(64, generator=g) * 0.01
        return dict(op="linear", x=x, W=W, bias=b, p=INF, eps=0.01, words=1)
    if cfg == 1:     # relu / tanh relaxations, two perturbed words
        L = sc(128)
        x = _bounds(g, (1, L, 256, 512), (1, L, 512), 0.05, 0.005, 1.0, 0.5)
        return dict(op="act", x=x, ps=(1.0, 2.0, INF), eps=0.01, words=2)
    if cfg == 2:     # large linear + concretize(p=2)
        L = sc(256)
        x = _bounds(g, (1, L, 512, 1024), (1, L, 1024), 0.02, 0.002, 1.0, 0.1)
        W = torch.randn(1024, 1024, generator=g) / 32
        b = torch.randn(1024, generator=g) * 0.01
        return dict(op="linear", x=x, W=W, bias=b, p=2.0, eps=0.01, words=1)
    if cfg == 3:     # attention Q.K^T, 4 heads folded into the batch axis
        L = sc(128, 2)
        qs, ks = [], []
        for _ in range(4):
            qs.append(_bounds(g, (1, L, 256, 64), (1, L, 64), 0.05, 0.005, 1.0, 0.2))
            ks.append(_bounds(g, (1, L, 256, 64), (1, L, 64), 0.05, 0.005, 1.0, 0.2))

        def stack(bs):
            return {k: torch.cat([b[k] for b in bs], 0) for k in bs[0]}
        return dict(op="dot", x=stack(qs), y=stack(ks), p=INF, eps=0.01, words=1)
    if cfg == 4:     # 3x3 convolution, 64 -> 128 channels
        D = sc(256)
        x = _bounds(g, (1, D, 64, 32, 32), (1, 64, 32, 32), 0.05, 0.005, 1.0, 0.1)
        W = torch.randn(128, 64, 3, 3, generator=g) * math.sqrt(2.0 / (9 * 64))
        b = torch.randn(128, generator=g) * 0.01
        return dict(op="conv", x=x, W=W, bias=b, stride=1, padding=1, p=INF, eps=2.0 / 255)
    raise ValueError(f"no such configuration: {cfg}")


# ------------------------------------------------------------------ a whole encoder layer
def random_layer(g, hidden, heads, inter, scale=0.5):
    """Random weights of one Transformer encoder layer, laid out like the reference's BERT modules
    (the attribute names faith_amd/forward.py reads)."""
    def lin(n_out, n_in):
        return SimpleNamespace(weight=torch.randn(n_out, n_in, generator=g) * scale / n_in ** 0.5,
                               bias=torch.randn(n_out, generator=g) * 0.05)

    def norm(n):
        return SimpleNamespace(weight=1.0 + 0.1 * torch.randn(n, generator=g), bias=0.05 * torch.randn(n, generator=g))
    att_self = SimpleNamespace(query=lin(hidden, hidden), key=lin(hidden, hidden), value=lin(hidden, hidden),
                               num_attention_heads=heads, attention_head_size=hidden // heads)
    attention = SimpleNamespace(self=att_self, output=SimpleNamespace(dense=lin(hidden, hidden), LayerNorm=norm(hidden)))
    return SimpleNamespace(attention=attention, intermediate=SimpleNamespace(dense=lin(inter, hidden)),
                           output=SimpleNamespace(dense=lin(hidden, inter), LayerNorm=norm(hidden)))


def to_device(obj, device):
    """Deep copy of a layer description with every tensor moved to `device`."""
    if isinstance(obj, torch.Tensor):
        return obj.to(device)
    if isinstance(obj, SimpleNamespace):
        return SimpleNamespace(**{k: to_device(v, device) for k, v in vars(obj).items()})
    return obj
