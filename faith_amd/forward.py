"""Forward bound propagation through a Transformer encoder layer, written against the `Bounds`
operator surface only.

Host-side mirror of the reference's per-network propagation
(Transformer_Verification_Code/Verifiers/VerifierForward.py): `bound_input` (:127-156),
`bound_attention` (:198-267), `bound_layer` (:158-196), `bound_pooling` (:269-287) and
`bound_classifier` (:289-319).  Nothing here touches tensors except to fold attention heads into
the batch axis and back (reshape / permute, as the reference does); all arithmetic happens in the
methods of the bound object that is passed in, so the same code drives `faith_amd.Bounds` (HIP
kernels) and any other object with those methods (the tests drive the CPU oracle with it).

Layers are plain objects with `.weight` / `.bias` tensors, laid out like the reference's BERT:

    layer.attention.self.{query,key,value}         dense [H, H]
    layer.attention.self.num_attention_heads, .attention_head_size
    layer.attention.output.{dense, LayerNorm}
    layer.intermediate.dense                        dense [I, H]
    layer.output.{dense, LayerNorm}                 dense [H, I]
"""
from __future__ import annotations

import math

import torch


def bound_input(make_bounds, embeddings, index, eps, perturbed_words=1, p=2.0, norm=None, layer_norm="no_var"):
    """VerifierForward._bound_input: identity coefficients at the perturbed position(s).

    embeddings [1, L, dim]; index: position (int) or list of positions; make_bounds(p, eps, lw, lb,
    uw, ub) builds the bound object.  Returns bounds of the (layer-normed) embeddings."""
    length, dim = embeddings.shape[1], embeddings.shape[2]
    w = torch.zeros((length, dim * perturbed_words, dim), device=embeddings.device)
    positions = [index] if perturbed_words == 1 else list(index)
    for i, pos in enumerate(positions):
        w[pos, dim * i:dim * (i + 1), :] = torch.eye(dim, device=embeddings.device)
    lw = w.unsqueeze(0)
    b = embeddings[0].unsqueeze(0)
    bounds = make_bounds(p, eps, lw, b.clone(), lw.clone(), b.clone())
    if norm is not None:
        bounds = bounds.layer_norm(norm, layer_norm)
    return bounds


def _fold_heads(x, heads, size):
    """transpose_for_scores (VerifierForward.py:208-229): [1, L, D, heads*size] -> [heads, L, D, size]."""
    def w(t):
        return t.reshape(t.shape[0], t.shape[1], t.shape[2], heads, size).permute(0, 3, 1, 2, 4) \
                .reshape(-1, t.shape[1], t.shape[2], size)

    def b(t):
        return t.reshape(t.shape[0], t.shape[1], heads, size).permute(0, 2, 1, 3).reshape(-1, t.shape[1], size)
    x.lw, x.uw, x.lb, x.ub = w(x.lw), w(x.uw), b(x.lb), b(x.ub)
    x.update_shape()
    return x


def _unfold_heads(x):
    """transpose_back (VerifierForward.py:253-263): [heads, L, D, size] -> [1, L, D, heads*size]."""
    def w(t):
        return t.permute(1, 2, 0, 3).reshape(1, t.shape[1], t.shape[2], -1)

    def b(t):
        return t.permute(1, 0, 2).reshape(1, t.shape[1], -1)
    x.lw, x.uw, x.lb, x.ub = w(x.lw), w(x.uw), b(x.lb), b(x.ub)
    x.update_shape()
    return x


def bound_attention(bounds_input, attention):
    """VerifierForward._bound_attention: scores = Q.K^T / sqrt(d), probs = softmax, context = probs.V."""
    heads = attention.self.num_attention_heads
    size = attention.self.attention_head_size
    query = bounds_input.dense(attention.self.query)
    key = bounds_input.dense(attention.self.key)
    value = bounds_input.dense(attention.self.value)
    if hasattr(query, "attention_scores"):
        # the HIP kernels address the heads where the dense layers leave them: no permuted copies
        scores = query.attention_scores(key, heads).multiply(1.0 / math.sqrt(size))
        probs = scores.softmax()
        return scores, probs, probs.attention_context(value)
    _fold_heads(query, heads, size)
    _fold_heads(key, heads, size)
    scores = query.dot_product(key).multiply(1.0 / math.sqrt(size))
    probs = scores.softmax()
    _fold_heads(value, heads, size)
    context = probs.context(value)
    _unfold_heads(context)
    return scores, probs, context


def bound_layer(bounds_input, layer, layer_norm="no_var", hidden_act="relu"):
    """VerifierForward._bound_layer: attention block, residual + norm, feed-forward, residual + norm."""
    scores, probs, attention = bound_attention(bounds_input, layer.attention)
    attention = attention.dense(layer.attention.output.dense)
    attention = attention.add(bounds_input).layer_norm(layer.attention.output.LayerNorm, layer_norm)
    intermediate = attention.dense(layer.intermediate.dense).act(hidden_act)
    dense = intermediate.dense(layer.output.dense).add(attention)
    output = dense.layer_norm(layer.output.LayerNorm, layer_norm)
    return scores, probs, output


def bound_pooling(bounds, pooler_dense, make_bounds):
    """VerifierForward._bound_pooling: first position, dense, tanh."""
    first = make_bounds(bounds.p, bounds.eps, bounds.lw[:, :1], bounds.lb[:, :1], bounds.uw[:, :1], bounds.ub[:, :1])
    return first.dense(pooler_dense).tanh()


def bound_classifier(bounds, classifier, label):
    """VerifierForward._bound_classifier: margin logit[0] - logit[1], concretized; True if provably safe."""
    class Margin:
        weight = classifier.weight.clone()
        bias = classifier.bias.clone()
    Margin.weight[0, :] -= Margin.weight[1, :]
    Margin.bias[0] -= Margin.bias[1]
    out = bounds.dense(Margin)
    l, u = out.concretize()
    safe = bool(l[0][0][0] > 0) if label == 0 else bool(u[0][0][0] < 0)
    return safe, l, u
