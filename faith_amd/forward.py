"""Forward bound propagation through a Transformer encoder layer, written against the `Bounds`
operator surface only.

Host-side mirror of the reference's per-network propagation
(Transformer_Verification_Code/Verifiers/VerifierForward.py): `bound_input` (:127-156),
`bound_attention` (:198-267), `bound_layer` (:158-196), `bound_pooling` (:269-287) and
`bound_classifier` (:289-319), `verify_safety` (:93-125), and of the search for the certified radius
of every position (Verifiers/Verifier.py:107-147).  Nothing here touches tensors except to build the
input object and to fold attention heads into the batch axis and back where the bound object cannot
address them in place; all arithmetic happens in the methods of the bound object that is passed in,
so the same code drives `faith_amd.Bounds` (HIP kernels) and any other object with those methods
(the tests drive the CPU oracle with it).

The reference verifies one (position, radius) at a time.  Every operator here is independent
across the batch axis, so `certified_radii` can also run the bisections of all positions in
lockstep, one batch element per position (`bound_inputs`): the radius of an element is folded into
its input coefficients (w = r * I with eps = 1 describes the same set as w = I with eps = r), so
elements with different radii share every launch.

Layers are plain objects with `.weight` / `.bias` tensors, laid out like the reference's BERT:

    layer.attention.self.{query,key,value}         dense [H, H]
    layer.attention.self.num_attention_heads, .attention_head_size
    layer.attention.output.{dense, LayerNorm}
    layer.intermediate.dense                        dense [I, H]
    layer.output.{dense, LayerNorm}                 dense [H, I]
"""
from __future__ import annotations

import contextlib
import math

import torch


def _scope(buffers):
    """`buffers`: None, or persistent result buffers for the operator calls of one propagation -- any object
    whose scope() is a context manager (faith_amd.ops.Workspace): the caller owns results and scratch across
    calls, as the reference's adapters do (Bounds.py:1270-1277), and a repeated propagation allocates none."""
    return buffers.scope() if buffers is not None else contextlib.nullcontext()


def bound_input(make_bounds, embeddings, index, eps, perturbed_words=1, p=2.0, norm=None, layer_norm="no_var",
                ibp=False):
    """VerifierForward._bound_input (:127-156): identity coefficients at the perturbed position(s); with
    ibp (interval bound propagation) zero coefficients and the constant terms widened by eps there.

    embeddings [1, L, dim]; index: position (int) or list of positions; make_bounds(p, eps, lw, lb,
    uw, ub) builds the bound object.  Returns bounds of the (layer-normed) embeddings."""
    length, dim = embeddings.shape[1], embeddings.shape[2]
    positions = _checked_positions([[index] if perturbed_words == 1 else list(index)], length)[0]
    if len(positions) != perturbed_words:
        raise ValueError(f"{len(positions)} positions given for {perturbed_words} perturbed words")
    compact = _compact_maker(make_bounds, 1, length, dim * perturbed_words, dim)
    dev = embeddings.device
    if compact is not None and not ibp:
        # a maker that can hold the coefficients of the perturbed positions alone: the zero rows of
        # every other position are never written, read or multiplied
        w = _input_coefficients(make_bounds, 1, perturbed_words, perturbed_words, dim, dev)
        b = embeddings[0].unsqueeze(0)
        bounds = compact(p, eps, _positions(make_bounds, [positions], dev), w, b, w, b)
        return bounds if norm is None else bounds.layer_norm(norm, layer_norm)
    if ibp:
        lw = torch.zeros((1, length, dim * perturbed_words, dim), device=dev)
        lb, ub = embeddings[0].unsqueeze(0).clone(), embeddings[0].unsqueeze(0).clone()
        for pos in positions:
            lb[0, pos] -= eps
            ub[0, pos] += eps
    else:
        # lower and upper start out equal and no operator writes into its inputs: one tensor serves both
        # (the reference copies ub and uw, :131, :149)
        lb = ub = embeddings[0].unsqueeze(0)
        lw = _input_coefficients(make_bounds, 1, length, perturbed_words, dim, dev,
                                 _positions(make_bounds, [positions], dev))
    bounds = make_bounds(p, eps, lw, lb, lw, ub)
    if norm is not None:
        bounds = bounds.layer_norm(norm, layer_norm)
    return bounds


def _checked_positions(groups, length):
    """Positions as the input builders take them: `groups` is one list of perturbed positions per batch element.
    Every position must lie in 0 ... length-1 and the positions of one batch element must be distinct; they index
    device tensors further on (an out-of-range index there is a device-side assert that ends the process, and a
    repeated one makes the written-out object depend on the order of the writes), so they are checked here, on the
    host, where the lists still are."""
    out = []
    for b, group in enumerate(groups):
        g = [int(v) for v in group]
        for v, raw in zip(g, group):
            if v != raw:
                raise ValueError(f"position {raw!r} of batch element {b} is not an integer")
            if not 0 <= v < length:
                raise ValueError(f"position {v} of batch element {b} lies outside 0 ... {length - 1}")
        if len(set(g)) != len(g):
            raise ValueError(f"the positions {g} of batch element {b} are not distinct")
        out.append(g)
    return out


def _compact_maker(make_bounds, batch, length, dim_in, dim_out, captured=False):
    """make_bounds.compact if the maker has one (faith_amd.BoundsMaker) and finds that leaving out the zero
    coefficient rows pays for an object of this shape, else None.  captured: the propagation is replayed from a
    graph, where a launch costs the device's time only."""
    compact = getattr(make_bounds, "compact", None)
    pays = getattr(make_bounds, "compact_pays", None)
    if compact is None:
        return None
    if pays is not None and not (pays(batch, length, dim_in, dim_out, captured=True) if captured else
                                 pays(batch, length, dim_in, dim_out)):
        return None
    return compact


def _positions(make_bounds, groups, device):
    """int64 [len(groups), P] on the device; a maker may keep them across calls (`positions_tensor`)."""
    keep = getattr(make_bounds, "positions_tensor", None)
    if keep is not None:
        return keep(groups, device)
    return torch.as_tensor(groups, dtype=torch.int64, device=device).reshape(len(groups), -1)


def _input_coefficients(make_bounds, batch, rows, words, dim, device, positions=None, scales=None, out=None):
    """[batch, rows, dim * words, dim]: scales[b] * identity (identity without scales) in block i of the row that
    holds perturbed word i -- row positions[b, i], or row i when positions is None (rows == words) -- and zero
    elsewhere.  One launch when the maker brings its own builder (`input_coefficients`), tensor expressions
    otherwise."""
    build = getattr(make_bounds, "input_coefficients", None)
    if build is not None:
        return build(batch, rows, words, dim, device, positions, scales, out)
    w = torch.zeros((batch, rows, dim * words, dim), device=device) if out is None else out.zero_()
    eye = _eye(dim, device)
    block = eye.expand(batch, dim, dim) if scales is None else scales[:, None, None] * eye
    every = torch.arange(batch, device=device)
    for i in range(words):
        at = positions[:, i] if positions is not None else torch.full((batch,), i, device=device)
        w[every, at, dim * i:dim * (i + 1), :] = block
    return w


def _verdict(bounds_type, l, u, failed, label):
    """VerifierForward._bound_classifier (:311-314) per batch element, and not a failed precondition; a list of bools."""
    own = getattr(bounds_type, "verdict", None)
    if own is not None:
        return own(l, u, failed.mask, label, host=True)
    ok = (l[:, 0, 0] > 0) if label == 0 else (u[:, 0, 0] < 0)
    return [bool(v) for v in (ok & ~failed.mask).tolist()]


_EYES = {}


def _eye(dim, device):
    key = (dim, str(device))
    if key not in _EYES:
        _EYES[key] = torch.eye(dim, device=device)
    return _EYES[key]


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


def _unfold_heads(x, heads):
    """transpose_back (VerifierForward.py:253-263): [B*heads, L, D, size] -> [B, L, D, heads*size]."""
    def w(t):
        n, L, D, size = t.shape
        return t.reshape(n // heads, heads, L, D, size).permute(0, 2, 3, 1, 4).reshape(n // heads, L, D, -1)

    def b(t):
        n, L, size = t.shape
        return t.reshape(n // heads, heads, L, size).permute(0, 2, 1, 3).reshape(n // heads, L, -1)
    x.lw, x.uw, x.lb, x.ub = w(x.lw), w(x.uw), b(x.lb), b(x.ub)
    x.update_shape()
    return x


def bound_attention(bounds_input, attention, want_scores=True):
    """VerifierForward._bound_attention: scores = Q.K^T / sqrt(d), probs = softmax, context = probs.V.
    want_scores = False (the layer pipeline, which uses the context only) leaves the scaled scores unmaterialised
    where the bound object's softmax takes the factor itself; the first element returned is then None."""
    heads = attention.self.num_attention_heads
    size = attention.self.attention_head_size
    if hasattr(bounds_input, "dense_group"):
        query, key, value = bounds_input.dense_group([attention.self.query, attention.self.key, attention.self.value])
    else:
        query = bounds_input.dense(attention.self.query)
        key = bounds_input.dense(attention.self.key)
        value = bounds_input.dense(attention.self.value)
    if hasattr(query, "attention_scores"):
        # the HIP kernels address the heads where the dense layers leave them: no permuted copies
        if not want_scores:
            probs = query.attention_scores(key, heads).softmax(scale=1.0 / math.sqrt(size))
            return None, probs, probs.attention_context(value)
        scores = query.attention_scores(key, heads).multiply(1.0 / math.sqrt(size))
        probs = scores.softmax()
        return scores, probs, probs.attention_context(value)
    _fold_heads(query, heads, size)
    _fold_heads(key, heads, size)
    scores = query.dot_product(key).multiply(1.0 / math.sqrt(size))
    probs = scores.softmax()
    _fold_heads(value, heads, size)
    context = probs.context(value)
    _unfold_heads(context, heads)
    return scores, probs, context


def _add_norm(x, residual, normalizer, layer_norm):
    """x.add(residual).layer_norm(...); one launch where the bound object takes the residual itself."""
    if hasattr(x, "attention_scores"):        # the HIP-backed object (the oracle's keeps the reference's signature)
        return x.layer_norm(normalizer, layer_norm, residual=residual)
    return x.add(residual).layer_norm(normalizer, layer_norm)


def _dense_add_norm(x, dense, residual, normalizer, layer_norm):
    """x.dense(dense).add(residual).layer_norm(...); one pass where the bound object has the operator for it."""
    if hasattr(x, "dense_layer_norm"):
        return x.dense_layer_norm(dense, normalizer, layer_norm, residual=residual)
    return _add_norm(x.dense(dense), residual, normalizer, layer_norm)


def bound_layer(bounds_input, layer, layer_norm="no_var", hidden_act="relu", want_scores=False):
    """VerifierForward._bound_layer: attention block, residual + norm, feed-forward, residual + norm.
    Returns (scores, probs, output); scores is None unless asked for (see bound_attention)."""
    scores, probs, attention = bound_attention(bounds_input, layer.attention, want_scores)
    attention = _dense_add_norm(attention, layer.attention.output.dense, bounds_input, layer.attention.output.LayerNorm,
                                layer_norm)
    if hasattr(attention, "dense_act"):
        intermediate = attention.dense_act(layer.intermediate.dense, hidden_act)
    else:
        intermediate = attention.dense(layer.intermediate.dense).act(hidden_act)
    output = _dense_add_norm(intermediate, layer.output.dense, attention, layer.output.LayerNorm, layer_norm)
    return scores, probs, output


def bound_pooling(bounds, pooler_dense, make_bounds):
    """VerifierForward._bound_pooling: first position, dense, tanh."""
    own = getattr(bounds, "first_position", None)
    if own is not None:
        return own().dense(pooler_dense).tanh()
    first = make_bounds(bounds.p, bounds.eps, bounds.lw[:, :1], bounds.lb[:, :1], bounds.uw[:, :1], bounds.ub[:, :1])
    return first.dense(pooler_dense).tanh()


class _MarginLayer:
    def __init__(self, classifier):
        self.weight = classifier.weight.detach().clone()
        self.bias = classifier.bias.detach().clone()
        self.weight[0, :] -= self.weight[1, :]
        self.bias[0] -= self.bias[1]
        self.made_from = _stamp(classifier)


def _stamp(layer):
    # identifies the parameter values: the storage and torch's in-place modification counter
    return tuple((t.data_ptr(), t._version) for t in (layer.weight, layer.bias))


def _margin(bounds, classifier):
    """Row 0 of the classifier minus row 1 (VerifierForward.py:289-292 builds it by a deep copy on every call); kept on the
    classifier object until its parameters change."""
    cached = getattr(classifier, "_faith_margin", None)
    if cached is None or cached.made_from != _stamp(classifier):
        cached = _MarginLayer(classifier)
        try:
            classifier._faith_margin = cached
        except AttributeError:          # an object that takes no new attributes: rebuilt per call
            pass
    fused = getattr(bounds, "dense_concretize", None)
    if fused is not None:
        _, l, u = fused(cached)
        return l, u
    return bounds.dense(cached).concretize()


def bound_classifier(bounds, classifier, label):
    """VerifierForward._bound_classifier: margin logit[0] - logit[1], concretized; True if provably safe."""
    l, u = _margin(bounds, classifier)
    safe = bool(l[0][0][0] > 0) if label == 0 else bool(u[0][0][0] < 0)
    return safe, l, u


def bound_inputs(make_bounds, embeddings, indices, radii, p=2.0, norm=None, layer_norm="no_var"):
    """Independent problems in one object: batch element b perturbs position indices[b] of the same
    sentence within radius radii[b].  The radius goes into the coefficients and the object carries
    eps = 1 (see the module docstring).  embeddings [1, L, dim]."""
    length, dim = embeddings.shape[1], embeddings.shape[2]
    n = len(indices)
    if len(radii) != n:
        raise ValueError(f"{n} positions, {len(radii)} radii")
    indices = [g[0] for g in _checked_positions([[i] for i in indices], length)]
    dev = embeddings.device
    scale = torch.as_tensor(radii, dtype=torch.float32, device=dev)
    b = embeddings[0].unsqueeze(0).expand(n, length, dim).contiguous()
    compact = _compact_maker(make_bounds, n, length, dim, dim)
    # lower and upper start out equal and no operator writes into its inputs: one tensor serves both
    at = _positions(make_bounds, [[i] for i in indices], dev)
    if compact is not None:
        w = _input_coefficients(make_bounds, n, 1, 1, dim, dev, scales=scale)
        bounds = compact(p, 1.0, at, w, b, w, b)
    else:
        w = _input_coefficients(make_bounds, n, length, 1, dim, dev, at, scale)
        bounds = make_bounds(p, 1.0, w, b, w, b)
    if norm is not None:
        bounds = bounds.layer_norm(norm, layer_norm)
    return bounds


def propagate(bounds, network):
    """Embedding bounds -> bounds of the pooled output: every encoder layer, then the pooler
    (the body of VerifierForward.verify_safety, :98-116)."""
    for layer in network.layers:
        _, _, bounds = bound_layer(bounds, layer, network.layer_norm, network.hidden_act)
    return bounds


def verify_safety(make_bounds, network, embeddings, index, eps, label, p=2.0, perturbed_words=1, buffers=None):
    """VerifierForward.verify_safety (:93-125): True if the label provably survives every
    perturbation of norm <= eps of the embedding at `index`.  A failed precondition inside the
    propagation (reciprocal or sqrt of a bound that reaches zero) counts as not verified, as there."""
    with _scope(buffers):
        return _verify_safety(make_bounds, network, embeddings, index, eps, label, p, perturbed_words)


def _verify_safety(make_bounds, network, embeddings, index, eps, label, p, perturbed_words):
    x = bound_input(make_bounds, embeddings, index, eps, perturbed_words, p)
    collector = getattr(type(x), "collect_failures", None)
    try:
        if collector is None:
            if network.embedding_norm is not None:
                x = x.layer_norm(network.embedding_norm, network.layer_norm)
            x = propagate(x, network)
            pooled = bound_pooling(x, network.pooler, make_bounds)
            return bound_classifier(pooled, network.classifier, label)[0]
        # a bound object that can record a failed precondition on the device: nothing waits for the GPU
        # before the verdict is read
        with collector(1, embeddings.device) as failed:
            if network.embedding_norm is not None:
                x = x.layer_norm(network.embedding_norm, network.layer_norm)
            x = propagate(x, network)
            pooled = bound_pooling(x, network.pooler, make_bounds)
            l, u = _margin(pooled, network.classifier)
            return _verdict(type(x), l, u, failed, label)[0]
    except AssertionError:
        return False


def verify_safety_batch(make_bounds, network, embeddings, indices, radii, label, p=2.0, buffers=None):
    """verify_safety for several (position, radius) pairs of one sentence in one propagation.
    Returns a list of bools.  Needs a bound object that reports failed preconditions per batch
    element instead of raising (`collect_failures`, as faith_amd.Bounds has)."""
    x = bound_inputs(make_bounds, embeddings, indices, radii, p)
    with _scope(buffers), type(x).collect_failures(len(indices), embeddings.device) as failed:
        if network.embedding_norm is not None:
            x = x.layer_norm(network.embedding_norm, network.layer_norm)
        x = propagate(x, network)
        pooled = bound_pooling(x, network.pooler, make_bounds)
        l, u = _margin(pooled, network.classifier)
        return _verdict(type(x), l, u, failed, label)


def certified_radii(make_bounds, network, embeddings, positions, label, p=2.0, max_eps=0.1, num_iters=10,
                    batched=False, captured=False, buffers=None):
    """The bisection of Verifier.verify (Verifiers/Verifier.py:131-139) for every position: l, r = 0,
    max_eps; num_iters times { m = (l + r) / 2; verified at m ? l = m : r = m }; the answer is l.
    batched = True runs step j of all positions as one propagation; captured = True also replays
    that propagation from a HIP graph captured at the first step.  buffers: persistent result buffers shared
    by all steps (see _scope); every step overwrites what the one before produced."""
    lo = [0.0] * len(positions)
    hi = [float(max_eps)] * len(positions)
    if batched or captured:
        step = CapturedVerifier(make_bounds, network, embeddings, len(positions), label, p) if captured else \
            (lambda idx, r: verify_safety_batch(make_bounds, network, embeddings, idx, r, label, p, buffers))
        for _ in range(num_iters):
            mid = [(a + b) / 2 for a, b in zip(lo, hi)]
            safe = step(positions, mid)
            for i, s in enumerate(safe):
                if s:
                    lo[i] = mid[i]
                else:
                    hi[i] = mid[i]
        return lo
    for i, pos in enumerate(positions):
        for _ in range(num_iters):
            m = (lo[i] + hi[i]) / 2
            if verify_safety(make_bounds, network, embeddings, pos, m, label, p, buffers=buffers):
                lo[i] = m
            else:
                hi[i] = m
    return lo


class CapturedVerifier:
    """verify_safety_batch for one sentence with the whole propagation captured ONCE as a HIP graph.

    A propagation is a fixed sequence of launches whose arguments depend on shapes only: the radius
    lives in the input coefficients (eps = 1, see bound_inputs) and failed preconditions are recorded
    on the device, so nothing in it waits for the host.  Replaying the graph takes the per-launch
    host work (23 C-ABI calls and about as many tensor allocations per layer) out of every
    (positions, radii) query after the first.  Needs a bound object with collect_failures
    (faith_amd.Bounds).  `batch` is the number of (position, radius) pairs per replay."""

    def __init__(self, make_bounds, network, embeddings, batch, label, p=2.0):
        length, dim = embeddings.shape[1], embeddings.shape[2]
        dev = embeddings.device
        self.batch, self.label, self.dim, self.length, self.make_bounds = batch, label, dim, length, make_bounds
        self.b = embeddings[0].unsqueeze(0).expand(batch, length, dim).contiguous()
        compact = _compact_maker(make_bounds, batch, length, dim, dim, captured=True)
        if compact is not None:
            # the graph reads the perturbed positions and the scaled identities from these two
            self.at = torch.zeros((batch, 1), dtype=torch.int64, device=dev)
            self.w = torch.zeros((batch, 1, dim, dim), device=dev)
        else:
            self.at = None
            self.w = torch.zeros((batch, length, dim, dim), device=dev)

        def body():
            if compact is not None:
                x = compact(p, 1.0, self.at, self.w, self.b, self.w, self.b)
            else:
                x = make_bounds(p, 1.0, self.w, self.b, self.w, self.b)
            with type(x).collect_failures(batch, dev) as failed:
                if network.embedding_norm is not None:
                    x = x.layer_norm(network.embedding_norm, network.layer_norm)
                pooled = bound_pooling(propagate(x, network), network.pooler, make_bounds)
                l, u = _margin(pooled, network.classifier)
            own = getattr(type(x), "verdict", None)
            if own is not None:
                return own(l, u, failed.mask, label)
            ok = (l[:, 0, 0] > 0) if label == 0 else (u[:, 0, 0] < 0)
            return ok & ~failed.mask

        # torch's capture protocol: run eagerly on a side stream first (library handles, caches of
        # device properties, the allocator's pools), then capture
        side = torch.cuda.Stream(device=dev)
        side.wait_stream(torch.cuda.current_stream(dev))
        with torch.cuda.stream(side):
            for _ in range(2):
                body()
        torch.cuda.current_stream(dev).wait_stream(side)
        torch.cuda.synchronize(dev)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph):
            self.safe = body()

    def __call__(self, indices, radii):
        """Verdicts for batch element b = (position indices[b], radius radii[b]); len == batch."""
        if len(indices) != self.batch or len(radii) != self.batch:
            raise ValueError(f"this graph was captured for {self.batch} (position, radius) pairs per replay")
        indices = [g[0] for g in _checked_positions([[i] for i in indices], self.length)]
        dev = self.w.device
        scale = torch.as_tensor(radii, dtype=torch.float32, device=dev)
        at = _positions(self.make_bounds, [[i] for i in indices], dev)
        if self.at is not None:
            self.at.copy_(at)
            _input_coefficients(self.make_bounds, self.batch, 1, 1, self.dim, dev, scales=scale, out=self.w)
        else:
            _input_coefficients(self.make_bounds, self.batch, self.length, 1, self.dim, dev, at, scale, out=self.w)
        self.graph.replay()
        return [bool(v) for v in self.safe.tolist()]
