"""One Transformer encoder layer end to end: embeddings -> layer norm -> self-attention -> feed
forward -> pooling -> classifier, driven by faith_amd/forward.py.

CPU: the pipeline on the oracle is sound (the true network output of sampled perturbations lies
inside the propagated bounds).  GPU: the same pipeline on faith_amd.Bounds reproduces the oracle's
bounds and is sound as well.  Mirrors VerifierForward.verify_safety (VerifierForward.py:93-125)."""
from types import SimpleNamespace

import pytest
import torch

from faith_amd import forward as F
from tests.oracle_bounds import OracleBounds, random_layer, to_device, true_layer

HIDDEN, HEADS, INTER, LENGTH = 32, 4, 64, 6


def build(seed, mode):
    g = torch.Generator().manual_seed(seed)
    layer = random_layer(g, HIDDEN, HEADS, INTER)
    embed_norm = SimpleNamespace(weight=1.0 + 0.1 * torch.randn(HIDDEN, generator=g),
                                 bias=0.05 * torch.randn(HIDDEN, generator=g))
    pooler = SimpleNamespace(weight=torch.randn(HIDDEN, HIDDEN, generator=g) / HIDDEN ** 0.5,
                             bias=0.05 * torch.randn(HIDDEN, generator=g))
    classifier = SimpleNamespace(weight=torch.randn(2, HIDDEN, generator=g) / HIDDEN ** 0.5,
                                 bias=0.05 * torch.randn(2, generator=g))
    emb = torch.randn(1, LENGTH, HIDDEN, generator=g)
    return layer, embed_norm, pooler, classifier, emb


def propagate(make, emb, parts, mode, p, eps, index):
    layer, embed_norm, pooler, classifier = parts
    x = F.bound_input(make, emb, index, eps, 1, p, embed_norm, mode)
    scores, probs, out = F.bound_layer(x, layer, mode, "relu")
    pooled = F.bound_pooling(out, pooler, make)
    safe, l, u = F.bound_classifier(pooled, classifier, 0)
    return out, l, u, safe


def check_sound(out_l, out_u, l, u, emb, parts, mode, p, eps, index, g):
    layer, embed_norm, pooler, classifier = parts
    d = torch.randn(64, HIDDEN, generator=g, dtype=torch.float64)
    if p == float("inf"):
        d = torch.sign(d) * eps
    else:
        d = d / torch.linalg.vector_norm(d, ord=p, dim=1, keepdim=True) * eps
    x = emb.double().repeat(64, 1, 1)
    x[:, index] += d
    out, margin = true_layer(x, layer, embed_norm, mode, pooler, classifier)
    slack = 1e-4
    assert bool((out >= out_l.double() - slack).all()) and bool((out <= out_u.double() + slack).all())
    lo, hi = l.double()[0, 0, 0], u.double()[0, 0, 0]        # output 0 of the margin classifier
    assert bool((margin >= lo - slack).all()) and bool((margin <= hi + slack).all())


@pytest.mark.parametrize("mode", ["no_var", "standard"])
@pytest.mark.parametrize("p", [2.0, float("inf")])
def test_pipeline_on_the_oracle_is_sound(mode, p):
    layer, embed_norm, pooler, classifier, emb = build(7, mode)
    eps, index = 0.02, 2
    make = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub)
    out, l, u, _ = propagate(make, emb, (layer, embed_norm, pooler, classifier), mode, p, eps, index)
    ol, ou = out.concretize()
    assert bool((l <= u).all()) and bool((ol <= ou).all())
    check_sound(ol, ou, l, u, emb, (layer, embed_norm, pooler, classifier), mode, p, eps, index,
                torch.Generator().manual_seed(8))


def test_margin_layer_is_kept_until_the_classifier_changes():
    g = torch.Generator().manual_seed(9)
    classifier = SimpleNamespace(weight=torch.randn(2, HIDDEN, generator=g), bias=torch.randn(2, generator=g))
    lw = torch.randn(1, 1, 5, HIDDEN, generator=g)
    lb = torch.randn(1, 1, HIDDEN, generator=g)
    x = OracleBounds(2.0, 0.1, lw, lb, lw + 0.01, lb + 0.1)

    def expected():
        w = classifier.weight.clone()
        b = classifier.bias.clone()
        w[0] -= w[1]
        b[0] -= b[1]
        return x.dense(SimpleNamespace(weight=w, bias=b)).concretize()
    l, u = F._margin(x, classifier)
    el, eu = expected()
    assert torch.equal(l, el) and torch.equal(u, eu)
    first = classifier._faith_margin
    F._margin(x, classifier)
    assert classifier._faith_margin is first                 # unchanged parameters: not rebuilt
    classifier.weight[1, 3] += 0.5                           # in place: the stamp changes
    l, u = F._margin(x, classifier)
    el, eu = expected()
    assert classifier._faith_margin is not first and torch.equal(l, el) and torch.equal(u, eu)
    classifier.bias = torch.zeros(2)                         # replaced: another storage
    l, u = F._margin(x, classifier)
    el, eu = expected()
    assert torch.equal(l, el) and torch.equal(u, eu)
    assert not torch.equal(classifier.weight[0], first.weight[0])        # the classifier itself is never modified


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["no_var", "standard"])
@pytest.mark.parametrize("p", [2.0, float("inf")])
def test_pipeline_on_hip_matches_the_oracle_and_is_sound(mode, p):
    from faith_amd import Bounds
    layer, embed_norm, pooler, classifier, emb = build(7, mode)
    eps, index = 0.02, 2
    parts = (layer, embed_norm, pooler, classifier)
    omake = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub)
    o_out, o_l, o_u, o_safe = propagate(omake, emb, parts, mode, p, eps, index)

    gparts = tuple(to_device(x, "cuda") for x in parts)
    gmake = lambda p_, e_, lw, lb, uw, ub: Bounds(None, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    g_out, g_l, g_u, g_safe = propagate(gmake, emb.cuda(), gparts, mode, p, eps, index)
    torch.cuda.synchronize()

    # ~25 chained operators: compare at a tolerance that allows rounding to compound, relative to the
    # size of the quantities involved
    def near(a, b, what, rel=2e-4):
        a, b = a.cpu().double(), b.double()
        err = float((a - b).abs().max())
        scale = float(b.abs().max())
        assert err <= rel * max(scale, 1.0), f"{what}: max err {err:.3g} at scale {scale:.3g}"
    near(g_out.lw, o_out.lw, "output lw"); near(g_out.uw, o_out.uw, "output uw")
    near(g_out.lb, o_out.lb, "output lb"); near(g_out.ub, o_out.ub, "output ub")
    # behind the pooler's tanh the chord slopes divide by interval widths of ~1e-2, which amplifies
    # the accumulated differences once more
    near(g_l, o_l, "margin l", 1e-3); near(g_u, o_u, "margin u", 1e-3)
    gl, gu = g_out.concretize()
    check_sound(gl.cpu(), gu.cpu(), g_l.cpu(), g_u.cpu(), emb, parts, mode, p, eps, index,
                torch.Generator().manual_seed(9))


# ------------------------------------------------------------------ verification driver
def network_of(parts, mode):
    layer, embed_norm, pooler, classifier = parts
    return SimpleNamespace(embedding_norm=embed_norm, layers=[layer], pooler=pooler, classifier=classifier,
                           layer_norm=mode, hidden_act="relu")


def test_certified_radius_on_the_oracle_brackets_the_verdict():
    """Bisection of Verifier.verify: the radius it returns verifies, one step above it does not, and
    the true network keeps its label inside the radius."""
    layer, embed_norm, pooler, classifier, emb = build(11, "no_var")
    net = network_of((layer, embed_norm, pooler, classifier), "no_var")
    make = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub)
    _, margin = true_layer(emb.double(), layer, embed_norm, "no_var", pooler, classifier)
    label = 0 if float(margin[0, 0]) > 0 else 1
    max_eps, iters = 0.5, 6
    (r,) = F.certified_radii(make, net, emb, [2], label, 2.0, max_eps, iters)
    step = max_eps / 2 ** iters
    assert 0 <= r < max_eps
    if r > 0:
        assert F.verify_safety(make, net, emb, 2, r, label, 2.0)
    assert not F.verify_safety(make, net, emb, 2, r + step, label, 2.0)
    # soundness: perturbations inside the certified radius do not flip the label
    g = torch.Generator().manual_seed(12)
    d = torch.randn(256, HIDDEN, generator=g, dtype=torch.float64)
    d = d / d.norm(dim=1, keepdim=True) * r
    x = emb.double().repeat(256, 1, 1)
    x[:, 2] += d
    _, m = true_layer(x, layer, embed_norm, "no_var", pooler, classifier)
    assert bool(((m[:, 0] > 0) == (label == 0)).all())


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["no_var", "standard"])
def test_batched_bisection_on_hip_matches_one_at_a_time_and_the_oracle(mode):
    """All positions in lockstep (one batch element each, radius folded into the coefficients) give
    the radii of the reference's one-at-a-time search, on the HIP path and on the oracle."""
    from faith_amd import Bounds
    layer, embed_norm, pooler, classifier, emb = build(11, mode)
    parts = (layer, embed_norm, pooler, classifier)
    _, margin = true_layer(emb.double(), layer, embed_norm, mode, pooler, classifier)
    label = 0 if float(margin[0, 0]) > 0 else 1
    positions, max_eps, iters = [1, 2, 3, 4], 0.5, 6
    step = max_eps / 2 ** iters
    omake = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub)
    want = F.certified_radii(omake, network_of(parts, mode), emb, positions, label, 2.0, max_eps, iters)

    gnet = network_of(tuple(to_device(x, "cuda") for x in parts), mode)
    gmake = lambda p_, e_, lw, lb, uw, ub: Bounds(None, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    one = F.certified_radii(gmake, gnet, emb.cuda(), positions, label, 2.0, max_eps, iters)
    lock = F.certified_radii(gmake, gnet, emb.cuda(), positions, label, 2.0, max_eps, iters, batched=True)
    print(f"[case] radii oracle {want} hip {one} hip batched {lock}", flush=True)
    # a verdict that sits within rounding of the decision threshold may fall either way: one step
    for a, b, c in zip(want, one, lock):
        assert abs(a - b) <= step + 1e-12 and abs(a - c) <= step + 1e-12
    assert sum(a == c for a, c in zip(want, lock)) >= len(positions) - 1


@pytest.mark.gpu
@pytest.mark.parametrize("batched", [False, True])
def test_persistent_buffers_give_the_same_radii_and_stop_allocating(batched):
    """The caller owns results and scratch across propagations (ops.Workspace, as the reference's adapters own
    theirs, Bounds.py:1270-1277): the same radii as with per-call allocation, and after the first propagation
    the operator calls allocate no buffer."""
    from faith_amd import Bounds, ops
    layer, embed_norm, pooler, classifier, emb = build(11, "no_var")
    parts = (layer, embed_norm, pooler, classifier)
    _, margin = true_layer(emb.double(), layer, embed_norm, "no_var", pooler, classifier)
    label = 0 if float(margin[0, 0]) > 0 else 1
    positions, max_eps, iters = [1, 2, 3], 0.5, 5
    gnet = network_of(tuple(to_device(x, "cuda") for x in parts), "no_var")
    gmake = lambda p_, e_, lw, lb, uw, ub: Bounds(None, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    want = F.certified_radii(gmake, gnet, emb.cuda(), positions, label, 2.0, max_eps, iters, batched=batched)
    ws = ops.Workspace()
    if batched:
        F.verify_safety_batch(gmake, gnet, emb.cuda(), positions, [0.01] * 3, label, 2.0, buffers=ws)
    else:
        F.verify_safety(gmake, gnet, emb.cuda(), 1, 0.01, label, 2.0, buffers=ws)
    first = ws.allocations
    assert first > 20 and ws.bytes() > 0
    got = F.certified_radii(gmake, gnet, emb.cuda(), positions, label, 2.0, max_eps, iters, batched=batched, buffers=ws)
    assert got == want
    assert ws.allocations == first, "a repeated propagation allocated result buffers"
    assert ops._WORKSPACE is None


@pytest.mark.gpu
def test_failed_preconditions_are_recorded_per_batch_element():
    """Inside collect_failures a reciprocal whose interval reaches zero marks its own batch element
    only and nothing raises; outside it asserts, as the reference does."""
    from faith_amd import Bounds
    g = torch.Generator().manual_seed(13)
    lw = 0.01 * torch.randn(3, 4, 8, 16, generator=g)
    lb = torch.rand(3, 4, 16, generator=g) + 1.0
    lb[1, 2, 5] = -0.5                                      # element 1 crosses zero
    b = Bounds(None, 2.0, 0.1, lw=lw.cuda(), lb=lb.cuda(), uw=lw.cuda() + 0.001, ub=lb.cuda() + 0.1)
    with Bounds.collect_failures(3, "cuda") as f:
        b.reciprocal()
        assert f.mask.tolist() == [False, True, False]
    with pytest.raises(AssertionError):
        b.reciprocal()


@pytest.mark.gpu
def test_captured_propagation_replays_like_the_eager_one():
    """The propagation captured as a HIP graph: every replay -- with other radii and positions, and
    with eager work and synchronisations in between -- gives the eager verdicts and margins."""
    from faith_amd import Bounds
    layer, embed_norm, pooler, classifier, emb = build(11, "standard")
    parts = (layer, embed_norm, pooler, classifier)
    _, margin = true_layer(emb.double(), layer, embed_norm, "standard", pooler, classifier)
    label = 0 if float(margin[0, 0]) > 0 else 1
    gnet = network_of(tuple(to_device(x, "cuda") for x in parts), "standard")
    gmake = lambda p_, e_, lw, lb, uw, ub: Bounds(None, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    ge = emb.cuda()
    cap = F.CapturedVerifier(gmake, gnet, ge, 4, label, 2.0)
    queries = [([1, 2, 3, 4], [0.004, 0.004, 0.004, 0.004]), ([4, 3, 2, 1], [0.001, 0.02, 0.008, 0.3]),
               ([1, 1, 1, 1], [0.0005, 0.009, 0.0078125, 1.0]), ([2, 4, 2, 4], [0.012, 0.012, 0.25, 0.004]),
               ([1, 2, 3, 4], [0.004, 0.004, 0.004, 0.004])]
    seen = set()
    for idx, radii in queries:
        print(f"[case] captured replay positions {idx} radii {radii}", flush=True)
        got = cap(idx, radii)
        want = F.verify_safety_batch(gmake, gnet, ge, idx, radii, label, 2.0)      # eager work between replays
        torch.cuda.synchronize()
        assert got == want, (idx, radii, got, want)
        seen.update(got)
    assert seen == {True, False}                  # the queries exercise both verdicts
    # and the search built on it finds the same radii
    a = F.certified_radii(gmake, gnet, ge, [1, 2, 3, 4], label, 2.0, 0.5, 6, batched=True)
    b = F.certified_radii(gmake, gnet, ge, [1, 2, 3, 4], label, 2.0, 0.5, 6, captured=True)
    assert a == b


def two_layer_network(seed, mode):
    g = torch.Generator().manual_seed(seed)
    layers = [random_layer(g, HIDDEN, HEADS, INTER), random_layer(g, HIDDEN, HEADS, INTER)]
    embed_norm = SimpleNamespace(weight=1.0 + 0.1 * torch.randn(HIDDEN, generator=g),
                                 bias=0.05 * torch.randn(HIDDEN, generator=g))
    pooler = SimpleNamespace(weight=torch.randn(HIDDEN, HIDDEN, generator=g) / HIDDEN ** 0.5,
                             bias=0.05 * torch.randn(HIDDEN, generator=g))
    classifier = SimpleNamespace(weight=torch.randn(2, HIDDEN, generator=g) / HIDDEN ** 0.5,
                                 bias=0.05 * torch.randn(2, generator=g))
    emb = torch.randn(1, LENGTH, HIDDEN, generator=g)
    net = SimpleNamespace(embedding_norm=embed_norm, layers=layers, pooler=pooler, classifier=classifier,
                          layer_norm=mode, hidden_act="relu")
    return net, emb


@pytest.mark.gpu
@pytest.mark.parametrize("mode", ["no_var", "standard"])
def test_two_layers_with_two_perturbed_words_match_the_oracle(mode):
    """Two encoder layers, two perturbed positions (dim_in = 2 * hidden, perturbed_words = 2): the
    margin bounds of the HIP path against the oracle's."""
    from faith_amd import Bounds
    net, emb = two_layer_network(21, mode)
    eps, index, p = 0.01, [1, 4], 2.0

    def margins(make, network, e):
        x = F.bound_input(make, e, index, eps, 2, p, network.embedding_norm, network.layer_norm)
        pooled = F.bound_pooling(F.propagate(x, network), network.pooler, make)
        return F.bound_classifier(pooled, network.classifier, 0)

    omake = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub, words=2)
    _, ol, ou = margins(omake, net, emb)

    two_words = SimpleNamespace(perturbed_words=2)
    gmake = lambda p_, e_, lw, lb, uw, ub: Bounds(two_words, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    gnet = SimpleNamespace(**{k: (to_device(v, "cuda") if k in ("embedding_norm", "pooler", "classifier") else v)
                              for k, v in vars(net).items()})
    gnet.layers = [to_device(l, "cuda") for l in net.layers]
    _, gl, gu = margins(gmake, gnet, emb.cuda())
    torch.cuda.synchronize()
    assert bool((gl <= gu).all())
    width = float((ou - ol).abs().max())
    # ~50 chained operators, tanh slopes at the end: compare relative to the width of the interval
    assert float((gl.cpu() - ol).abs().max()) <= 2e-3 * max(width, 1.0), (gl, ol)
    assert float((gu.cpu() - ou).abs().max()) <= 2e-3 * max(width, 1.0), (gu, ou)
