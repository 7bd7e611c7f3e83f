"""`CompactBounds`: the input object of a query with its zero rows left out.

The input of a verification query has coefficients at the perturbed position(s) only
(VerifierForward.py:127-156).  The compact object runs the embedding layer norm and the first dense
layers on those rows alone; these tests hold it to the results of the ordinary object that carries the
zeros -- bit for bit where the same kernel sees the same rows (layer norm), to the parity bar where the
affine kernel may pick another tiling for the smaller problem -- and the whole propagation built on it
to the verdicts and margins of the one built on the ordinary object."""
from types import SimpleNamespace

import pytest
import torch

from faith_amd import forward as F
from tests.helpers import ATOL, RTOL, worst
from tests.oracle_bounds import OracleBounds, to_device, true_layer
from tests.parity import KAPPA, U32
from tests.test_layer_pipeline import HIDDEN, LENGTH, build, network_of, two_layer_network

pytestmark = pytest.mark.gpu


def compact_and_dense(seed, B=3, P=2, D=10, H=24, L=5, words=1, shared=False, positions=None, p=2.0):
    from faith_amd import Bounds, CompactBounds
    g = torch.Generator().manual_seed(seed)
    at = positions
    positions = torch.stack([torch.randperm(L, generator=g)[:P] for _ in range(B)]) if at is None else at.cpu()
    lw = torch.randn(B, P, D, H, generator=g)
    uw = lw if shared else lw + 0.05 * torch.rand(B, P, D, H, generator=g)
    lb = torch.randn(B, L, H, generator=g)
    ub = lb if shared else lb + 0.3 * torch.rand(B, L, H, generator=g)
    args = SimpleNamespace(perturbed_words=words)
    dev = lambda t: t.cuda()
    c = CompactBounds(args, p, 0.1, dev(positions) if at is None else at, dev(lw), dev(lb), dev(lw if shared else uw), dev(ub))
    rows = torch.arange(B)[:, None]
    dlw = torch.zeros(B, L, D, H); dlw[rows, positions] = lw
    duw = torch.zeros(B, L, D, H); duw[rows, positions] = uw
    d = Bounds(args, p, 0.1, lw=dev(dlw), lb=dev(lb), uw=dev(duw), ub=dev(ub))
    return c, d


def same_bits(a, b, what):
    for name in ("lw", "lb", "uw", "ub"):
        x, y = getattr(a, name), getattr(b, name)
        assert x.shape == y.shape, (what, name, x.shape, y.shape)
        assert torch.equal(x, y), f"{what}.{name}: {int((x != y).sum())} values differ"


def at_the_bar(a, b, what, src=None, weight=None):
    """rtol 1e-5 / atol 1e-6.  With `src` and `weight` (an affine layer applied to the object src): two fp32
    sums of the same K products in different orders -- the affine kernel tiles the smaller problem its own
    way -- cannot be held to atol against each other where the products are larger than the sum, so each of
    the two gets the forward-error allowance of an fp32 dot product, KAPPA * u * sum_k |a_k w_k|, on top."""
    for name in ("lw", "lb", "uw", "ub"):
        x, y = getattr(a, name), getattr(b, name)
        assert x.shape == y.shape, (what, name, x.shape, y.shape)
        err, of_bar = worst(x, y)
        if of_bar <= 1.0:
            continue
        assert src is not None, f"{what}.{name}: max err {err:.3g}, {of_bar:.2f} of the bar"
        lo, hi = (src.lw, src.uw) if name in ("lw", "uw") else (src.lb, src.ub)
        terms = (lo.double().abs() + hi.double().abs()).cpu() @ weight.double().abs().cpu().T
        tol = ATOL + RTOL * y.double().abs().cpu() + 2 * KAPPA * U32 * terms
        over = float(((x.double() - y.double()).abs().cpu() / tol).max())
        assert over <= 1.0, f"{what}.{name}: max err {err:.3g}, {over:.2f} of the accumulation-aware bar"


def layer_of(g, h_in, h_out, bias=True):
    return SimpleNamespace(weight=(torch.randn(h_out, h_in, generator=g) / h_in ** 0.5).cuda(),
                           bias=(0.1 * torch.randn(h_out, generator=g)).cuda() if bias else None)


@pytest.mark.parametrize("shared", [False, True])
def test_dense_form_writes_the_zeros_out(shared):
    c, d = compact_and_dense(3, shared=shared)
    same_bits(c.dense_form(), d, "dense form")
    assert c.dense_form() is c.dense_form()
    # what the compact object does not define is the dense object's
    assert c.lw.shape == d.lw.shape and c.dim_in == d.dim_in and c.batch_size == d.batch_size
    (cl, cu), (dl, du) = c.concretize(), d.concretize()
    assert torch.equal(cl, dl) and torch.equal(cu, du)
    same_bits(c.relu(), d.relu(), "relu through the dense form")


def test_layer_norm_keeps_the_form_and_the_bits():
    from faith_amd import CompactBounds
    g = torch.Generator().manual_seed(5)
    c, d = compact_and_dense(4, B=4, P=1, D=12, H=40, L=7)
    norm = SimpleNamespace(weight=(1.0 + 0.2 * torch.randn(40, generator=g)).cuda(), bias=(0.1 * torch.randn(40, generator=g)).cuda())
    out = c.layer_norm(norm, "no_var")
    assert isinstance(out, CompactBounds) and out._lw.shape == c._lw.shape
    same_bits(out, d.layer_norm(norm, "no_var"), "layer norm, no_var")
    # the variance mixes nothing across positions either, but has no compact kernel: through the dense form
    same_bits(c.layer_norm(norm, "standard"), d.layer_norm(norm, "standard"), "layer norm, standard")
    assert c.layer_norm(norm, "no") is c
    # as the residual of another object's layer norm, and with a residual of its own
    other = d.relu()
    same_bits(other.layer_norm(norm, "no_var", residual=c), other.layer_norm(norm, "no_var", residual=d), "as residual")
    same_bits(c.layer_norm(norm, "no_var", residual=other), d.layer_norm(norm, "no_var", residual=other), "with residual")


@pytest.mark.parametrize("shape", [(3, 2, 10, 24, 5, 16), (2, 1, 64, 64, 9, 96), (5, 3, 33, 20, 4, 7), (1, 1, 256, 256, 32, 256)])
def test_dense_layers_on_the_rows_that_are_not_zero(shape):
    from faith_amd import CompactBounds
    B, P, D, H, L, N = shape
    g = torch.Generator().manual_seed(B * 100 + N)
    c, d = compact_and_dense(6, B, P, D, H, L)
    for bias in (True, False):
        layer = layer_of(g, H, N, bias)
        out = c.dense(layer)
        assert isinstance(out, CompactBounds) and out.positions is c.positions
        at_the_bar(out, d.dense(layer), f"dense {shape} bias={bias}", d, layer.weight)
        at_the_bar(c.matmul(layer.weight, layer.bias), d.matmul(layer.weight, layer.bias), "matmul", d, layer.weight)
    # positions without coefficients get exact zeros, whatever the buffer held before
    zero_rows = torch.ones(B, L, dtype=torch.bool)
    zero_rows[torch.arange(B)[:, None], c.positions.cpu()] = False
    assert float(out.lw.cpu()[zero_rows].abs().max()) == 0.0 and float(out.uw.cpu()[zero_rows].abs().max()) == 0.0
    layers = [layer_of(g, H, N), layer_of(g, H, N, False), layer_of(g, H, N)]
    for got, want, layer in zip(c.dense_group(layers), d.dense_group(layers), layers):
        at_the_bar(got, want, f"dense_group {shape}", d, layer.weight)
    # layers of different shapes: one call each
    mixed = [layer_of(g, H, N), layer_of(g, H, N + 3)]
    for got, want, layer in zip(c.dense_group(mixed), d.dense_group(mixed), mixed):
        at_the_bar(got, want, f"dense_group of two shapes {shape}", d, layer.weight)


def score_terms(x, y, heads):
    """sum_k |a| |x.w| + |b| |y.w| per coefficient of the scores and the like for the constants: what two fp32
    summations of the same products in different orders may differ by, up to KAPPA * u."""
    (xl, xu), (yl, yu) = x.concretize(), y.concretize()
    f = lambda t: t.double().cpu()
    B, L, D, H = x.lw.shape
    size = H // heads
    heads_of = lambda t: f(t).reshape(B, L, *t.shape[2:-1], heads, size)
    xa, ya = heads_of(x.lw.abs() + x.uw.abs()), heads_of(y.lw.abs() + y.uw.abs())          # [B, L, D, h, k]
    a, b = heads_of(yl.abs() + yu.abs()), heads_of(xl.abs())                                 # [B, L, h, k]
    w = torch.einsum("bjhk,bimhk->bhimj", a, xa) + torch.einsum("bihk,bjmhk->bhimj", b, ya)
    xb, yb = heads_of(x.lb.abs() + x.ub.abs()), heads_of(y.lb.abs() + y.ub.abs())
    c = torch.einsum("bjhk,bihk->bhij", a, xb + b) + torch.einsum("bihk,bjhk->bhij", b, yb)
    return w.reshape(B * heads, L, D, L), c.reshape(B * heads, L, L)


def context_terms(probs, dv, heads):
    """sum_k |a| |x.w| + |b| |y.w| per coefficient of the context and the like for the constants: what two fp32 sums
    of the same products in different orders may differ by, up to KAPPA * u."""
    f = lambda t: t.double().cpu()
    BH, L, D, Lk = probs.lw.shape
    B = BH // heads
    size = dv.lw.shape[3] // heads
    (xl, xu), (yl, yu) = probs.concretize(), dv.concretize()
    a = f(yl.abs() + yu.abs()).reshape(B, Lk, heads, size)                             # [b, k, h, c]
    xa = f(probs.lw.abs() + probs.uw.abs()).reshape(B, heads, L, D, Lk)                # [b, h, i, m, k]
    ya = f(dv.lw.abs() + dv.uw.abs()).reshape(B, Lk, D, heads, size)                   # [b, k, m, h, c]
    bt = f(xl.abs()).reshape(B, heads, L, Lk)                                          # [b, h, i, k]
    tw = (torch.einsum("bkhc,bhimk->bimhc", a, xa) + torch.einsum("bhik,bkmhc->bimhc", bt, ya)).reshape(B, L, D, heads * size)
    xb = f(probs.lb.abs() + probs.ub.abs()).reshape(B, heads, L, Lk)
    yb = f(dv.lb.abs() + dv.ub.abs()).reshape(B, Lk, heads, size)
    tb = (torch.einsum("bkhc,bhik->bihc", a, xb + bt) + torch.einsum("bhik,bkhc->bihc", bt, yb)).reshape(B, L, heads * size)
    return tw, tb


@pytest.mark.parametrize("shape", [(3, 1, 24, 2, 16, 8), (2, 2, 64, 4, 16, 12), (5, 3, 130, 3, 20, 16),
                                   (4, 1, 256, 4, 64, 32), (1, 2, 512, 4, 64, 32),
                                   (1, 1, 64, 2, 64, 128)])      # the last: 129 KB of LDS (more than the default 64 KB)
@pytest.mark.parametrize("p", [2.0, float("inf"), 1.0])
def test_scores_from_compact_operands(shape, p):
    """Query and key with coefficients at the same few positions: the kernel that writes the dense scores from the
    compact rows against the dense kernel on the operands with the zeros written out."""
    from faith_amd import Bounds, ops
    B, P, D, heads, size, L = shape
    words = 2 if D % 2 == 0 and P == 2 else 1
    print(f"[case] compact scores B={B} P={P} D={D} heads={heads} size={size} L={L} p={p} words={words}", flush=True)
    assert ops.attention_scores_compact_fits(L, P, size, D)
    cq, dq = compact_and_dense(31, B, P, D, heads * size, L, words=words, p=p)
    ck, dk = compact_and_dense(32, B, P, D, heads * size, L, words=words, p=p, positions=cq.positions)
    got, want = cq.attention_scores(ck, heads), dq.attention_scores(dk, heads)
    assert isinstance(got, Bounds) and got.lw.shape == (B * heads, L, D, L)
    tw, tb = score_terms(dq, dk, heads)
    for name, terms in (("lw", tw), ("uw", tw), ("lb", tb), ("ub", tb)):
        x, y = getattr(got, name), getattr(want, name)
        tol = ATOL + RTOL * y.double().abs().cpu() + 2 * KAPPA * U32 * terms
        over = float(((x.double() - y.double()).abs().cpu() / tol).max())
        assert over <= 1.0, f"scores.{name}: {over:.2f} of the accumulation-aware bar"
    # exact zeros wherever neither the query's nor the key's position has coefficients
    at = cq.positions.cpu()
    has = torch.zeros(B, L, dtype=torch.bool)
    has[torch.arange(B)[:, None], at] = True
    neither = ~(has[:, :, None] | has[:, None, :])                                     # [B, i, j]
    neither = neither[:, None].expand(B, heads, L, L).reshape(B * heads, L, L)
    lw = got.lw.cpu().permute(0, 1, 3, 2)                                             # [B*heads, i, j, m]
    assert float(lw[neither].abs().max()) == 0.0 and float(got.uw.cpu().permute(0, 1, 3, 2)[neither].abs().max()) == 0.0


@pytest.mark.parametrize("shape", [(3, 1, 24, 2, 16, 8), (2, 2, 64, 4, 16, 12), (5, 3, 130, 3, 20, 6),
                                   (4, 1, 256, 4, 64, 32), (1, 2, 96, 2, 8, 30)])
@pytest.mark.parametrize("p", [2.0, float("inf")])
def test_context_from_a_compact_value_operand(shape, p):
    """Probabilities times a value object with coefficients at a few key positions only: the context kernel that
    takes the rows that exist against the same kernel on the value object with the zeros written out (key lengths
    that are multiples of 8 and others: the two instantiations)."""
    from faith_amd import Bounds, ops
    B, P, D, heads, size, L = shape
    print(f"[case] compact context B={B} P={P} D={D} heads={heads} size={size} L={L} p={p}", flush=True)
    assert ops.attention_context_compact_fits(L, size, D)
    cv, dv = compact_and_dense(41, B, P, D, heads * size, L, p=p)
    g = torch.Generator().manual_seed(42)
    lw = 0.3 * torch.randn(B * heads, L, D, L, generator=g); uw = lw + 0.02 * torch.rand(B * heads, L, D, L, generator=g)
    lb = torch.rand(B * heads, L, L, generator=g); ub = lb + 0.1 * torch.rand(B * heads, L, L, generator=g)
    probs = Bounds(cv.args, p, 0.1, lw=lw.cuda(), lb=lb.cuda(), uw=uw.cuda(), ub=ub.cuda())
    got, want = probs.attention_context(cv), probs.attention_context(dv)
    assert cv._dense is None, "the compact value operand was written out"
    assert got.lw.shape == (B, L, D, heads * size)
    tw, tb = context_terms(probs, dv, heads)
    for name, terms in (("lw", tw), ("uw", tw), ("lb", tb), ("ub", tb)):
        x, y = getattr(got, name), getattr(want, name)
        tol = ATOL + RTOL * y.double().abs().cpu() + 2 * KAPPA * U32 * terms
        over = float(((x.double() - y.double()).abs().cpu() / tol).max())
        assert over <= 1.0, f"context.{name}: {over:.2f} of the accumulation-aware bar"


def test_context_from_a_compact_value_operand_falls_back():
    """More than 80 key positions, or a value object that has been written out already: the dense kernel, same bits."""
    from faith_amd import Bounds, ops
    B, P, D, heads, size, L = 1, 1, 16, 2, 8, 88
    assert not ops.attention_context_compact_fits(L, size, D)
    cv, dv = compact_and_dense(43, B, P, D, heads * size, L)
    g = torch.Generator().manual_seed(44)
    lw = 0.3 * torch.randn(B * heads, 8, D, L, generator=g); lb = torch.rand(B * heads, 8, L, generator=g)
    probs = Bounds(cv.args, 2.0, 0.1, lw=lw.cuda(), lb=lb.cuda(), uw=(lw + 0.01).cuda(), ub=(lb + 0.1).cuda())
    same_bits(probs.attention_context(cv), probs.attention_context(dv), "88 key positions")
    cv, dv = compact_and_dense(45, 2, 1, 16, heads * size, 8)
    lw = 0.3 * torch.randn(2 * heads, 8, 16, 8, generator=g); lb = torch.rand(2 * heads, 8, 8, generator=g)
    probs = Bounds(cv.args, 2.0, 0.1, lw=lw.cuda(), lb=lb.cuda(), uw=(lw + 0.01).cuda(), ub=(lb + 0.1).cuda())
    cv.dense_form()
    same_bits(probs.attention_context(cv), probs.attention_context(dv), "written out before")


def test_scores_from_compact_operands_fall_back_to_the_dense_kernel():
    """Shapes the compact kernel does not take (a length that is no multiple of 4, a key with other positions, an
    ordinary key): the dense kernel on the written-out operands, same results as for ordinary objects."""
    from faith_amd import ops
    B, P, D, heads, size, L = 2, 1, 24, 2, 8, 6
    assert not ops.attention_scores_compact_fits(L, P, size, D)
    cq, dq = compact_and_dense(33, B, P, D, heads * size, L)
    ck, dk = compact_and_dense(34, B, P, D, heads * size, L, positions=cq.positions)
    same_bits(cq.attention_scores(ck, heads), dq.attention_scores(dk, heads), "length 6")
    cq, dq = compact_and_dense(35, B, P, D, heads * size, 8)
    ck, dk = compact_and_dense(36, B, P, D, heads * size, 8)                          # positions of its own
    same_bits(cq.attention_scores(ck, heads), dq.attention_scores(dk, heads), "other positions")
    same_bits(cq.attention_scores(dk, heads), dq.attention_scores(dk, heads), "ordinary key")
    same_bits(dq.attention_scores(ck, heads), dq.attention_scores(dk, heads), "ordinary query")


def test_compact_scores_entry_point_checks_its_arguments():
    from faith_amd import _lib, ops
    cq, _ = compact_and_dense(37, 2, 1, 24, 16, 8)
    ck, _ = compact_and_dense(38, 2, 1, 24, 16, 8, positions=cq.positions)
    x = (cq._lw, cq._lb, cq._uw, cq._ub)
    y = (ck._lw, ck._lb, ck._uw, ck._ub)
    (x_l, _), (y_l, y_u) = cq.concrete_intervals(), ck.concrete_intervals()
    with pytest.raises(ValueError):
        ops.attention_scores_compact(x, y, x_l, y_l, y_u, cq.positions.int(), 2)
    with pytest.raises(ValueError):
        ops.attention_scores_compact(x, y, x_l, y_l, y_u, cq.positions, 3)
    with pytest.raises(_lib.FaithError) as err:                 # head size 2: not a multiple of 4
        ops.attention_scores_compact(x, y, x_l, y_l, y_u, cq.positions, 8)
    assert err.value.code == _lib.ERR_UNSUPPORTED
    # a position outside the sentence: that row is not there, nothing is read or written out of bounds
    far = cq.positions.clone()
    far[0, 0] = 1000
    out = ops.attention_scores_compact(x, y, x_l, y_l, y_u, far, 2)
    torch.cuda.synchronize()
    assert float(out[0][:2].abs().max()) == 0.0 and float(out[0][2:].abs().max()) > 0.0


def test_a_position_outside_the_sentence_means_the_row_is_not_there():
    """Both compact entry points with two positions per batch element of which one lies outside 0 ... length-1: that
    row is skipped (include/faith_amd.h), so the results are those of the dense entry points on operands that have
    coefficients at the other position only.  Nothing is read or written out of bounds, the kernels run normally."""
    from faith_amd import Bounds, ops
    B, P, D, heads, size, L = 2, 2, 32, 2, 16, 12
    cq, _ = compact_and_dense(51, B, P, D, heads * size, L)
    ck, _ = compact_and_dense(52, B, P, D, heads * size, L, positions=cq.positions)
    far = cq.positions.clone()
    far[:, 1] = torch.tensor([L, -3], device=far.device)          # just past the end; negative
    rows = torch.arange(B, device=far.device)

    def dense_without_second_row(c):
        lw = torch.zeros(B, L, D, heads * size, device="cuda")
        uw = torch.zeros_like(lw)
        lw[rows, cq.positions[:, 0]] = c._lw[:, 0]
        uw[rows, cq.positions[:, 0]] = c._uw[:, 0]
        return Bounds(c.args, c.p, c.eps, lw=lw, lb=c._lb, uw=uw, ub=c._ub)
    dq, dk = dense_without_second_row(cq), dense_without_second_row(ck)
    (x_l, _), (y_l, y_u) = dq.concretize(), dk.concretize()
    got = ops.attention_scores_compact((cq._lw, cq._lb, cq._uw, cq._ub), (ck._lw, ck._lb, ck._uw, ck._ub),
                                       x_l, y_l, y_u, far, heads)
    torch.cuda.synchronize()
    want = dq.attention_scores(dk, heads)
    tw, tb = score_terms(dq, dk, heads)
    for name, x, terms in zip(("lw", "lb", "uw", "ub"), got, (tw, tb, tw, tb)):
        y = getattr(want, name)
        tol = ATOL + RTOL * y.double().abs().cpu() + 2 * KAPPA * U32 * terms
        over = float(((x.double() - y.double()).abs().cpu() / tol).max())
        assert over <= 1.0, f"scores.{name} with a position outside the sentence: {over:.2f} of the accumulation-aware bar"
    # the context with a compact value operand: same convention
    g = torch.Generator().manual_seed(53)
    lw = 0.3 * torch.randn(B * heads, L, D, L, generator=g); lb = torch.rand(B * heads, L, L, generator=g)
    probs = Bounds(cq.args, 2.0, 0.1, lw=lw.cuda(), lb=lb.cuda(), uw=(lw + 0.01).cuda(), ub=(lb + 0.1).cuda())
    gotc = ops.attention_context_compact((probs.lw, probs.lb, probs.uw, probs.ub), (ck._lw, ck._lb, ck._uw, ck._ub),
                                         y_l, y_u, far, 2.0, 0.1)
    torch.cuda.synchronize()
    wantc = probs.attention_context(dk)
    cw, cb = context_terms(probs, dk, heads)
    for name, x, terms in zip(("lw", "lb", "uw", "ub"), gotc, (cw, cb, cw, cb)):
        y = getattr(wantc, name)
        tol = ATOL + RTOL * y.double().abs().cpu() + 2 * KAPPA * U32 * terms
        over = float(((x.double() - y.double()).abs().cpu() / tol).max())
        assert over <= 1.0, f"context.{name} with a position outside the sentence: {over:.2f} of the accumulation-aware bar"


@pytest.mark.parametrize("shape", [(2, 5, 12, 24, 16), (1, 32, 256, 256, 256), (3, 7, 33, 20, 7)])
def test_row_count_entry_points_on_an_ordinary_object(shape):
    """faith_matmul_rows_verification / _group_rows_ with rows_w = rows_b * dim_in: the ordinary entry points' bits."""
    from faith_amd import ops
    B, L, D, H, N = shape
    g = torch.Generator().manual_seed(sum(shape))
    lw = torch.randn(B, L, D, H, generator=g).cuda(); uw = (lw + 0.05 * torch.rand(B, L, D, H, generator=g).cuda())
    lb = torch.randn(B, L, H, generator=g).cuda(); ub = lb + 0.3 * torch.rand(B, L, H, generator=g).cuda()
    layers = [layer_of(g, H, N), layer_of(g, H, N, False), layer_of(g, H, N)]
    W, b = [x.weight for x in layers], [x.bias for x in layers]
    for got, want in zip(ops.linear_rows(lw, lb, uw, ub, W[:1], b[:1]), [ops.linear(lw, lb, uw, ub, W[0], b[0])]):
        assert all(torch.equal(x, y) for x, y in zip(got, want))
    for got, want in zip(ops.linear_rows(lw, lb, uw, ub, W, b), ops.linear_group(lw, lb, uw, ub, W, b)):
        assert all(torch.equal(x, y) for x, y in zip(got, want))
    with pytest.raises(ValueError):
        ops.linear_rows(lw, lb[..., :-1].contiguous(), uw, ub[..., :-1].contiguous(), W, b)


def test_compact_object_matches_the_oracle():
    """Against the CPU oracle directly (not only against the HIP path's own dense object)."""
    g = torch.Generator().manual_seed(8)
    c, d = compact_and_dense(9, B=2, P=2, D=20, H=32, L=6)
    norm = SimpleNamespace(weight=1.0 + 0.2 * torch.randn(32, generator=g), bias=0.1 * torch.randn(32, generator=g))
    layer = SimpleNamespace(weight=torch.randn(48, 32, generator=g) / 32 ** 0.5, bias=0.1 * torch.randn(48, generator=g))
    o = OracleBounds(2.0, 0.1, d.lw.cpu(), d.lb.cpu(), d.uw.cpu(), d.ub.cpu())
    want = o.layer_norm(norm, "no_var").dense(layer)
    got = c.layer_norm(to_device(norm, "cuda"), "no_var").dense(to_device(layer, "cuda"))
    at_the_bar(got, want, "layer norm + dense against the oracle")


def sentence(emb, length):
    """The test network's embeddings at another length (6 positions: the scores of compact operands fall back to
    the dense kernel; a multiple of 4: they take the compact one)."""
    if length == emb.shape[1]:
        return emb
    return torch.randn(1, length, emb.shape[2], generator=torch.Generator().manual_seed(length))


@pytest.mark.parametrize("length", [LENGTH, 8])
@pytest.mark.parametrize("mode", ["no_var", "standard"])
def test_propagation_from_the_compact_input_gives_the_ordinary_ones_margins(mode, length):
    from faith_amd import Bounds, BoundsMaker, CompactBounds
    layer, embed_norm, pooler, classifier, emb = build(7, mode)
    emb = sentence(emb, length)
    gparts = tuple(to_device(x, "cuda") for x in (layer, embed_norm, pooler, classifier))
    ge = emb.cuda()
    plain = lambda p_, e_, lw, lb, uw, ub: Bounds(None, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    maker = BoundsMaker(compact_from=0)
    assert isinstance(F.bound_input(maker, ge, 2, 0.02, 1, 2.0), CompactBounds)
    # an object this small is written out at once unless the maker is told otherwise
    assert isinstance(F.bound_input(BoundsMaker(), ge, 2, 0.02, 1, 2.0), Bounds)
    assert isinstance(F.bound_inputs(BoundsMaker(compact_from=4 * 3 * length * HIDDEN * HIDDEN), ge, [1, 2, 3], [0.1] * 3), CompactBounds)
    assert isinstance(F.bound_inputs(BoundsMaker(compact_from=4 * 3 * length * HIDDEN * HIDDEN + 1), ge, [1, 2, 3], [0.1] * 3), Bounds)
    assert isinstance(F.bound_input(maker, ge, 2, 0.02, 1, 2.0, ibp=True), Bounds)

    def run(make):
        x = F.bound_input(make, ge, 2, 0.02, 1, 2.0, gparts[1], mode)
        _, _, out = F.bound_layer(x, gparts[0], mode, "relu")
        return out, F.bound_classifier(F.bound_pooling(out, gparts[2], make), gparts[3], 0)
    out_c, (safe_c, l_c, u_c) = run(maker)
    out_d, (safe_d, l_d, u_d) = run(plain)
    # the same operators on the same values from the first attention scores on; before them the affine
    # kernel rounds in its own order for the smaller problem
    for name in ("lw", "lb", "uw", "ub"):
        a, b = getattr(out_c, name).double(), getattr(out_d, name).double()
        assert float((a - b).abs().max()) <= 1e-5 * max(float(b.abs().max()), 1.0), name
    assert safe_c == safe_d
    assert float((l_c - l_d).abs().max()) <= 1e-4 and float((u_c - u_d).abs().max()) <= 1e-4
    # and the oracle's
    omake = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub)
    x = F.bound_input(omake, emb, 2, 0.02, 1, 2.0, embed_norm, mode)
    _, _, o_out = F.bound_layer(x, layer, mode, "relu")
    for name in ("lw", "lb", "uw", "ub"):
        a, b = getattr(out_c, name).double().cpu(), getattr(o_out, name).double()
        assert float((a - b).abs().max()) <= 2e-4 * max(float(b.abs().max()), 1.0), name


@pytest.mark.parametrize("mode", ["no_var", "standard"])
def test_two_perturbed_words_from_the_compact_input(mode):
    from faith_amd import Bounds, BoundsMaker
    net, emb = two_layer_network(21, mode)
    two_words = SimpleNamespace(perturbed_words=2)
    gnet = SimpleNamespace(**{k: (to_device(v, "cuda") if k in ("embedding_norm", "pooler", "classifier") else v)
                              for k, v in vars(net).items()})
    gnet.layers = [to_device(x, "cuda") for x in net.layers]
    ge = emb.cuda()

    def margins(make):
        x = F.bound_input(make, ge, [1, 4], 0.01, 2, 2.0, gnet.embedding_norm, gnet.layer_norm)
        pooled = F.bound_pooling(F.propagate(x, gnet), gnet.pooler, make)
        return F.bound_classifier(pooled, gnet.classifier, 0)
    _, l_c, u_c = margins(BoundsMaker(two_words, compact_from=0))
    _, l_d, u_d = margins(lambda p_, e_, lw, lb, uw, ub: Bounds(two_words, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub))
    assert float((l_c - l_d).abs().max()) <= 1e-4 and float((u_c - u_d).abs().max()) <= 1e-4
    omake = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub, words=2)
    x = F.bound_input(omake, emb, [1, 4], 0.01, 2, 2.0, net.embedding_norm, net.layer_norm)
    _, ol, ou = F.bound_classifier(F.bound_pooling(F.propagate(x, net), net.pooler, omake), net.classifier, 0)
    assert float((l_c.cpu() - ol).abs().max()) <= 2e-3 and float((u_c.cpu() - ou).abs().max()) <= 2e-3


@pytest.mark.parametrize("length", [LENGTH, 8])
def test_search_from_the_compact_input_finds_the_same_radii(length):
    """One at a time, batched, with persistent buffers and from a captured graph: the radii of the search on the
    ordinary object (a verdict within rounding of its threshold may fall either way: one step)."""
    from faith_amd import Bounds, BoundsMaker, ops
    layer, embed_norm, pooler, classifier, emb = build(11, "no_var")
    emb = sentence(emb, length)
    parts = (layer, embed_norm, pooler, classifier)
    _, margin = true_layer(emb.double(), layer, embed_norm, "no_var", pooler, classifier)
    label = 0 if float(margin[0, 0]) > 0 else 1
    gnet = network_of(tuple(to_device(x, "cuda") for x in parts), "no_var")
    ge = emb.cuda()
    positions, max_eps, iters = [1, 2, 3, 4], 0.5, 6
    step = max_eps / 2 ** iters
    plain = lambda p_, e_, lw, lb, uw, ub: Bounds(None, p_, e_, lw=lw, lb=lb, uw=uw, ub=ub)
    maker = BoundsMaker(compact_from=0)
    want = F.certified_radii(plain, gnet, ge, positions, label, 2.0, max_eps, iters)
    one = F.certified_radii(maker, gnet, ge, positions, label, 2.0, max_eps, iters)
    lock = F.certified_radii(maker, gnet, ge, positions, label, 2.0, max_eps, iters, batched=True)
    ws = ops.Workspace()
    F.verify_safety_batch(maker, gnet, ge, positions, [0.01] * 4, label, 2.0, buffers=ws)
    first = ws.allocations
    kept = F.certified_radii(maker, gnet, ge, positions, label, 2.0, max_eps, iters, batched=True, buffers=ws)
    assert ws.allocations == first, "a repeated propagation allocated result buffers"
    graph = F.certified_radii(maker, gnet, ge, positions, label, 2.0, max_eps, iters, captured=True)
    print(f"[case] radii ordinary {want} compact {one} batched {lock} buffers {kept} graph {graph}", flush=True)
    assert lock == kept == graph
    for a, b, c in zip(want, one, lock):
        assert abs(a - b) <= step + 1e-12 and abs(a - c) <= step + 1e-12


@pytest.mark.parametrize("length", [LENGTH, 8])
def test_captured_graph_on_the_compact_input_follows_new_positions_and_radii(length):
    from faith_amd import BoundsMaker
    layer, embed_norm, pooler, classifier, emb = build(11, "standard")
    emb = sentence(emb, length)
    parts = (layer, embed_norm, pooler, classifier)
    _, margin = true_layer(emb.double(), layer, embed_norm, "standard", pooler, classifier)
    label = 0 if float(margin[0, 0]) > 0 else 1
    gnet = network_of(tuple(to_device(x, "cuda") for x in parts), "standard")
    ge = emb.cuda()
    maker = BoundsMaker(compact_from=0)
    cap = F.CapturedVerifier(maker, gnet, ge, 4, label, 2.0)
    queries = [([1, 2, 3, 4], [0.004, 0.004, 0.004, 0.004]), ([4, 3, 2, 1], [0.001, 0.02, 0.008, 0.3]),
               ([1, 1, 1, 1], [0.0005, 0.009, 0.0078125, 1.0]), ([2, 4, 2, 4], [0.012, 0.012, 0.25, 0.004]),
               ([1, 2, 3, 4], [0.004, 0.004, 0.004, 0.004])]
    seen = set()
    for idx, radii in queries:
        print(f"[case] captured replay on the compact input, positions {idx} radii {radii}", flush=True)
        got = cap(idx, radii)
        want = F.verify_safety_batch(maker, gnet, ge, idx, radii, label, 2.0)      # eager work between replays
        torch.cuda.synchronize()
        assert got == want, (idx, radii, got, want)
        seen.update(got)
    assert len(seen) == 2 or length != LENGTH                 # at the test network's own length both verdicts occur
    # a maker that would write a propagation this small out keeps the compact form for the graph, where the extra
    # launches cost the device's time only; one query per replay, against the written-out eager propagation
    default, plain = BoundsMaker(), (lambda p_, e_, lw, lb, uw, ub: BoundsMaker()(p_, e_, lw, lb, uw, ub))
    assert not default.compact_pays(1, length, HIDDEN, HIDDEN) and default.compact_pays(1, length, HIDDEN, HIDDEN, captured=True)
    assert not BoundsMaker(SimpleNamespace(method="ibp")).compact_pays(1, length, HIDDEN, HIDDEN, captured=True)
    one = F.CapturedVerifier(default, gnet, ge, 1, label, 2.0)
    assert one.at is not None
    for idx, radius in ((1, 0.004), (3, 0.3), (2, 0.0005), (1, 0.004)):
        got = one([idx], [radius])
        want = F.verify_safety(plain, gnet, ge, idx, radius, label, 2.0)
        torch.cuda.synchronize()
        assert got == [bool(want)], (idx, radius, got, want)


def test_rows_of_a_compact_object_are_gathered_and_put_back_by_the_library():
    """faith_rows_gather / faith_rows_put against indexing on the CPU, a pair of tensors a launch; a position
    outside the sentence reads as zero and replaces nothing."""
    from faith_amd import ops
    g = torch.Generator().manual_seed(140)
    B, L, P, H = 3, 7, 2, 20
    a, b = torch.randn(B, L, H, generator=g), torch.randn(B, L, H, generator=g)
    ra, rb = torch.randn(B, P, H, generator=g), torch.randn(B, P, H, generator=g)
    positions = torch.stack([torch.randperm(L, generator=g)[:P] for _ in range(B)])
    positions[1, 0] = L + 2
    ga, gb = ops.gather_positions(a.cuda(), b.cuda(), positions.cuda())
    pa, pb = ops.put_positions(a.cuda(), b.cuda(), positions.cuda(), ra.cuda(), rb.cuda())
    torch.cuda.synchronize()
    ea, eb, fa, fb = torch.zeros(B, P, H), torch.zeros(B, P, H), a.clone(), b.clone()
    for i in range(B):
        for j in range(P):
            l = int(positions[i, j])
            if 0 <= l < L:
                ea[i, j], eb[i, j] = a[i, l], b[i, l]
                fa[i, l], fb[i, l] = ra[i, j], rb[i, j]
    assert torch.equal(ga.cpu(), ea) and torch.equal(gb.cpu(), eb)
    assert torch.equal(pa.cpu(), fa) and torch.equal(pb.cpu(), fb)


@pytest.mark.parametrize("shape", [(3, 2, 7, 5, 8), (2, 1, 4, 3, 6), (1, 3, 9, 2, 5)])
def test_rows_are_spread_into_the_written_out_object_by_the_library(shape):
    """faith_rows_spread against a fill and an indexed copy on the CPU (16-byte and 4-byte rows); a position outside
    the sentence names no row."""
    from faith_amd import ops
    B, P, L, D, H = shape
    g = torch.Generator().manual_seed(141)
    t = torch.randn(B, P, D, H, generator=g)
    positions = torch.stack([torch.randperm(L, generator=g)[:P] for _ in range(B)])
    if B > 1:
        positions[1, 0] = L + 3
    got = ops.spread_positions(t.cuda(), positions.cuda(), L)
    const = ops.spread_positions(t[:, :, 0].contiguous().cuda(), positions.cuda(), L)      # [B, P, H] rows
    torch.cuda.synchronize()
    want = torch.zeros(B, L, D, H)
    for i in range(B):
        for j in range(P):
            if 0 <= int(positions[i, j]) < L:
                want[i, int(positions[i, j])] = t[i, j]
    assert torch.equal(got.cpu(), want) and torch.equal(const.cpu(), want[:, :, 0])


@pytest.mark.parametrize("shape", [(1, 1, 64, 4, 64, 32), (2, 2, 256, 4, 64, 32), (3, 1, 128, 2, 32, 32), (1, 2, 64, 1, 32, 64)])
@pytest.mark.parametrize("p", [2.0, float("inf"), 1.0])
def test_rows_of_the_perturbed_positions_on_the_matrix_unit(shape, p):
    """Where length and dim_in are multiples of 32 and a head is 32 or 64 wide the score rows of the perturbed
    positions come from the matrix-unit kernel; knob 4 of the dot product's variant sends them to the vector-ALU
    kernel.  Both sum the same head_size products, in different orders."""
    from faith_amd import _lib
    B, P, D, heads, size, L = shape
    words = 2 if P == 2 else 1
    print(f"[case] compact scores, matrix unit against vector ALU B={B} P={P} D={D} heads={heads} size={size} L={L} p={p}", flush=True)
    cq, dq = compact_and_dense(51, B, P, D, heads * size, L, words=words, p=p)
    ck, dk = compact_and_dense(52, B, P, D, heads * size, L, words=words, p=p, positions=cq.positions)
    got = cq.attention_scores(ck, heads)
    _lib.call("faith_tune_set", 2, 4)
    try:
        want = cq.attention_scores(ck, heads)
        torch.cuda.synchronize()
    finally:
        _lib.call("faith_tune_set", 2, 0)
    tw, tb = score_terms(dq, dk, heads)
    for name, terms in (("lw", tw), ("uw", tw), ("lb", tb), ("ub", tb)):
        x, y = getattr(got, name), getattr(want, name)
        tol = ATOL + RTOL * y.double().abs().cpu() + 2 * KAPPA * U32 * terms
        over = float(((x.double() - y.double()).abs().cpu() / tol).max())
        assert over <= 1.0, f"scores.{name}: {over:.2f} of the accumulation-aware bar"
    # the constants and the rows without coefficients do not go through the matrix unit: same bits
    assert torch.equal(got.lb, want.lb) and torch.equal(got.ub, want.ub)
    assert torch.equal(got.lw == 0, want.lw == 0) and torch.equal(got.uw == 0, want.uw == 0)


@pytest.mark.parametrize("shape", [(3, 2, 10, 24, 5, 1), (2, 2, 64, 100, 9, 2), (1, 1, 256, 256, 32, 1), (4, 3, 33, 70, 6, 3),
                                   (2, 1, 7, 130, 300, 1)])
@pytest.mark.parametrize("p", [2.0, float("inf"), 1.0, 3.0])
def test_concrete_interval_of_a_compact_object_in_one_launch(shape, p):
    """faith_concretize_rows against its three-launch equivalent (constants gathered, faith_concretize on the rows,
    results put back) and against faith_concretize on the object with the zeros written out."""
    from faith_amd import ops
    B, P, D, H, L, words = shape
    print(f"[case] concretize rows B={B} P={P} D={D} H={H} L={L} words={words} p={p}", flush=True)
    c, d = compact_and_dense(61, B, P, D, H, L, words=words, p=p)
    l, u = ops.concretize_positions(c._lw, c._lb, c._uw, c._ub, c.positions, p, 0.1, words)
    rows_lb, rows_ub = ops.gather_positions(c._lb, c._ub, c.positions)
    rl, ru = ops.concretize(c._lw, rows_lb, c._uw, rows_ub, p, 0.1, words)
    l3, u3 = ops.put_positions(c._lb, c._ub, c.positions, rl, ru)
    dl, du = ops.concretize(d.lw, d.lb, d.uw, d.ub, p, 0.1, words)
    torch.cuda.synchronize()
    has = torch.zeros(B, L, dtype=torch.bool)
    has[torch.arange(B)[:, None], c.positions.cpu()] = True
    # no coefficients: the constants themselves
    assert torch.equal(l.cpu()[~has], c._lb.cpu()[~has]) and torch.equal(u.cpu()[~has], c._ub.cpu()[~has])
    for name, x, ys in (("l", l, (l3, dl)), ("u", u, (u3, du))):
        for y in ys:
            err, of_bar = worst(x, y)
            assert of_bar <= 1.0, f"{name}: max err {err:.3g}, {of_bar:.2f} of the bar"
    assert bool((l <= u).all())


def test_concrete_interval_of_a_compact_object_skips_a_position_outside_the_sentence():
    from faith_amd import ops
    B, P, D, H, L = 2, 2, 12, 40, 6
    g = torch.Generator().manual_seed(62)
    positions = torch.tensor([[1, L + 3], [-1, 4]])
    lw = torch.randn(B, P, D, H, generator=g)
    uw = lw + 0.05 * torch.rand(B, P, D, H, generator=g)
    lb = torch.randn(B, L, H, generator=g)
    ub = lb + 0.3 * torch.rand(B, L, H, generator=g)
    l, u = ops.concretize_positions(lw.cuda(), lb.cuda(), uw.cuda(), ub.cuda(), positions.cuda(), 2.0, 0.1, 1)
    torch.cuda.synchronize()
    want_l, want_u = lb.clone(), ub.clone()
    for b, j, at in ((0, 0, 1), (1, 1, 4)):
        want_l[b, at] = lb[b, at] - 0.1 * lw[b, j].double().norm(dim=0).float()
        want_u[b, at] = ub[b, at] + 0.1 * uw[b, j].double().norm(dim=0).float()
    for x, y in ((l, want_l), (u, want_u)):
        assert worst(x.cpu(), y)[1] <= 1.0
    keep = torch.ones(B, L, dtype=torch.bool); keep[0, 1] = keep[1, 4] = False
    assert torch.equal(l.cpu()[keep], lb[keep]) and torch.equal(u.cpu()[keep], ub[keep])
    with pytest.raises(ValueError):
        ops.concretize_positions(lw.cuda(), lb.cuda(), uw.cuda(), ub.cuda(), positions.int().cuda(), 2.0, 0.1, 1)
    with pytest.raises(Exception, match="words"):
        ops.concretize_positions(lw.cuda(), lb.cuda(), uw.cuda(), ub.cuda(), positions.cuda(), 2.0, 0.1, 5)
