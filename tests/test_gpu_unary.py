"""HIP exp / reciprocal / sqr / sqrt relaxations against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import rand_bounds, close, worst
from tests.parity import compare_unary

pytestmark = pytest.mark.gpu
INF = float("inf")
PS = [1.0, 2.0, INF, 3.0, 1.5]     # 3.0 and 1.5: dual exponents 1.5 and 3, the general-norm kernels
KINDS = ["exp", "reciprocal", "sqr", "sqrt"]


def make_input(kind, g, L, D, H, ordered=True):
    x = rand_bounds(g, 1, L, D, H, ordered=ordered, sw=0.05, sb=1.5, gap_w=0.01, gap_b=0.5)
    if kind in ("reciprocal", "sqrt"):          # strictly positive pre-activations for every p
        off = 1.0 + 0.05 * D * 0.06             # > eps * sum |lw| (q = 1, the largest norm)
        x = O.LinearBounds(x.lw, x.lb.abs() + off, x.uw, x.lb.abs() + off + (x.ub - x.lb))
    return x


def run(kind, x, p, eps, words, layout="natural"):
    from faith_amd import ops
    lw, lb, uw, ub = (t.cuda().contiguous() for t in x.tensors())
    fn = getattr(ops, kind)
    if layout == "natural":
        return fn(lw, lb, uw, ub, p, eps, words, return_interval=True)
    out = fn(lw.transpose(2, 3).contiguous(), lb, uw.transpose(2, 3).contiguous(), ub, p, eps, words,
             layout=ops.LAYOUT_TRANSPOSED, return_interval=True)
    return (out[0].transpose(2, 3), out[1], out[2].transpose(2, 3), out[3], out[4], out[5])


def check(kind, x, p, eps, words, layout="natural"):
    print(f"[case] {kind} shape={tuple(x.lw.shape)} p={p} eps={eps} words={words} layout={layout}", flush=True)
    got = run(kind, x, p, eps, words, layout)
    torch.cuda.synchronize()
    exp = getattr(O, kind)(x, p, eps, words)
    el, eu = O.concretize(x, p, eps, words)
    rep = compare_unary(kind, x, got[:4], exp.tensors(), got[4].cpu(), got[5].cpu(), el, eu)
    if rep["inherited_from_interval"]:
        print("   ", rep, flush=True)
    return rep


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("layout", ["natural", "transposed"])
def test_unary_shapes(kind, p, layout):
    g = torch.Generator().manual_seed(51)
    for (L, D, H, words) in [(4, 64, 64, 1), (3, 128, 192, 2), (2, 256, 64, 2), (1, 1100, 72, 1), (2, 48, 37, 3)]:
        check(kind, make_input(kind, g, L, D, H), p, 0.05, words, layout)


@pytest.mark.parametrize("kind", KINDS)
def test_unary_unordered_coefficients(kind):
    """lw and uw drawn independently, as the reference's op test draws them."""
    g = torch.Generator().manual_seed(52)
    check(kind, make_input(kind, g, 4, 64, 128, ordered=False), 2.0, 0.05, 1)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("p", [1.0, 2.0, float("inf")])
def test_unary_thread_shape_for_hbm_streams(kind, p):
    """Objects whose traffic is far beyond the memory-side cache take the register-resident kernel's sixteen-wavefront
    thread shape (tuning knob 7 forces it on a small object): against the oracle like every other shape."""
    from faith_amd import _lib
    g = torch.Generator().manual_seed(54)
    x = make_input(kind, g, 3, 256, 96)
    _lib.call("faith_tune_set", 0, 7)
    try:
        check(kind, x, p, 0.05, 2)
    finally:
        _lib.call("faith_tune_set", 0, 0)


def test_exp_above_the_cap():
    """Pre-activations beyond 12: the reference continues exp by its tangent (Bounds.py:984-989)."""
    g = torch.Generator().manual_seed(53)
    x = rand_bounds(g, 1, 2, 16, 64, sw=0.05, sb=1.0, gap_w=0.01, gap_b=0.5)
    x = O.LinearBounds(x.lw, x.lb + 12.0, x.uw, x.ub + 12.0)       # straddles the cap
    check("exp", x, 2.0, 0.05, 1)


@pytest.mark.parametrize("kind", KINDS)
def test_unary_config1_shape(kind):
    """Shape of benchmark configuration 1 at a quarter of its length."""
    from faith_amd.workloads import make_config
    c = make_config(1, scale=0.25)
    x = O.LinearBounds(c["x"]["lw"], c["x"]["lb"], c["x"]["uw"], c["x"]["ub"])
    if kind in ("reciprocal", "sqrt"):
        x = O.LinearBounds(x.lw, x.lb.abs() + 2.0, x.uw, x.lb.abs() + 2.0 + (x.ub - x.lb))
    for p in PS:
        check(kind, x, p, c["eps"], c["words"])


def test_bounds_class_unary_methods_and_assertions():
    from faith_amd import Bounds
    g = torch.Generator().manual_seed(54)
    x = make_input("sqrt", g, 2, 32, 64)
    b = Bounds(None, 2.0, 0.05, lw=x.lw.cuda(), lb=x.lb.cuda(), uw=x.uw.cuda(), ub=x.ub.cuda())
    for kind in KINDS:
        y = getattr(b, kind)()
        e = getattr(O, kind)(x, 2.0, 0.05)
        assert close(y.lw, e.lw) and close(y.ub, e.ub), kind
    neg = Bounds(None, 2.0, 0.05, lw=x.lw.cuda(), lb=(x.lb - 5).cuda(), uw=x.uw.cuda(), ub=(x.ub - 5).cuda())
    with pytest.raises(AssertionError):
        neg.sqrt()
    with pytest.raises(AssertionError):
        neg.reciprocal()
