"""Tensors that are 4-byte but not 16-byte aligned (a view that starts one float into its storage).

The fast kernels move 16 bytes per lane and are chosen only when every pointer allows it; a caller
that hands over such a view gets the kernels that move 4 bytes per lane.  The result must not
depend on that: every operator here is run on shifted copies of its inputs (and, where the wrapper
takes them, shifted outputs) and compared with the run on aligned tensors, to the parity bar."""
import pytest
import torch

from faith_amd import ops
from tests.helpers import rand_bounds, close, worst

pytestmark = pytest.mark.gpu
INF = float("inf")


def shifted(t):
    """A contiguous copy of t (on the GPU) whose first element sits 4 bytes past a 16-byte boundary."""
    buf = torch.empty(t.numel() + 1, device="cuda", dtype=torch.float32)
    v = buf[1:].view(t.shape)
    v.copy_(t)
    assert v.data_ptr() % 16 == 4 and v.is_contiguous()
    return v


def both(x):
    """(aligned, shifted) GPU copies of the four tensors of a bound object."""
    return tuple(t.cuda() for t in x.tensors()), tuple(shifted(t) for t in x.tensors())


def same(got, exp, what, rtol=1e-5, atol=1e-6):
    for i, (a, b) in enumerate(zip(got, exp)):
        assert a.shape == b.shape
        assert close(a, b, rtol=rtol, atol=atol), f"{what} output {i}: {worst(a, b)}"


@pytest.mark.parametrize("layout", ["natural", "transposed"])
@pytest.mark.parametrize("op", ["concretize", "relu", "tanh", "exp", "sqr"])
@pytest.mark.parametrize("shape", [(3, 64, 64), (2, 256, 32), (1, 300, 128)])
def test_relaxations(op, layout, shape):
    L, D, H = shape
    g = torch.Generator().manual_seed(80)
    lay = ops.LAYOUT_TRANSPOSED if layout == "transposed" else ops.LAYOUT_NATURAL
    x = rand_bounds_transposed(g, L, D, H) if layout == "transposed" else rand_bounds(g, 1, L, D, H, sw=0.2, gap_w=0.02)
    al, sh = both(x)
    print(f"[case] unaligned {op} {layout} {shape}", flush=True)
    if op == "concretize":
        same(ops.concretize(*sh, 2.0, 0.05, 2, lay), ops.concretize(*al, 2.0, 0.05, 2, lay), op)
    else:
        fn = getattr(ops, op)
        same(fn(*sh, 2.0, 0.05, 2, lay, True), fn(*al, 2.0, 0.05, 2, lay, True), op)


def rand_bounds_transposed(g, L, D, H):
    """lw [1, L, H, D], lb [1, L, H]."""
    from oracle.bounds_oracle import LinearBounds
    lw = (torch.rand(1, L, H, D, generator=g) - 0.5) * 0.4
    uw = lw + torch.rand(1, L, H, D, generator=g) * 0.02
    lb = torch.rand(1, L, H, generator=g) * 2 - 1
    ub = lb + torch.rand(1, L, H, generator=g) * 0.3
    return LinearBounds(lw, lb, uw, ub)


def test_relaxation_into_unaligned_outputs():
    g = torch.Generator().manual_seed(81)
    x = rand_bounds(g, 1, 3, 256, 64, sw=0.2, gap_w=0.02)
    al, _ = both(x)
    exp = ops.tanh(*al, 2.0, 0.05)
    out = tuple(shifted(torch.zeros_like(t)) for t in x.tensors())
    got = ops.tanh(*al, 2.0, 0.05, out=out)
    assert got[0].data_ptr() == out[0].data_ptr()
    same(got, exp, "tanh into shifted outputs")


@pytest.mark.parametrize("shape", [(2, 64, 64), (1, 256, 32), (2, 40, 100)])
def test_whole_object_operators_and_product(shape):
    L, D, H = shape
    g = torch.Generator().manual_seed(82)
    x, y = rand_bounds(g, 1, L, D, H, ordered=False, sw=0.1), rand_bounds(g, 1, L, D, H, ordered=False, sw=0.1)
    (xa, xs), (ya, ys) = both(x), both(y)
    scale = torch.randn(H, generator=g)
    shift = torch.randn(H, generator=g)
    sa, ss, ha, hs = scale.cuda(), shifted(scale), shift.cuda(), shifted(shift)
    print(f"[case] unaligned whole-object operators {shape}", flush=True)
    same(ops.affine(xs, scale=ss, other=ys, shift=hs), ops.affine(xa, scale=sa, other=ya, shift=ha), "affine")
    same(ops.rowsum(*xs), ops.rowsum(*xa), "row sum")
    same(ops.layer_norm(*xs, ss, hs, other=ys), ops.layer_norm(*xa, sa, ha, other=ya), "layer norm")
    same(ops.multiply(xs, ys, 2.0, 0.05, 1), ops.multiply(xa, ya, 2.0, 0.05, 1), "product", atol=4e-6)


def test_softmax_of_unaligned_bounds():
    """16-byte loads are out, so are the slab shapes that need them: Bounds.softmax composes when the
    one-launch kernel declines."""
    from types import SimpleNamespace
    from faith_amd import Bounds
    g = torch.Generator().manual_seed(83)
    for (L, D, H) in [(3, 64, 32), (2, 32, 128)]:
        x = rand_bounds(g, 1, L, D, H, sw=0.05, sb=1.0, gap_w=0.005, gap_b=0.1)
        al, sh = both(x)
        a = Bounds(SimpleNamespace(perturbed_words=1), 2.0, 0.05, lw=al[0], lb=al[1], uw=al[2], ub=al[3]).softmax()
        s = Bounds(SimpleNamespace(perturbed_words=1), 2.0, 0.05, lw=sh[0], lb=sh[1], uw=sh[2], ub=sh[3]).softmax()
        same((s.lw, s.lb, s.uw, s.ub), (a.lw, a.lb, a.uw, a.ub), f"softmax {L, D, H}", rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("shape", [(4, 32, 64, 64), (3, 50, 36, 72), (1, 1, 256, 256)])
def test_linear(shape):
    L, D, K, N = shape
    g = torch.Generator().manual_seed(84)
    x = rand_bounds(g, 1, L, D, K, ordered=False, sw=0.5)
    W = torch.randn(N, K, generator=g) / K ** 0.5
    bias = torch.randn(N, generator=g)
    al, sh = both(x)
    print(f"[case] unaligned linear {shape}", flush=True)
    exp = ops.linear(*al, W.cuda(), bias.cuda())
    # coefficient rows, weight, or only the outputs off the 16-byte grid
    same(ops.linear(*sh, W.cuda(), bias.cuda()), exp, "linear, shifted x", atol=4e-6)
    same(ops.linear(*al, shifted(W), shifted(bias)), exp, "linear, shifted W", atol=4e-6)
    out = (shifted(torch.zeros(1, L, D, N)), shifted(torch.zeros(1, L, N)), shifted(torch.zeros(1, L, D, N)),
           shifted(torch.zeros(1, L, N)))
    same(ops.linear(*al, W.cuda(), bias.cuda(), out=out), exp, "linear, shifted outputs", atol=4e-6)


@pytest.mark.parametrize("shape", [(2, 32, 32, 16, 32), (1, 128, 64, 8, 64), (2, 20, 24, 12, 16)])
def test_dot_products(shape):
    B, Lx, Ly, D, d = shape
    g = torch.Generator().manual_seed(85)
    x = rand_bounds(g, B, Lx, D, d, ordered=False, sw=0.3)
    y = rand_bounds(g, B, Ly, D, d, ordered=False, sw=0.3)
    (xa, xs), (ya, ys) = both(x), both(y)
    print(f"[case] unaligned dot products {shape}", flush=True)
    same(ops.dot_product_qk(xs, ys, 2.0, 0.05), ops.dot_product_qk(xa, ya, 2.0, 0.05), "scores", atol=1e-5)
    same(ops.dot_product_qk(xs, ya, 2.0, 0.05), ops.dot_product_qk(xa, ya, 2.0, 0.05), "scores, only x shifted", atol=1e-5)
    probs = rand_bounds(g, B, Lx, D, Ly, ordered=False, sw=0.1)
    pa, ps = both(probs)
    same(ops.dot_product_v(ps, ys, 2.0, 0.05), ops.dot_product_v(pa, ya, 2.0, 0.05), "context", atol=1e-5)


def test_attention_heads_in_place():
    heads, L, D, size = 4, 32, 16, 32
    g = torch.Generator().manual_seed(86)
    q = rand_bounds(g, 1, L, D, heads * size, ordered=False, sw=0.3)
    k = rand_bounds(g, 1, L, D, heads * size, ordered=False, sw=0.3)
    (qa, qs), (ka, ks) = both(q), both(k)
    exp = ops.attention_scores(qa, ka, heads, 2.0, 0.05)
    same(ops.attention_scores(qs, ks, heads, 2.0, 0.05), exp, "attention scores", atol=1e-5)
    v = rand_bounds(g, 1, L, D, heads * size, ordered=False, sw=0.3)
    va, vs = both(v)
    probs = tuple(t.contiguous() for t in exp)
    same(ops.attention_context(tuple(shifted(t) for t in probs), vs, 2.0, 0.05),
         ops.attention_context(probs, va, 2.0, 0.05), "attention context", atol=1e-5)


def test_convolution():
    g = torch.Generator().manual_seed(87)
    D, C, HW, CO = 6, 8, 12, 16
    lw = torch.randn(1, D, C, HW, HW, generator=g) * 0.1
    uw = lw + torch.rand(1, D, C, HW, HW, generator=g) * 0.01
    lb = torch.randn(1, C, HW, HW, generator=g)
    ub = lb + torch.rand(1, C, HW, HW, generator=g) * 0.1
    W = torch.randn(CO, C, 3, 3, generator=g) * (2 / (9 * C)) ** 0.5
    bias = torch.randn(CO, generator=g) * 0.01
    exp = ops.conv2d(lw.cuda(), lb.cuda(), uw.cuda(), ub.cuda(), W.cuda(), bias.cuda(), 1, 1)
    same(ops.conv2d(shifted(lw), shifted(lb), shifted(uw), shifted(ub), W.cuda(), bias.cuda(), 1, 1), exp,
         "convolution, shifted x", atol=4e-6)
    same(ops.conv2d(lw.cuda(), lb.cuda(), uw.cuda(), ub.cuda(), shifted(W), shifted(bias), 1, 1), exp,
         "convolution, shifted W", atol=4e-6)


def test_interval_operators():
    g = torch.Generator().manual_seed(88)
    l = torch.rand(3, 5, 7, generator=g) + 0.1
    u = l + torch.rand(3, 5, 7, generator=g)
    for kind in ("relu", "tanh", "exp", "reciprocal", "sqr", "sqrt"):
        same(ops.interval_unary(kind, shifted(l), shifted(u)), ops.interval_unary(kind, l.cuda(), u.cuda()), kind)
    yl = torch.randn(3, 5, 7, generator=g)
    yu = yl + torch.rand(3, 5, 7, generator=g)
    same(ops.interval_product(shifted(l), shifted(u), shifted(yl), shifted(yu)),
         ops.interval_product(l.cuda(), u.cuda(), yl.cuda(), yu.cuda()), "interval product")
