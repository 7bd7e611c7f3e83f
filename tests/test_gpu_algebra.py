"""HIP elementwise algebra (multiply / divide / scale / add) and the composites built from it
(softmax, layer_norm) against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import rand_bounds, close, worst

pytestmark = pytest.mark.gpu
INF = float("inf")
PS = [1.0, 2.0, INF, 3.0, 1.5]     # 3.0 and 1.5: dual exponents 1.5 and 3, the general-norm kernels


def dev(x):
    return tuple(t.cuda().contiguous() for t in x.tensors())


def gpu_bounds(x, p, eps, words=1):
    from faith_amd import Bounds
    from types import SimpleNamespace
    lw, lb, uw, ub = dev(x)
    return Bounds(SimpleNamespace(perturbed_words=words), p, eps, lw=lw, lb=lb, uw=uw, ub=ub)


def assert_bounds_close(got, exp, rtol=1e-5, atol=1e-6, what=""):
    for name, g_, e in zip(("lw", "lb", "uw", "ub"), (got.lw, got.lb, got.uw, got.ub), exp.tensors()):
        assert g_.shape == e.shape, (what, name, g_.shape, e.shape)
        assert close(g_, e, rtol=rtol, atol=atol), f"{what} {name}: {worst(g_, e)}"


@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("words", [1, 2])
def test_multiply_shapes(p, words):
    from faith_amd import ops
    g = torch.Generator().manual_seed(61)
    for (L, D, H) in [(4, 64, 64), (3, 128, 96), (2, 256, 64), (1, 600, 40), (2, 12, 37), (1, 2, 5)]:
        x = rand_bounds(g, 1, L, D, H, ordered=False, sw=0.1)
        y = rand_bounds(g, 1, L, D, H, ordered=False, sw=0.1)
        print(f"[case] multiply {L,D,H} p={p} words={words}", flush=True)
        z = ops.multiply(dev(x), dev(y), p, 0.05, words)
        e = O.multiply(x, y, p, 0.05, words)
        # constant terms are sums of O(1) products of concrete bounds: allow for the ulp-level
        # difference between the two norm reductions that feed them
        for name, g_, ee, tol in zip(("lw", "lb", "uw", "ub"), z, e.tensors(), (1e-6, 4e-6, 1e-6, 4e-6)):
            assert close(g_, ee, rtol=1e-5, atol=tol), f"{name}: {worst(g_, ee)}"


def test_scale_add_shift_are_exact():
    """One rounding per operation on both sides: these must agree bit for bit."""
    g = torch.Generator().manual_seed(62)
    x = rand_bounds(g, 2, 3, 16, 24, ordered=False)
    y = rand_bounds(g, 2, 3, 16, 24, ordered=False)
    bx, by = gpu_bounds(x, 2.0, 0.1), gpu_bounds(y, 2.0, 0.1)
    W = torch.randn(24, generator=g)
    W[3] = 0.0
    for got, exp in ((bx.multiply(2.5), O.scale(x, 2.5)), (bx.multiply(-0.75), O.scale(x, -0.75)),
                     (bx.multiply(W.cuda()), O.scale(x, W)), (bx.add(by), O.add(x, y)),
                     (bx.add(W.cuda()), O.add(x, W)), (bx.add(0.25), O.add(x, 0.25))):
        for a, b in zip((got.lw, got.lb, got.uw, got.ub), exp.tensors()):
            assert torch.equal(a.cpu(), b)


@pytest.mark.parametrize("p", PS)
def test_divide_and_softmax(p):
    g = torch.Generator().manual_seed(63)
    x = rand_bounds(g, 2, 6, 32, 16, sw=0.05, sb=1.0, gap_w=0.005, gap_b=0.1)
    pos = rand_bounds(g, 2, 6, 32, 16, sw=0.02, sb=0.5, gap_w=0.005, gap_b=0.1)
    pos = O.LinearBounds(pos.lw, pos.lb.abs() + 1.0, pos.uw, pos.lb.abs() + 1.0 + (pos.ub - pos.lb))
    eps = 0.05
    bx, bp = gpu_bounds(x, p, eps), gpu_bounds(pos, p, eps)
    assert_bounds_close(bx.divide(bp), O.divide(x, pos, p, eps), rtol=2e-5, atol=4e-6, what="divide")
    assert_bounds_close(bx.softmax(), O.softmax(x, p, eps), rtol=5e-5, atol=4e-6, what="softmax")
    # a row of probability bounds brackets a distribution
    lo, hi = bx.softmax().concretize()
    assert bool((lo.sum(-1) <= 1 + 1e-4).all()) and bool((hi.sum(-1) >= 1 - 1e-4).all())


SOFTMAX_SHAPES = [
    # B, L, D, H, words
    (1, 5, 256, 32, 1),      # the common case: 8 threads a slab row, 256 threads, 8 rows each
    (2, 3, 64, 32, 2),       # fewer rows than the threads hold
    (1, 4, 100, 16, 4),      # D_in no multiple of the rows in flight
    (1, 2, 768, 32, 1),      # 1024 threads
    (1, 3, 48, 128, 3),      # 32 threads a row
    (1, 2, 40, 256, 1),      # a full wavefront a row
    (1, 3, 30, 4, 1),        # one thread a row
    (2, 2, 33, 23, 1),       # H no multiple of 4: one column per thread
    (1, 2, 300, 7, 2),       # the same, more rows per thread
    (1, 3, 256, 31, 1),      # a sentence of 31 tokens at dim_in 256: 1024 threads, one column each
    (1, 2, 300, 50, 1),      # 1024 threads, 24 rows per thread
    (1, 2, 20, 1, 1),        # softmax of a single score
    (1, 2, 64, 256, 2),      # sixteen wavefronts, a full wavefront a row, two words: 71 KB of LDS
    (1, 2, 32, 256, 4),      # the same with four words: 137 KB
]


def softmax_case(g, B, L, D, H):
    return rand_bounds(g, B, L, D, H, sw=0.05, sb=1.0, gap_w=0.005, gap_b=0.1)


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES)
@pytest.mark.parametrize("p", [1.0, 2.0, INF, 3.0])
def test_softmax_in_one_launch(shape, p):
    """faith_softmax_verification against the oracle's composition of exp, sum, reciprocal and multiply."""
    from faith_amd import ops
    B, L, D, H, words = shape
    g = torch.Generator().manual_seed(70)
    x = softmax_case(g, B, L, D, H)
    eps = 0.05
    print(f"[case] softmax {shape} p={p}", flush=True)
    assert ops.softmax_fits(D, H)
    out = ops.softmax(*dev(x), p, eps, words, return_sum_bound=True)
    exp = O.softmax(x, p, eps, words)
    for name, g_, e in zip(("lw", "lb", "uw", "ub"), out, exp.tensors()):
        assert close(g_, e, rtol=5e-5, atol=4e-6), f"softmax {name}: {worst(g_, e)}"
    e_ = O.exp(x, p, eps, words)
    total = O.LinearBounds(e_.lw.sum(-1, keepdim=True), e_.lb.sum(-1, keepdim=True), e_.uw.sum(-1, keepdim=True),
                           e_.ub.sum(-1, keepdim=True))
    l_sum, _ = O.concretize(total, p, eps, words)
    assert close(out[4], l_sum[..., 0], rtol=2e-5, atol=1e-6), f"lower bound of the sum: {worst(out[4], l_sum[..., 0])}"


@pytest.mark.parametrize("shape", SOFTMAX_SHAPES[:11])
def test_softmax_in_one_launch_equals_the_four_launches(shape):
    """Same per-neuron code and the same roundings between the operators: the fused kernel and the
    composition differ only by the order of the row sum and of the norm reductions."""
    from faith_amd import ops
    B, L, D, H, words = shape
    g = torch.Generator().manual_seed(71)
    x = dev(softmax_case(g, B, L, D, H))
    fused = ops.softmax(*x, 2.0, 0.05, words)
    e = ops.exp(*x, 2.0, 0.05, words)
    s = ops.rowsum(*e)
    r = ops.reciprocal(*s, 2.0, 0.05, words)
    apart = ops.multiply(e, r, 2.0, 0.05, words)
    for name, a, b in zip(("lw", "lb", "uw", "ub"), fused, apart):
        assert close(a, b.cpu(), rtol=1e-5, atol=1e-6), f"{name}: {worst(a, b.cpu())}"


@pytest.mark.parametrize("shape", [(1, 5, 256, 32, 1), (2, 2, 33, 23, 1), (1, 2, 8, 300, 1)])
def test_softmax_takes_the_scale_of_the_scores(shape):
    """softmax(scale=s) is multiply(s).softmax(), bit for bit in the one-launch kernel (one rounding of the product
    either way), composed when the slab does not fit."""
    B, L, D, H, words = shape
    g = torch.Generator().manual_seed(75)
    x = gpu_bounds(softmax_case(g, B, L, D, H), 2.0, 0.05, words)
    fused, apart = x.softmax(scale=0.17), x.multiply(0.17).softmax()
    for name in ("lw", "lb", "uw", "ub"):
        assert torch.equal(getattr(fused, name), getattr(apart, name)), name
    neg = x.softmax(scale=-0.5)                       # a negative factor swaps the bounds: scaled separately
    ref = x.multiply(-0.5).softmax()
    for name in ("lw", "lb", "uw", "ub"):
        assert torch.equal(getattr(neg, name), getattr(ref, name)), name


def test_softmax_that_does_not_fit_is_composed():
    from faith_amd import ops, _lib
    assert not ops.softmax_fits(64, 300) and not ops.softmax_fits(64, 66) and not ops.softmax_fits(5000, 32)
    assert ops.softmax_fits(1024, 32) and ops.softmax_fits(8192, 4) and ops.softmax_fits(128, 256)
    g = torch.Generator().manual_seed(72)
    x = softmax_case(g, 1, 2, 8, 300)
    with pytest.raises(_lib.FaithError) as err:
        ops.softmax(*dev(x), 2.0, 0.05)
    assert err.value.code == _lib.ERR_UNSUPPORTED
    assert_bounds_close(gpu_bounds(x, 2.0, 0.05).softmax(), O.softmax(x, 2.0, 0.05), rtol=5e-5, atol=4e-6,
                        what="composed softmax")


def test_softmax_precondition_is_checked():
    """A sum whose lower bound falls below 1e-12 fails as the reference's assertion does (Bounds.py:1140).
    The tangent of exp is taken at most 0.99 above l, which keeps the sum's lower bound positive; only scores
    so negative that their exponentials vanish get there."""
    g = torch.Generator().manual_seed(73)
    x = rand_bounds(g, 1, 2, 16, 8, sw=0.05, sb=1.0, gap_w=0.005, gap_b=0.1)
    x = O.LinearBounds(x.lw, x.lb - 40.0, x.uw, x.ub - 40.0)
    with pytest.raises(AssertionError, match="reciprocal"):
        gpu_bounds(x, 2.0, 0.05).softmax()
    with pytest.raises(AssertionError):
        O.softmax(x, 2.0, 0.05)


@pytest.mark.parametrize("mode", ["no", "no_var", "standard"])
@pytest.mark.parametrize("p", [2.0, INF])
def test_layer_norm(mode, p):
    g = torch.Generator().manual_seed(64)
    H = 64
    x = rand_bounds(g, 1, 8, 32, H, sw=0.02, sb=1.0, gap_w=0.002, gap_b=0.02)
    weight, bias = torch.randn(H, generator=g), torch.randn(H, generator=g)

    class Norm:
        pass
    n = Norm()
    n.weight, n.bias = weight.cuda(), bias.cuda()
    got = gpu_bounds(x, p, 0.01).layer_norm(n, mode)
    exp = O.layer_norm(x, weight, bias, mode, p, 0.01)
    # a chain of six to ten operators: rounding differences compound
    assert_bounds_close(got, exp, rtol=1e-4, atol=2e-5, what=f"layer_norm/{mode}")


def test_rowsum_of_a_whole_object():
    from faith_amd import ops
    g = torch.Generator().manual_seed(65)
    # last axis: vector path, scalar path, longer than a wavefront keeps in registers (both paths)
    for B, L, D, H in [(2, 3, 7, 64), (1, 5, 3, 100), (3, 1, 2, 5), (1, 2, 3, 1284), (1, 2, 2, 330)]:
        x = rand_bounds(g, B, L, D, H, ordered=False)
        out = ops.rowsum(*(t.cuda() for t in x.tensors()))
        for a, t in zip(out, x.tensors()):
            assert close(a, t.sum(-1, keepdim=True).expand_as(t), rtol=1e-5, atol=1e-5 * H ** 0.5)


@pytest.mark.parametrize("H", [64, 10, 1284, 330])
@pytest.mark.parametrize("with_affine", [True, False])
def test_fused_mean_subtraction_against_float64(H, with_affine):
    """faith_layer_norm_verification against the definition in float64: c_l = l - mean(u),
    c_u = u - mean(l), then weight split by sign and bias on the constant terms."""
    from faith_amd import ops
    g = torch.Generator().manual_seed(66)
    x = rand_bounds(g, 1, 5, 6, H, ordered=False)
    weight = torch.randn(H, generator=g) if with_affine else None
    bias = torch.randn(H, generator=g) if with_affine else None
    if with_affine:
        weight[1] = 0.0
    got = ops.layer_norm(*(t.cuda() for t in x.tensors()), None if weight is None else weight.cuda(),
                         None if bias is None else bias.cuda())
    lw, lb, uw, ub = (t.double() for t in x.tensors())

    def centre(lo, up):
        return lo - up.mean(-1, keepdim=True), up - lo.mean(-1, keepdim=True)
    (clw, cuw), (clb, cub) = centre(lw, uw), centre(lb, ub)
    if with_affine:
        wp, wn = weight.double().clamp(min=0), weight.double().clamp(max=0)
        clw, cuw = clw * wp + cuw * wn, clw * wn + cuw * wp
        clb, cub = clb * wp + cub * wn + bias.double(), clb * wn + cub * wp + bias.double()
    for a, e in zip(got, (clw, clb, cuw, cub)):
        assert close(a, e, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("H", [64, 10, 1284, 330])
@pytest.mark.parametrize("mode", ["no", "no_var", "standard"])
def test_residual_inside_layer_norm(H, mode):
    """layer_norm(..., residual=y) is x.add(y).layer_norm(...) in one launch: same values bit for bit
    (the sum is rounded to fp32 before the mean, as the separate launch stores it)."""
    g = torch.Generator().manual_seed(68)
    x = gpu_bounds(rand_bounds(g, 2, 5, 6, H, sw=0.02, sb=1.0, gap_w=0.002, gap_b=0.02), 2.0, 0.01)
    y = gpu_bounds(rand_bounds(g, 2, 5, 6, H, sw=0.02, sb=1.0, gap_w=0.002, gap_b=0.02), 2.0, 0.01)

    class Norm:
        weight, bias = torch.randn(H, generator=g).cuda(), torch.randn(H, generator=g).cuda()
    fused = x.layer_norm(Norm, mode, residual=y)
    apart = x.add(y).layer_norm(Norm, mode)
    for a, e, name in zip((fused.lw, fused.lb, fused.uw, fused.ub), (apart.lw, apart.lb, apart.uw, apart.ub),
                          ("lw", "lb", "uw", "ub")):
        assert torch.equal(a, e), f"{name} differs between the fused and the separate residual sum"


def test_residual_inside_layer_norm_in_place():
    """The row-wise entry points may write over their inputs, the added object included."""
    from faith_amd import ops, _lib
    g = torch.Generator().manual_seed(69)
    x = [t.cuda() for t in rand_bounds(g, 1, 4, 3, 1284, ordered=False).tensors()]
    y = [t.cuda() for t in rand_bounds(g, 1, 4, 3, 1284, ordered=False).tensors()]
    exp = ops.layer_norm(*x, other=tuple(y))
    lw, lb, uw, ub = y                 # results go where the added object was
    _lib.call("faith_layer_norm_verification", x[1].data_ptr(), x[3].data_ptr(), x[0].data_ptr(), x[2].data_ptr(),
              lb.data_ptr(), ub.data_ptr(), lw.data_ptr(), uw.data_ptr(), None, None,
              lb.data_ptr(), ub.data_ptr(), lw.data_ptr(), uw.data_ptr(), lw.numel() // 1284, lb.numel() // 1284, 1284,
              torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for a, e in zip((lw, lb, uw, ub), exp):
        assert torch.equal(a, e)


def test_rowmean_is_the_averaging_matmul():
    """faith_rowmean_verification against Bounds.matmul with the H x H matrix of 1 / H (Bounds.py:1116)."""
    from faith_amd import ops
    g = torch.Generator().manual_seed(74)
    for B, L, D, H in [(2, 3, 7, 64), (1, 5, 3, 100), (1, 2, 3, 1284), (3, 1, 2, 5)]:
        x = rand_bounds(g, B, L, D, H, ordered=False)
        got = ops.rowmean(*dev(x))
        exp = O.linear(x, torch.full((H, H), 1.0 / H))
        for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
            assert close(a, e, rtol=1e-5, atol=2e-6), f"{name}: {worst(a, e)}"


def test_shift_shares_the_coefficients():
    """Bounds.add with a tensor returns the same lw / uw tensors (Bounds.py:391-395 does too)."""
    g = torch.Generator().manual_seed(67)
    x = gpu_bounds(rand_bounds(g, 1, 3, 4, 8), 2.0, 0.1)
    y = x.add(0.5)
    assert y.lw.data_ptr() == x.lw.data_ptr() and y.uw.data_ptr() == x.uw.data_ptr()
    assert torch.equal(y.lb, x.lb + 0.5) and torch.equal(y.ub, x.ub + 0.5)


@pytest.mark.gpu
def test_concretize_halves_and_clone():
    """Bounds.concretize_l / concretize_u (Bounds.py:311-317) and clone (:328-333)."""
    import math
    from faith_amd import Bounds
    g = torch.Generator().manual_seed(91)
    lw = torch.randn(2, 5, 24, 40, generator=g)
    lb = torch.randn(2, 5, 40, generator=g)
    for p in (1.0, 2.0, float("inf")):
        q = float("inf") if p == 1 else (1.0 if math.isinf(p) else 2.0)
        b = Bounds(None, p, 0.3, lw=lw.cuda(), lb=lb.cuda(), uw=(lw + 0.1).cuda(), ub=(lb + 0.1).cuda())
        want_l = -0.3 * torch.linalg.vector_norm(lw.double(), ord=q, dim=-2)
        want_u = 0.3 * torch.linalg.vector_norm((lw + 0.1).double(), ord=q, dim=-2)
        assert torch.allclose(b.concretize_l().cpu().double(), want_l, rtol=1e-5, atol=1e-6)
        assert torch.allclose(b.concretize_u().cpu().double(), want_u, rtol=1e-5, atol=1e-6)
        c = b.clone()
        assert c.lw.data_ptr() != b.lw.data_ptr() and torch.equal(c.lw, b.lw) and torch.equal(c.ub, b.ub)
