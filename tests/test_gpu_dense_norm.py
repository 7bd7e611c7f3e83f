"""The one-pass operators of the encoder sub-blocks against the separate launches and the CPU oracle:
dense -> residual add -> layer normalisation without the variance (faith_matmul_layer_norm_verification) and
dense -> ReLU (faith_matmul_relu_verification)."""
from types import SimpleNamespace

import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import rand_bounds, close, worst

pytestmark = pytest.mark.gpu
U = 2.0 ** -24


def dev(x):
    return tuple(t.cuda().contiguous() for t in x.tensors())


def separate(x, W, bias, weight, shift, other):
    """The launches the fused entry point replaces; also returns the sum in front of the normalisation."""
    from faith_amd import ops
    lin = ops.linear(*x, W, bias)
    summed = lin if other is None else ops.add(lin, other)
    return ops.layer_norm(*lin, weight, shift, other), summed


def mean_order_bound(summed, weight, name):
    """What a different order of the H additions of a row's mean can change: 2 (H - 1) u mean|x| of the OTHER side
    (the mean subtracted from the lower tensor is the upper one's), times |weight|."""
    lw, lb, uw, ub = summed
    src = {"lw": uw, "uw": lw, "lb": ub, "ub": lb}[name]
    H = src.shape[-1]
    b = 2 * (H - 1) * U * src.abs().double().mean(-1, keepdim=True)
    return b * (1.0 if weight is None else weight.abs().double())


SHAPES = [
    # B, L, D, H (reduction), N
    (1, 3, 64, 64, 256),
    (2, 2, 128, 512, 256),      # the feed-forward output layer: long reduction
    (1, 2, 64, 36, 128),        # reduction not a multiple of the K-step
    (1, 3, 40, 64, 128),        # coefficient rows not a multiple of the 64-row tile
    (1, 1, 192, 256, 128),
]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("residual", [True, False])
@pytest.mark.parametrize("affine", [True, False])
def test_one_pass_equals_the_separate_launches_up_to_the_order_of_the_row_means(shape, residual, affine):
    from faith_amd import ops
    B, L, D, H, N = shape
    print(f"[case] dense+add+layer_norm shape={shape} residual={residual} affine={affine}", flush=True)
    g = torch.Generator().manual_seed(130)
    x = dev(rand_bounds(g, B, L, D, H, ordered=False, sw=0.5))
    W = (torch.randn(N, H, generator=g) / H ** 0.5).cuda()
    bias = (0.1 * torch.randn(N, generator=g)).cuda()
    other = dev(rand_bounds(g, B, L, D, N, ordered=False, sw=0.5)) if residual else None
    weight = torch.randn(N, generator=g).cuda() if affine else None
    shift = torch.randn(N, generator=g).cuda() if affine else None
    if affine:
        weight[3] = 0.0
    assert ops.linear_layer_norm_fits(B * L, D, H, N) >= 1
    got = ops.linear_layer_norm(*x, W, bias, weight, shift, other)
    exp, summed = separate(x, W, bias, weight, shift, other)
    torch.cuda.synchronize()
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp):
        bound = mean_order_bound(summed, weight, name)
        err = (a.double() - e.double()).abs()
        # the products and the sum are the same operations on the same bits; only the mean may differ
        assert bool((err <= bound + 2 * U * e.abs().double()).all()), \
            f"{name}: {float((err - bound).max()):.3g} beyond the bound; {worst(a, e)}"
        if name in ("lb", "ub"):
            assert torch.equal(a, e), f"{name}: the constant terms run through the same two kernels"


@pytest.mark.parametrize("p", [2.0, float("inf")])
def test_one_pass_against_the_oracle_chain(p):
    from faith_amd import ops
    B, L, D, H, N = 1, 3, 64, 128, 128
    g = torch.Generator().manual_seed(131)
    x = rand_bounds(g, B, L, D, H, sw=0.05, sb=1.0, gap_w=0.002, gap_b=0.02)
    r = rand_bounds(g, B, L, D, N, sw=0.05, sb=1.0, gap_w=0.002, gap_b=0.02)
    W = torch.randn(N, H, generator=g) / H ** 0.5
    bias = 0.1 * torch.randn(N, generator=g)
    weight, shift = 1.0 + 0.1 * torch.randn(N, generator=g), 0.05 * torch.randn(N, generator=g)
    got = ops.linear_layer_norm(*dev(x), W.cuda(), bias.cuda(), weight.cuda(), shift.cuda(), dev(r))
    exp = O.layer_norm(O.add(O.linear(x, W, bias), r), weight, shift, "no_var", p, 0.01)
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
        assert close(a, e, rtol=1e-4, atol=2e-5), f"{name}: {worst(a, e)}"


@pytest.mark.parametrize("shape", [(2, 5, 64, 64, 128), (3, 4, 128, 32, 256)])
def test_a_residual_held_for_some_positions_only_equals_the_same_residual_written_out(shape):
    """The added object of the first sub-block is the layer's input, whose coefficients are zero outside the
    perturbed positions: the kernel reads the rows it holds and adds nothing elsewhere.  Bit for bit."""
    from faith_amd import ops
    B, L, D, H, N = shape
    P = 2
    g = torch.Generator().manual_seed(132)
    x = dev(rand_bounds(g, B, L, D, H, ordered=False, sw=0.5))
    W = (torch.randn(N, H, generator=g) / H ** 0.5).cuda()
    weight, shift = torch.randn(N, generator=g).cuda(), torch.randn(N, generator=g).cuda()
    # distinct positions per batch element; one entry outside the sentence: that row is not there
    positions = torch.stack([torch.randperm(L, generator=g)[:P] for _ in range(B)])
    positions[0, 1] = L + 3
    r = rand_bounds(g, B, P, D, N, ordered=False, sw=0.5)
    rb = rand_bounds(g, B, L, 1, N, ordered=False, sw=0.5)
    full_l, full_u = torch.zeros(B, L, D, N), torch.zeros(B, L, D, N)
    for b in range(B):
        for i in range(P):
            if 0 <= int(positions[b, i]) < L:
                full_l[b, positions[b, i]] = r.lw[b, i]
                full_u[b, positions[b, i]] = r.uw[b, i]
    assert ops.linear_layer_norm_fits(B * L, D, H, N, P) >= 1
    compact = (r.lw.cuda(), rb.lb.cuda(), r.uw.cuda(), rb.ub.cuda())
    written_out = (full_l.cuda(), rb.lb.cuda(), full_u.cuda(), rb.ub.cuda())
    a = ops.linear_layer_norm(*x, W, None, weight, shift, compact, positions.cuda())
    e = ops.linear_layer_norm(*x, W, None, weight, shift, written_out)
    torch.cuda.synchronize()
    for name, s, t in zip(("lw", "lb", "uw", "ub"), a, e):
        assert torch.equal(s, t), f"{name}: {worst(s, t)}"


def test_shapes_the_kernel_does_not_take_are_refused_before_anything_is_written():
    from faith_amd import ops, _lib
    g = torch.Generator().manual_seed(133)
    x = dev(rand_bounds(g, 1, 2, 8, 16, ordered=False))
    W = torch.randn(64, 16, generator=g).cuda()          # 64 columns: no whole-row tile
    assert not ops.linear_layer_norm_fits(2, 8, 16, 64)
    with pytest.raises(_lib.FaithError) as err:
        ops.linear_layer_norm(*x, W, None)
    assert err.value.code == _lib.ERR_UNSUPPORTED
    # a residual for some positions needs tiles that lie inside one position
    assert not ops.linear_layer_norm_fits(2, 40, 64, 128, 1) and ops.linear_layer_norm_fits(2, 40, 64, 128, 0) == 1
    # enough tiles to fill the device twice over: the one-pass operator is the faster choice
    assert ops.linear_layer_norm_fits(960, 256, 512, 256, 1) == 2


@pytest.mark.parametrize("shape", [
    # B, L, D, H (reduction), N
    (1, 3, 128, 64, 128),
    (2, 2, 128, 40, 200),       # columns ragged against the 128-column tile, reduction not a multiple of the K-step
    (1, 3, 256, 256, 512),      # the feed-forward input layer of the benchmark network
    (1, 9, 256, 36, 70),        # more positions than XCDs, columns ragged against the 64-column tile
])
@pytest.mark.parametrize("p", [1.0, 2.0, float("inf"), 3.0])
def test_dense_and_relu_in_one_pass_equal_the_separate_launches(shape, p):
    """The layer's result has the same bits either way; a neuron's interval comes from column norms summed in another
    order, so the slopes may differ in the last bits -- and a neuron whose interval ends within rounding of zero,
    or of |l| = |u|, may take another case of the relaxation (none does on this data)."""
    from faith_amd import ops
    B, L, D, H, N = shape
    print(f"[case] dense+relu shape={shape} p={p}", flush=True)
    g = torch.Generator().manual_seed(135)
    xb = rand_bounds(g, B, L, D, H, sw=0.05, sb=0.3, gap_w=0.002, gap_b=0.02)
    x = dev(xb)
    W = (torch.randn(N, H, generator=g) / H ** 0.5).cuda()
    bias = (0.1 * torch.randn(N, generator=g)).cuda()
    eps = 0.05
    assert ops.linear_relu_fits(B * L, D, H, N) >= 1
    got = ops.linear_relu(*x, W, bias, p, eps)
    lin = ops.linear(*x, W, bias)
    exp = ops.relu(*lin, p, eps)
    torch.cuda.synchronize()
    l, u = ops.concretize(*lin, p, eps)
    assert bool(((l < 0) & (u > 0)).float().mean() > 0.05), "the data exercises the straddling case"
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp):
        assert close(a, e, rtol=1e-5, atol=1e-6), f"{name}: {worst(a, e)}"
    # and the oracle's chain
    oexp = O.relu(O.linear(xb, W.cpu(), bias.cpu()), p, eps)
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got, oexp.tensors()):
        assert close(a, e, rtol=1e-4, atol=2e-5), f"oracle {name}: {worst(a, e)}"


def test_dense_and_relu_shapes_the_kernel_does_not_take_are_refused():
    from faith_amd import ops, _lib
    g = torch.Generator().manual_seed(136)
    x = dev(rand_bounds(g, 1, 2, 64, 16, ordered=False))
    W = torch.randn(64, 16, generator=g).cuda()
    assert ops.linear_relu_fits(2, 64, 16, 64) == 0          # a tile holds 128 or 256 rows of one position
    assert ops.linear_relu_fits(2, 256, 16, 64, 2) == 0      # one perturbed word
    assert ops.linear_relu_fits(2, 256, 16, 64) == 1 and ops.linear_relu_fits(960, 256, 256, 512) == 2
    with pytest.raises(_lib.FaithError) as err:
        ops.linear_relu(*x, W, None, 2.0, 0.01)
    assert err.value.code == _lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("batched", [False, True])
def test_encoder_layer_with_the_one_pass_sub_blocks_matches_the_separate_operators_and_the_oracle(batched, monkeypatch):
    """forward.bound_layer at a hidden size the kernel takes (128): against the same propagation with the fused
    operator switched off, and against the CPU oracle."""
    from faith_amd import BoundsMaker, forward as F, ops
    from tests.oracle_bounds import OracleBounds, random_layer, to_device
    hidden, heads, inter, length, eps, p = 128, 4, 128, 4, 0.02, 2.0
    g = torch.Generator().manual_seed(134)
    layer = random_layer(g, hidden, heads, inter)
    norm = SimpleNamespace(weight=1.0 + 0.1 * torch.randn(hidden, generator=g), bias=0.05 * torch.randn(hidden, generator=g))
    emb = torch.randn(1, length, hidden, generator=g)
    glayer, gnorm = to_device(layer, "cuda"), to_device(norm, "cuda")
    make = BoundsMaker()

    def run():
        if batched:
            x = F.bound_inputs(make, emb.cuda(), [1, 2], [eps, eps], p, gnorm, "no_var")
        else:
            x = F.bound_input(make, emb.cuda(), 2, eps, 1, p, gnorm, "no_var")
        return F.bound_layer(x, glayer, "no_var", "relu")[2]

    calls = []
    real, real_fits = ops.linear_layer_norm, ops.linear_layer_norm_fits
    real_relu, real_relu_fits = ops.linear_relu, ops.linear_relu_fits
    monkeypatch.setattr(ops, "linear_layer_norm", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    monkeypatch.setattr(ops, "linear_relu", lambda *a, **k: (calls.append(10), real_relu(*a, **k))[1])
    # a problem this small would go to the separate launches: take the one-pass operators wherever the shape allows
    monkeypatch.setattr(ops, "linear_layer_norm_fits", lambda *a: 2 * min(real_fits(*a), 1))
    monkeypatch.setattr(ops, "linear_relu_fits", lambda *a: 2 * min(real_relu_fits(*a), 1))
    fused = run()
    assert sum(calls) == 12, "both residual sub-blocks and the feed-forward input layer take the one-pass operators"
    monkeypatch.setattr(ops, "linear_layer_norm_fits", lambda *a: 0)
    monkeypatch.setattr(ops, "linear_relu_fits", lambda *a: 0)
    apart = run()
    assert sum(calls) == 12
    torch.cuda.synchronize()
    for name in ("lw", "lb", "uw", "ub"):
        a, e = getattr(fused, name), getattr(apart, name)
        assert close(a, e, rtol=1e-5, atol=2e-6), f"{name}: {worst(a, e)}"
    omake = lambda p_, e_, lw, lb, uw, ub: OracleBounds(p_, e_, lw, lb, uw, ub)
    if not batched:
        ox = F.bound_input(omake, emb, 2, eps, 1, p, norm, "no_var")
        oout = F.bound_layer(ox, layer, "no_var", "relu")[2]
        for name in ("lw", "lb", "uw", "ub"):
            a, e = getattr(fused, name).cpu().double(), getattr(oout, name).double()
            err, scale = float((a - e).abs().max()), float(e.abs().max())
            assert err <= 2e-4 * max(scale, 1.0), f"{name}: max err {err:.3g} at scale {scale:.3g}"
