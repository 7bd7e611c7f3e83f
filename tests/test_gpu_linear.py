"""HIP sign-split affine propagation (fp32 MFMA) against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import rand_bounds, as_bounds, close, worst
from tests.parity import compare_contraction, UNIT_SCALE_ALL, CONFIG_RATIO

pytestmark = pytest.mark.gpu
INF = float("inf")


def dev(*ts):
    return [None if t is None else t.cuda().contiguous() for t in ts]


def run_linear(x, W, bias):
    from faith_amd import ops
    lw, lb, uw, ub, W, bias = dev(*x.tensors(), W, bias)
    return ops.linear(lw, lb, uw, ub, W, bias)


def linear64(x, W, bias):
    """float64 value of the same fp32 inputs, and sum_k |a_k w_k| per output."""
    Wp, Wn = W.double().clamp(min=0).t(), W.double().clamp(max=0).t()
    a = {k: v.double() for k, v in zip(("lw", "lb", "uw", "ub"), x.tensors())}
    b = 0 if bias is None else bias.double()
    ref = dict(lw=a["lw"] @ Wp + a["uw"] @ Wn, uw=a["uw"] @ Wp + a["lw"] @ Wn,
               lb=a["lb"] @ Wp + a["ub"] @ Wn + b, ub=a["ub"] @ Wp + a["lb"] @ Wn + b)
    mag = dict(lw=a["lw"].abs() @ Wp - a["uw"].abs() @ Wn, uw=a["uw"].abs() @ Wp - a["lw"].abs() @ Wn,
               lb=a["lb"].abs() @ Wp - a["ub"].abs() @ Wn, ub=a["ub"].abs() @ Wp - a["lb"].abs() @ Wn)
    return ref, mag


def check(x, W, bias, what="", allow=None, ratio_ceiling=None):
    print(f"[case] linear {what} x={tuple(x.lw.shape)} W={tuple(W.shape)} bias={bias is not None}", flush=True)
    got = run_linear(x, W, bias)
    torch.cuda.synchronize()
    exp = O.linear(x, W, bias)
    ref, mag = linear64(x, W, bias)
    for name, g, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
        compare_contraction(name, g, e, ref[name], mag[name], allow, ratio_ceiling=ratio_ceiling)
    return got


@pytest.mark.parametrize("shape", [
    (1, 16, 64, 64, 64),       # benchmark configuration 0
    (1, 2, 64, 64, 64), (1, 8, 128, 256, 128), (1, 4, 64, 512, 512),   # reference sweep corners
    (2, 3, 50, 72, 200),       # M, N not multiples of the tile
    (1, 1, 1, 4, 1),           # degenerate
    (1, 5, 33, 100, 130),      # ragged everywhere, K % 4 == 0
    (1, 3, 17, 37, 29),        # K % 4 != 0: any-shape kernel
    (1, 130, 2, 16, 8),        # more constant-term rows than one tile
])
@pytest.mark.parametrize("with_bias", [True, False])
def test_linear_shapes(shape, with_bias):
    B, L, D, H, N = shape
    g = torch.Generator().manual_seed(21)
    x = rand_bounds(g, B, L, D, H, ordered=False, sw=0.5)
    W = torch.randn(N, H, generator=g) / H ** 0.5
    if N * H > 4:
        W.view(-1)[::7] = 0.0          # exact zeros belong to neither sign
    bias = torch.randn(N, generator=g) if with_bias else None
    check(x, W, bias, "sweep")


@pytest.mark.parametrize("shape", [
    (1, 1, 256, 256, 256),     # a pooler: first position only
    (1, 1, 256, 256, 2),       # a classifier's margin
    (1, 3, 85, 128, 50),       # ragged rows and columns, shortest reduction that is split
    (2, 2, 40, 512, 96),
    (1, 1, 64, 3072, 64),      # long reduction, many fetch rounds
    (1, 1, 33, 160, 33),       # K / 4 = 40: five steps, the last fetch round partly empty
])
@pytest.mark.parametrize("with_bias", [True, False])
def test_linear_tiny_problems_split_reduction(shape, with_bias):
    """Problems of a few tiles with K % 32 == 0 and K >= 128 take the kernel that splits the reduction
    over the four wavefronts of a workgroup."""
    B, L, D, H, N = shape
    g = torch.Generator().manual_seed(22)
    x = rand_bounds(g, B, L, D, H, ordered=False, sw=0.5)
    W = torch.randn(N, H, generator=g) / H ** 0.5
    W.view(-1)[::7] = 0.0
    bias = torch.randn(N, generator=g) if with_bias else None
    check(x, W, bias, "tiny")


@pytest.mark.parametrize("shape", [
    (1, 32, 256, 256, 256, 3),     # attention of the small model: one round of 64 x 64 tiles, taken together
    (1, 16, 96, 72, 200, 3),       # ragged rows and columns, K % 16 != 0
    (2, 8, 64, 128, 64, 2),        # two layers
    (1, 1, 64, 256, 64, 3),        # each problem tiny: separate launches of the split-reduction kernel
    (1, 64, 512, 64, 512, 3),      # many tiles: separate launches
    (1, 3, 17, 37, 29, 3),         # K % 4 != 0: separate launches of the any-shape kernel
    (1, 4, 32, 64, 64, 1),
])
@pytest.mark.parametrize("with_bias", [True, False])
def test_linear_group_equals_separate_launches(shape, with_bias):
    """faith_matmul_group_verification gives what faith_matmul_verification gives per layer, bit for bit."""
    from faith_amd import ops
    B, L, D, K, N, n = shape
    g = torch.Generator().manual_seed(23)
    x = rand_bounds(g, B, L, D, K, ordered=False, sw=0.5)
    lw, lb, uw, ub = dev(*x.tensors())
    Ws = [(torch.randn(N, K, generator=g) / K ** 0.5).cuda() for _ in range(n)]
    bs = [torch.randn(N, generator=g).cuda() if with_bias and i != 1 else None for i in range(n)]   # one layer without
    print(f"[case] linear group {shape} bias={with_bias}", flush=True)
    got = ops.linear_group(lw, lb, uw, ub, Ws, bs)
    for i in range(n):
        exp = ops.linear(lw, lb, uw, ub, Ws[i], bs[i])
        for name, a, e in zip(("lw", "lb", "uw", "ub"), got[i], exp):
            assert torch.equal(a, e), f"layer {i} {name} differs from the separate launch"
    if n == 3 and K % 4 == 0:
        ref = O.linear(x, Ws[2].cpu(), None if bs[2] is None else bs[2].cpu())
        r64, mag = linear64(x, Ws[2].cpu(), None if bs[2] is None else bs[2].cpu())
        for name, a, e in zip(("lw", "lb", "uw", "ub"), got[2], ref.tensors()):
            compare_contraction(name, a, e, r64[name], mag[name])


def test_linear_config0_with_concretize():
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(0)
    x = as_bounds(c["x"])
    got = check(x, c["W"], c["bias"], "config0", ratio_ceiling=CONFIG_RATIO)
    l, u = ops.concretize(*got, c["p"], c["eps"], c["words"])
    el, eu = O.concretize(O.linear(x, c["W"], c["bias"]), c["p"], c["eps"], c["words"])
    assert close(l, el) and close(u, eu)
    assert bool((l <= u).all())


def test_linear_config2_reduced():
    """Benchmark configuration 2 with L = 16 instead of 256 (same D_in = 512, H = N = 1024)."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(2, scale=1 / 16)
    x = as_bounds(c["x"])
    got = check(x, c["W"], c["bias"], "config2/16", ratio_ceiling=CONFIG_RATIO)
    l, u = ops.concretize(*got, c["p"], c["eps"], c["words"])
    # concretize is checked on the GPU's own propagated bounds (the constant terms of the two
    # fp32 summation orders differ by more than the bar, see tests/parity.py)
    el, eu = O.concretize(O.LinearBounds(*(t.cpu() for t in got)), c["p"], c["eps"], c["words"])
    assert close(l, el) and close(u, eu)
    assert bool((l <= u).all())


def test_linear_closed_forms_on_gpu():
    """Properties that hold at any size: non-negative W => plain product; degenerate bounds =>
    both sides equal; width identity uw' - lw' = (uw - lw) @ |W|^T."""
    g = torch.Generator().manual_seed(22)
    x = rand_bounds(g, 1, 6, 96, 256, ordered=True)
    W = torch.randn(192, 256, generator=g) / 16
    lw, lb, uw, ub = run_linear(x, W.abs(), None)
    assert close(lw, x.lw @ W.abs().t(), rtol=1e-5, atol=2e-6) and close(uw, x.uw @ W.abs().t(), rtol=1e-5, atol=2e-6)
    pt = O.LinearBounds(x.lw, x.lb, x.lw, x.lb)
    lw, lb, uw, ub = run_linear(pt, W, None)
    assert torch.equal(lw, uw) and torch.equal(lb, ub)
    lw, lb, uw, ub = run_linear(x, W, None)
    # the width against its float64 value at the bar, plus the rounding of the two fp32 results it is the difference of
    width = (x.uw.double() - x.lw.double()) @ W.double().abs().t()
    slack = 2.0 ** -24 * (lw.cpu().double().abs() + uw.cpu().double().abs())
    assert bool(((uw.cpu().double() - lw.cpu().double() - width).abs() <= 1e-6 + 1e-5 * width.abs() + slack).all())
    # ordered coefficients stay ordered EXACTLY: the kernels form uw' = M + R and lw' = M - R with a radius term
    # R that is a sum of non-negative products
    assert bool((uw >= lw).all())


def test_linear_config2_full_size_properties():
    """Full configuration 2 (1.1 TFLOP): linearity in the input and agreement of sampled rows
    with a float64 evaluation; preserves lw' <= uw' and l <= u."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(2)
    lw, lb, uw, ub, W, bias = dev(*(c["x"][k] for k in ("lw", "lb", "uw", "ub")), c["W"], c["bias"])
    olw, olb, ouw, oub = ops.linear(lw, lb, uw, ub, W, bias)
    assert bool((ouw >= olw).all()) and bool((oub >= olb).all())
    # sampled rows against float64
    Wp, Wn = W.double().clamp(min=0).t(), W.double().clamp(max=0).t()
    idx = torch.randint(0, 256 * 512, (64,), generator=torch.Generator().manual_seed(1)).cuda()
    a_l = lw.view(-1, 1024)[idx].double(); a_u = uw.view(-1, 1024)[idx].double()
    assert close(olw.view(-1, 1024)[idx], a_l @ Wp + a_u @ Wn)
    assert close(ouw.view(-1, 1024)[idx], a_u @ Wp + a_l @ Wn)
    assert close(olb, lb.double() @ Wp + ub.double() @ Wn + bias.double())      # summed in double, rounded once
    # scaling the input by 2 scales the coefficients by exactly 2 (power of two: bit-exact)
    o2 = ops.linear(lw * 2, lb, uw * 2, ub, W, bias)
    assert torch.equal(o2[0], olw * 2) and torch.equal(o2[2], ouw * 2)
    l, u = ops.concretize(olw, olb, ouw, oub, c["p"], c["eps"], c["words"])
    assert bool((l <= u).all())


def test_mfma_clock_measurement_is_plausible():
    """faith_mfma_clock: every workgroup reports a shader clock between 0.5 and 3.5 GHz."""
    from faith_amd import _lib
    out = torch.zeros(64, device="cuda")
    _lib.call("faith_mfma_clock", out.data_ptr(), 64, 200, torch._C._cuda_getCurrentRawStream(torch.cuda.current_device()))
    torch.cuda.synchronize()
    assert bool(((out > 500) & (out < 3500)).all()), out


# ---- affine layer + concretization through one entry point (one launch for small problems)
def run_fused(x, W, bias, p, eps, words, force=None):
    """force: None = built-in choice, 6 = the one-launch kernel wherever the shape allows (16 x 16 blocks where
    the reduction is 32, 64 or 128 long), 8 = the same with 32 x 32 blocks throughout, 1 = never."""
    from faith_amd import ops, _lib
    lw, lb, uw, ub, W, bias = dev(*x.tensors(), W, bias)
    if force is not None:
        _lib.call("faith_tune_set", 1, force)
    try:
        out = ops.linear_concretize(lw, lb, uw, ub, W, bias, p, eps, words)
        torch.cuda.synchronize()
    finally:
        if force is not None:
            _lib.call("faith_tune_set", 1, 0)
    return out


@pytest.mark.parametrize("shape", [
    (1, 16, 64, 64, 64, 1),      # benchmark configuration 0
    (1, 1, 256, 256, 2, 1),      # the margin classifier: two columns
    (1, 3, 128, 72, 40, 2),      # two perturbed words, columns ragged against the 32-column block
    (2, 5, 32, 8, 33, 1),        # one block per position, shortest reduction
    (1, 2, 512, 200, 100, 4),    # more blocks than wavefronts, four words
    (1, 4, 96, 64, 64, 3),       # blocks per word not a multiple of the wavefronts
    (1, 40, 256, 128, 96, 1),    # several rounds of workgroups (forced)
    (2, 3, 48, 32, 20, 3),       # 16-row blocks, one per word; reduction of 32; columns ragged against 16
    (1, 2, 144, 128, 17, 1),     # nine 16-row blocks over four wavefronts, reduction of 128
])
@pytest.mark.parametrize("p", [1.0, 2.0, INF, 3.0])
@pytest.mark.parametrize("form", [6, 8])
def test_linear_concretize_one_launch(shape, p, form):
    B, L, D, H, N, words = shape
    if form == 8 and H not in (32, 64, 128):
        pytest.skip("same kernel as form 6")
    print(f"[case] linear_concretize forced one-launch form={form} shape={shape} p={p}", flush=True)
    g = torch.Generator().manual_seed(77)
    x = rand_bounds(g, B, L, D, H, ordered=False, sw=0.5)
    W = torch.randn(N, H, generator=g) / H ** 0.5
    bias = 0.01 * torch.randn(N, generator=g)
    eps = 0.02
    got = run_fused(x, W, bias, p, eps, words, force=form)
    exp = O.linear(x, W, bias)
    ref, mag = linear64(x, W, bias)
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got[:4], exp.tensors()):
        compare_contraction(name, a, e, ref[name], mag[name])
    # the interval is checked on the GPU's own propagated bounds (summation orders of the contraction differ)
    el, eu = O.concretize(O.LinearBounds(*(t.cpu() for t in got[:4])), p, eps, words)
    assert close(got[4], el) and close(got[5], eu), (worst(got[4].cpu(), el), worst(got[5].cpu(), eu))
    # and it equals the two separate entry points within the bar
    sep = run_fused(x, W, bias, p, eps, words, force=1)
    for a, b in zip(got, sep):
        assert close(a, b.cpu()), worst(a.cpu(), b.cpu())


@pytest.mark.parametrize("shape,words", [
    ((1, 3, 17, 37, 29), 1),      # nothing divisible: the separate kernels
    ((1, 4, 48, 64, 64), 1),      # dim_in not a multiple of 32
    ((1, 64, 128, 256, 512), 2),  # more than one round of tiles: the tiled kernel and the concretize kernel
    ((1, 2, 64, 64, 64), 16),     # more words than the one-launch kernel keeps slots for
])
def test_linear_concretize_general_shapes(shape, words):
    B, L, D, H, N = shape
    print(f"[case] linear_concretize built-in choice shape={shape} words={words}", flush=True)
    g = torch.Generator().manual_seed(78)
    x = rand_bounds(g, B, L, D, H, ordered=False, sw=0.5)
    W = torch.randn(N, H, generator=g) / H ** 0.5
    got = run_fused(x, W, None, 2.0, 0.05, words)
    from faith_amd import ops
    lw, lb, uw, ub, Wd = dev(*x.tensors(), W)
    lin = ops.linear(lw, lb, uw, ub, Wd, None)
    l, u = ops.concretize(*lin, 2.0, 0.05, words)
    for a, b in zip(got, (*lin, l, u)):
        assert torch.equal(a, b)


@pytest.mark.parametrize("p", [2.0, float("inf"), 1.0, 3.0])
@pytest.mark.parametrize("shape,force", [
    ((1, 16, 256, 256, 512), None),    # 128 x 64 tiles (built-in choice), two tiles per position
    ((1, 128, 64, 128, 576), None),    # 64 x 64 tiles, one tile per position, ragged last column block
    ((2, 9, 384, 64, 200), 2),         # 128 x 128 tiles forced: three tiles per position, positions over two batch elements
    ((1, 24, 128, 1024, 1024), 2),     # configuration 2's reduction and width, 24 positions
])
def test_linear_concretize_tiled_kernel_with_norms_in_its_epilogue(shape, force, p):
    """Large problems: the tiled MFMA kernel walks the tiles of one position and finishes l, u itself.  Against the
    oracle's linear (the harness for contractions) and the oracle's concretize of the GPU's own coefficients; the
    coefficients must equal the plain layer bit for bit (same tiles, same reduction order)."""
    from faith_amd import ops, _lib
    B, L, D, H, N = shape
    print(f"[case] linear_concretize tiled with norms shape={shape} force={force} p={p}", flush=True)
    g = torch.Generator().manual_seed(79)
    x = rand_bounds(g, B, L, D, H, ordered=False, sw=0.5)
    W = torch.randn(N, H, generator=g) / H ** 0.5
    bias = 0.01 * torch.randn(N, generator=g)
    eps = 0.02
    got = run_fused(x, W, bias, p, eps, 1, force=force)
    exp = O.linear(x, W, bias)
    ref, mag = linear64(x, W, bias)
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got[:4], exp.tensors()):
        compare_contraction(name, a, e, ref[name], mag[name], UNIT_SCALE_ALL)
    el, eu = O.concretize(O.LinearBounds(*(t.cpu() for t in got[:4])), p, eps, 1)
    assert close(got[4], el) and close(got[5], eu), (worst(got[4].cpu(), el), worst(got[5].cpu(), eu))
    assert bool((got[4] <= got[5]).all())
    lw, lb, uw, ub, Wd, bd = dev(*x.tensors(), W, bias)
    if force is not None:
        _lib.call("faith_tune_set", 1, force)
    try:
        lin = ops.linear(lw, lb, uw, ub, Wd, bd)
    finally:
        _lib.call("faith_tune_set", 1, 0)
    for a, b in zip(got[:4], lin):
        assert torch.equal(a, b)
    # knob 7 keeps the two launches apart: the same values within the bar (another order of the norm's additions)
    sep = run_fused(x, W, bias, p, eps, 1, force=7)
    assert close(got[4], sep[4].cpu()) and close(got[5], sep[5].cpu())


def test_linear_concretize_config0_against_oracle():
    from faith_amd.workloads import make_config
    c = make_config(0)
    x = as_bounds(c["x"])
    got = run_fused(x, c["W"], c["bias"], c["p"], c["eps"], c["words"])
    el, eu = O.concretize(O.linear(x, c["W"], c["bias"]), c["p"], c["eps"], c["words"])
    assert close(got[4], el) and close(got[5], eu)
    assert bool((got[4] <= got[5]).all())


def test_bound_call_repeats_the_launch_on_new_contents():
    """ops.bind_linear_concretize converts the arguments once; every call of the object launches again into the same
    result tensors and sees whatever the operand tensors hold by then."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(0)
    x = {k: v.cuda() for k, v in c["x"].items()}
    W, bias = c["W"].cuda(), c["bias"].cuda()
    bound = ops.bind_linear_concretize(x["lw"], x["lb"], x["uw"], x["ub"], W, bias, c["p"], c["eps"], c["words"])
    first = [t.clone() for t in bound.results]
    ref = ops.linear_concretize(x["lw"], x["lb"], x["uw"], x["ub"], W, bias, c["p"], c["eps"], c["words"])
    assert all(torch.equal(a, b) for a, b in zip(first, ref))
    x["lb"].add_(0.25)                                   # same addresses, new contents
    x["ub"].add_(0.25)
    again = bound()
    assert again is bound.results
    ref = ops.linear_concretize(x["lw"], x["lb"], x["uw"], x["ub"], W, bias, c["p"], c["eps"], c["words"])
    assert all(torch.equal(a, b) for a, b in zip(again, ref))
    assert not torch.equal(again[1], first[1])


def test_linear_concretize_rejects_bad_words():
    from faith_amd import _lib
    g = torch.Generator().manual_seed(3)
    x = rand_bounds(g, 1, 2, 6, 8, ordered=False)
    with pytest.raises(_lib.FaithError):
        run_fused(x, torch.randn(4, 8, generator=g), None, 2.0, 0.1, 4)     # 4 does not divide dim_in = 6


def test_per_position_weight_of_matmul_runs_the_layer_kernel_position_by_position():
    """Bounds.matmul with a 3-D weight (Bounds.py:414-428: one [H_out, H] matrix per position, a single batch
    element): each position against the oracle's layer with that position's matrix."""
    from faith_amd import Bounds
    g = torch.Generator().manual_seed(90)
    L, D, H, N = 5, 24, 32, 20
    x = rand_bounds(g, 1, L, D, H, ordered=False, sw=0.5)
    W = torch.randn(L, N, H, generator=g) / H ** 0.5
    lw, lb, uw, ub = dev(*x.tensors())
    got = Bounds(None, 2.0, 0.01, lw=lw, lb=lb, uw=uw, ub=ub).matmul(W.cuda())
    torch.cuda.synchronize()
    assert got.lw.shape == (1, L, D, N) and got.lb.shape == (1, L, N)
    for i in range(L):
        xi = O.LinearBounds(x.lw[:, i:i + 1], x.lb[:, i:i + 1], x.uw[:, i:i + 1], x.ub[:, i:i + 1])
        exp = O.linear(xi, W[i], None)
        ref, mag = linear64(xi, W[i], None)
        for name, a, e in zip(("lw", "lb", "uw", "ub"), (got.lw, got.lb, got.uw, got.ub), exp.tensors()):
            compare_contraction(name, a[:, i:i + 1], e, ref[name], mag[name])
    with pytest.raises(ValueError):
        Bounds(None, 2.0, 0.01, lw=lw, lb=lb, uw=uw, ub=ub).matmul(W[:3].cuda())
