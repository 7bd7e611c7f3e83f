"""HIP convolution bounds (implicit GEMM on fp32 MFMA) against the CPU oracle, through the C ABI."""
import pytest
import torch
import torch.nn.functional as F

from oracle import bounds_oracle as O
from tests.helpers import close
from tests.parity import compare_contraction, CONSTANT_TERMS, CONFIG_RATIO

pytestmark = pytest.mark.gpu
INF = float("inf")


def make(g, D, Ci, Hh, Ww, ordered=True):
    lw = torch.randn(1, D, Ci, Hh, Ww, generator=g) * 0.1
    uw = lw + 0.01 * torch.rand(1, D, Ci, Hh, Ww, generator=g) if ordered else torch.randn(1, D, Ci, Hh, Ww, generator=g) * 0.1
    lb = torch.randn(1, Ci, Hh, Ww, generator=g)
    ub = lb + 0.2 * torch.rand(1, Ci, Hh, Ww, generator=g)
    return O.LinearBounds(lw, lb, uw, ub)


def conv64(x, W, bias, stride, pad):
    Wp, Wn = W.double().clamp(min=0), W.double().clamp(max=0)
    cv = lambda t, w: F.conv2d(t, w, None, stride, pad)
    a = {k: v.double() for k, v in zip(("lw", "lb", "uw", "ub"), x.tensors())}
    b = 0 if bias is None else bias.double().view(1, -1, 1, 1)
    ref = dict(lw=(cv(a["lw"][0], Wp) + cv(a["uw"][0], Wn)).unsqueeze(0),
               uw=(cv(a["uw"][0], Wp) + cv(a["lw"][0], Wn)).unsqueeze(0),
               lb=cv(a["lb"], Wp) + cv(a["ub"], Wn) + b, ub=cv(a["ub"], Wp) + cv(a["lb"], Wn) + b)
    mag = dict(lw=(cv(a["lw"][0].abs(), Wp) - cv(a["uw"][0].abs(), Wn)).unsqueeze(0),
               uw=(cv(a["uw"][0].abs(), Wp) - cv(a["lw"][0].abs(), Wn)).unsqueeze(0),
               lb=cv(a["lb"].abs(), Wp) - cv(a["ub"].abs(), Wn), ub=cv(a["ub"].abs(), Wp) - cv(a["lb"].abs(), Wn))
    return ref, mag


def check(x, W, bias, stride, pad, what="", ratio_ceiling=None):
    from faith_amd import ops
    print(f"[case] conv {what} x={tuple(x.lw.shape)} W={tuple(W.shape)} stride={stride} pad={pad}", flush=True)
    got = ops.conv2d(*(t.cuda() for t in x.tensors()), W.cuda(), None if bias is None else bias.cuda(), stride, pad)
    torch.cuda.synchronize()
    exp = O.conv2d(x, W, bias, stride, pad)
    ref, mag = conv64(x, W, bias, stride, pad)
    for name, g_, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
        assert g_.shape == e.shape
        compare_contraction(name, g_, e, ref[name], mag[name], CONSTANT_TERMS, ratio_ceiling=ratio_ceiling)
    return got


@pytest.mark.parametrize("case", [
    # D, Ci, Co, H, W, K, stride, pad
    (3, 8, 16, 32, 32, 3, 1, 1),
    (2, 3, 5, 7, 9, 3, 1, 1),          # ragged everything, Ci not a multiple of 4
    (2, 4, 130, 8, 8, 3, 1, 0),        # Co over one channel tile, no padding
    (2, 6, 8, 17, 40, 3, 2, 1),        # stride 2, Wo over one column tile
    (1, 5, 4, 9, 9, 1, 1, 0),          # 1x1
    (2, 2, 3, 12, 12, 5, 2, 2),        # 5x5 stride 2
    (1, 1, 1, 3, 3, 3, 1, 1),          # degenerate
    # the straight-line kernels of the common layers, each with and without 16-byte weight rows, ragged tiles included
    (2, 8, 130, 17, 40, 3, 2, 1),      # 3x3 stride 2, C_in % 4 == 0, two channel tiles
    (2, 12, 20, 9, 33, 3, 2, 0),       # 3x3 stride 2, three chunks, no padding
    (2, 3, 16, 32, 32, 3, 2, 1),       # 3x3 stride 2, C_in = 3 (4-byte weight loads)
    (3, 3, 64, 32, 32, 3, 1, 1),       # the first layer of an image classifier: 3x3 stride 1, C_in = 3
    (2, 6, 40, 11, 35, 3, 1, 1),       # 3x3 stride 1, C_in = 6: a chunk and a half
    (2, 32, 64, 8, 40, 1, 1, 0),       # 1x1, two chunks of 16 channels
    (2, 20, 130, 9, 9, 1, 1, 0),       # 1x1, C_in no multiple of the chunk (zero patch beyond the last channel)
    (2, 5, 7, 6, 6, 1, 1, 1),          # 1x1 with padding, C_in = 5
    (2, 8, 24, 14, 36, 5, 1, 2),       # 5x5 stride 1, two chunks (the weight slab goes to LDS in two parts)
    (1, 16, 130, 12, 12, 5, 1, 0),     # 5x5, four chunks, two channel tiles
    # tile variants: 16-column pixel blocks (two image rows a block), 64-channel workgroups, and both
    (2, 8, 128, 33, 33, 3, 2, 1),      # Wo = 17: 16 + 1 columns, full channel tile
    (2, 8, 40, 30, 64, 3, 1, 1),       # 64-channel workgroups (8 pixel blocks), 32-column blocks
    (2, 4, 64, 9, 16, 3, 1, 1),        # both: 64 channels, 16 columns, ragged rows
    (2, 16, 200, 16, 16, 1, 1, 0),     # 1x1: 128 + 72 channels -> 64-channel workgroups? no: (200-1)%128 = 71 -> full tiles; 16 columns
    (2, 16, 24, 7, 12, 1, 1, 0),       # 1x1: both small
    (1, 8, 32, 10, 10, 5, 1, 2),       # 5x5: both small
    (3, 3, 32, 16, 16, 3, 1, 1),       # C_in = 3, both small
    # at most 32 output channels: 32-channel tiles of eight pixel blocks, one channel block per wavefront
    (3, 16, 32, 32, 32, 3, 1, 1),
    (2, 16, 16, 20, 20, 3, 1, 1),      # half a channel block, ragged rows and columns
    (2, 8, 24, 33, 33, 3, 2, 1),       # stride 2, 16-column blocks
    (2, 16, 32, 14, 40, 5, 1, 2),      # 5x5
    (2, 32, 20, 9, 9, 1, 1, 0),        # 1x1
    # 4x4 kernels (the strided layers of the small image classifiers), with and without 16-byte weight rows
    (3, 3, 32, 32, 32, 4, 2, 1),
    (2, 32, 128, 16, 16, 4, 2, 1),
    (2, 16, 40, 15, 19, 4, 1, 1),
    (2, 6, 70, 12, 36, 4, 2, 0),
    (2, 1, 16, 28, 28, 5, 1, 2),       # 5x5 on one input channel (4-byte weight rows)
    # results of at most 8 x 8 pixels: pixel blocks of 8 columns x 4 rows
    (3, 64, 128, 8, 8, 3, 1, 1),
    (3, 32, 64, 16, 16, 4, 2, 1),
    (2, 16, 200, 7, 6, 3, 1, 1),       # ragged: 7 x 6 pixels, 128 + 72 channels
    (2, 20, 48, 16, 13, 3, 2, 1),      # 8 x 7 results from stride 2, half a channel tile
    (2, 64, 128, 8, 8, 1, 1, 0),
    (2, 16, 64, 8, 8, 5, 1, 2),
])
@pytest.mark.parametrize("with_bias", [True, False])
def test_conv_shapes(case, with_bias):
    D, Ci, Co, Hh, Ww, K, s, p = case
    g = torch.Generator().manual_seed(41)
    x = make(g, D, Ci, Hh, Ww, ordered=False)
    W = torch.randn(Co, Ci, K, K, generator=g) * (2.0 / (Ci * K * K)) ** 0.5
    W.view(-1)[::5] = 0.0
    bias = torch.randn(Co, generator=g) if with_bias else None
    check(x, W, bias, s, p, "sweep")


@pytest.mark.parametrize("case", [
    (140, 16, 64, 32, 32, 1, 1, 0),    # 1x1: 560 tiles of 64 channels x 8 rows
    (300, 8, 64, 64, 32, 3, 2, 1),     # 3x3 stride 2: 600 tiles (16-column pixel blocks)
    (150, 3, 64, 32, 32, 3, 1, 1),     # first layer, C_in = 3: 600 tiles
])
def test_conv_layers_with_more_tiles_than_resident_workgroups(case):
    """The straight-line kernels run on persistent workgroups (two per CU): with more tiles than that, a workgroup
    walks several, re-using its LDS stages from tile to tile.  Against the oracle, and against the general kernel
    (one tile per workgroup)."""
    from faith_amd import _lib, ops
    D, Ci, Co, Hh, Ww, K, s_, p = case
    g = torch.Generator().manual_seed(45)
    x = make(g, D, Ci, Hh, Ww, ordered=False)
    W = torch.randn(Co, Ci, K, K, generator=g) * (2.0 / (Ci * K * K)) ** 0.5
    bias = torch.randn(Co, generator=g)
    got = check(x, W, bias, s_, p, "many tiles")
    _lib.call("faith_tune_set", 4, 1)
    try:
        general = ops.conv2d(*(t.cuda() for t in x.tensors()), W.cuda(), bias.cuda(), s_, p)
    finally:
        _lib.call("faith_tune_set", 4, 0)
    for name, a_, b_ in zip(("lw", "lb", "uw", "ub"), got, general):
        assert close(a_, b_.cpu(), rtol=1e-5, atol=1e-6), name


@pytest.mark.parametrize("case", [(3, 8, 40, 17, 40, 3, 2, 1), (2, 32, 64, 8, 40, 1, 1, 0), (2, 8, 24, 14, 36, 5, 1, 2),
                                  (3, 3, 64, 32, 32, 3, 1, 1)])
def test_straight_line_conv_kernels_equal_the_general_kernel(case):
    """Same reduction order (channel chunks, channel pairs, taps) in both kernels of a layer: bit for bit where
    the chunk is the same (4 channels); the 1x1 kernel takes 16 channels a chunk and is held to the parity bar."""
    from faith_amd import _lib, ops
    D, Ci, Co, Hh, Ww, K, s_, p = case
    g = torch.Generator().manual_seed(43)
    x = make(g, D, Ci, Hh, Ww, ordered=False)
    W = (torch.randn(Co, Ci, K, K, generator=g) * (2.0 / (Ci * K * K)) ** 0.5).cuda()
    args = [t.cuda() for t in x.tensors()]
    fast = ops.conv2d(*args, W, None, s_, p)
    _lib.call("faith_tune_set", 4, 1)
    try:
        general = ops.conv2d(*args, W, None, s_, p)
    finally:
        _lib.call("faith_tune_set", 4, 0)
    for a, b in zip(fast, general):
        if K == 1:
            assert close(a, b.cpu())
        else:
            assert torch.equal(a, b)


@pytest.mark.parametrize("case", [
    (6, 64, 128, 32, 32, 1, 1, 0),     # 1x1, 128-channel tiles (four wavefronts over the channels)
    (8, 32, 64, 32, 32, 1, 1, 0),      # 1x1, 64-channel tiles, whole images per XCD
    (300, 3, 64, 32, 32, 3, 1, 1),     # first layer; 2400 tiles: more than four per CU, so workgroups walk several
    (3, 20, 100, 30, 30, 1, 1, 0),     # ragged: channels, rows and columns past the last full tile
    (4, 16, 48, 16, 16, 1, 1, 0),      # 16-column pixel blocks
    (2, 3, 200, 9, 70, 3, 1, 1),       # first layer, wide and short image, several channel tiles
    (40, 3, 32, 32, 32, 3, 1, 1),      # first layer of 32 channels: 32-channel tiles of eight image rows
    (5, 3, 96, 28, 28, 3, 1, 1),       # 96 = three 32-channel tiles; rows and columns past the last full tile
    (3, 1, 16, 28, 28, 3, 1, 1),       # one input channel, half a channel tile
])
def test_short_reductions_on_small_wavefront_tiles_equal_the_large_ones(case):
    """Layers with at most 64 products per result run with 1 x 2 MFMA blocks per wavefront (four workgroups per CU)
    instead of 2 x 2; the reduction order per result is the same, so the results are the same bits.  And against
    the oracle."""
    from faith_amd import _lib, ops
    D, Ci, Co, Hh, Ww, K, s_, p = case
    g = torch.Generator().manual_seed(47)
    x = make(g, D, Ci, Hh, Ww, ordered=False)
    W = torch.randn(Co, Ci, K, K, generator=g) * (2.0 / (Ci * K * K)) ** 0.5
    bias = torch.randn(Co, generator=g)
    got = check(x, W, bias, s_, p, "small wavefront tiles")
    _lib.call("faith_tune_set", 4, 3)
    try:
        large = ops.conv2d(*(t.cuda() for t in x.tensors()), W.cuda(), bias.cuda(), s_, p)
    finally:
        _lib.call("faith_tune_set", 4, 0)
    for name, a_, b_ in zip(("lw", "lb", "uw", "ub"), got, large):
        assert torch.equal(a_, b_), name


def test_conv_config4_reduced():
    """Benchmark configuration 4 with D_in = 8 instead of 256 (64 -> 128 channels, 32 x 32, 3x3)."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(4, scale=8 / 256)
    x = O.LinearBounds(c["x"]["lw"], c["x"]["lb"], c["x"]["uw"], c["x"]["ub"])
    got = check(x, c["W"], c["bias"], c["stride"], c["padding"], "config4 D=8", ratio_ceiling=CONFIG_RATIO)
    l, u = ops.concretize_conv(*got, c["p"], c["eps"])
    el, eu = O.concretize_conv(O.LinearBounds(*(t.cpu() for t in got)), c["p"], c["eps"])
    assert close(l, el) and close(u, eu) and bool((l <= u).all())


def test_conv_config4_full_size_properties():
    """Full configuration 4 (155 GFLOP): linearity over D_in (each D_in slice is an independent
    image, so slices computed alone must equal the slices of the full run, bit for bit),
    soundness at sampled corners of the eps-ball, and l <= u."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(4)
    x = {k: v.cuda() for k, v in c["x"].items()}
    W, bias = c["W"].cuda(), c["bias"].cuda()
    lw, lb, uw, ub = ops.conv2d(x["lw"], x["lb"], x["uw"], x["ub"], W, bias, 1, 1)
    sub = slice(100, 104)
    lw2, _, uw2, _ = ops.conv2d(x["lw"][:, sub].contiguous(), x["lb"], x["uw"][:, sub].contiguous(), x["ub"], W, bias, 1, 1)
    assert torch.equal(lw2, lw[:, sub]) and torch.equal(uw2, uw[:, sub])
    # ordered inputs (uw >= lw here) give ordered results exactly: uw' = M + R, lw' = M - R with R a sum of
    # non-negative products
    assert bool((uw >= lw).all()) and bool((ub >= lb).all())
    l, u = ops.concretize_conv(lw, lb, uw, ub, c["p"], c["eps"])
    assert bool((l <= u).all())
    g = torch.Generator().manual_seed(4)
    delta = (torch.sign(torch.randn(2, 256, generator=g)) * c["eps"]).cuda()
    for dl in delta:
        xin_l = torch.einsum("d,dchw->chw", dl, x["lw"][0]) + x["lb"][0]
        xin_u = torch.einsum("d,dchw->chw", dl, x["uw"][0]) + x["ub"][0]
        for tmix in (0.0, 1.0, 0.5):
            v = F.conv2d((xin_l + tmix * (xin_u - xin_l)).unsqueeze(0), W, bias, 1, 1)
            assert bool((v >= l - 1e-3).all()) and bool((v <= u + 1e-3).all())
    # one output channel plane against float64
    Wp, Wn = W.double().clamp(min=0), W.double().clamp(max=0)
    a_l, a_u = x["lw"][0, 7:8].double(), x["uw"][0, 7:8].double()
    ref = F.conv2d(a_l, Wp, None, 1, 1) + F.conv2d(a_u, Wn, None, 1, 1)
    assert close(lw[0, 7:8], ref, rtol=1e-5, atol=2e-6)
