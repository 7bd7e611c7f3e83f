"""HIP convolution bounds (implicit GEMM on fp32 MFMA) against the CPU oracle, through the C ABI."""
import pytest
import torch
import torch.nn.functional as F

from oracle import bounds_oracle as O
from tests.helpers import close
from tests.parity import compare_contraction, CONSTANT_TERMS

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


def check(x, W, bias, stride, pad, what=""):
    from faith_amd import ops
    print(f"[case] conv {what} x={tuple(x.lw.shape)} W={tuple(W.shape)} stride={stride} pad={pad}", flush=True)
    got = ops.conv2d(*(t.cuda() for t in x.tensors()), W.cuda(), None if bias is None else bias.cuda(), stride, pad)
    torch.cuda.synchronize()
    exp = O.conv2d(x, W, bias, stride, pad)
    ref, mag = conv64(x, W, bias, stride, pad)
    for name, g_, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
        assert g_.shape == e.shape
        compare_contraction(name, g_, e, ref[name], mag[name], CONSTANT_TERMS)
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


def test_conv_config4_reduced():
    """Benchmark configuration 4 with D_in = 8 instead of 256 (64 -> 128 channels, 32 x 32, 3x3)."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(4, scale=8 / 256)
    x = O.LinearBounds(c["x"]["lw"], c["x"]["lb"], c["x"]["uw"], c["x"]["ub"])
    got = check(x, c["W"], c["bias"], c["stride"], c["padding"], "config4 D=8")
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
