"""Seeded random shapes through every operator, against the CPU oracle: the shapes straddle the
thresholds at which the host side switches kernels (vector width, register-resident limits,
tile sizes, short-sequence kernels), which fixed parametrised lists only sample."""
import random
from types import SimpleNamespace

import pytest
import torch

from tests.helpers import rand_bounds
from tests.parity import UNIT_SCALE_ALL
from tests import test_gpu_act as T_act
from tests import test_gpu_conv as T_conv
from tests import test_gpu_dot as T_dot
from tests import test_gpu_linear as T_lin

pytestmark = pytest.mark.gpu
INF = float("inf")
PS = [1.0, 2.0, INF, 3.0]


def pick(rng, *choices):
    return rng.choice(choices)


def dims(rng, lo, hi, multiple_of):
    return rng.randrange(lo // multiple_of + (lo % multiple_of > 0), hi // multiple_of + 1) * multiple_of


@pytest.mark.parametrize("seed", range(24))
def test_random_relaxation_shapes(seed):
    rng = random.Random(1000 + seed)
    g = torch.Generator().manual_seed(2000 + seed)
    words = pick(rng, 1, 1, 2, 3, 4)
    D = dims(rng, words, pick(rng, 40, 300, 700), words)
    H = pick(rng, dims(rng, 4, 260, 4), dims(rng, 32, 256, 32), rng.randrange(1, 90))
    L = rng.randrange(1, 6)
    x = rand_bounds(g, 1, L, D, H, ordered=True, sw=0.2, sb=1.0, gap_w=0.02, gap_b=0.5)
    T_act.check(pick(rng, "relu", "tanh"), x, pick(rng, *PS), 0.05, words, pick(rng, "natural", "natural", "transposed"))


@pytest.mark.parametrize("seed", range(24))
def test_random_relaxation_shapes_on_the_register_resident_tiles(seed):
    """D_in and H multiples of 32 (the register-resident kernels' territory, which uniformly drawn sizes rarely hit),
    several positions, so that a tile that reaches past its own rows lands in a neighbour's."""
    rng = random.Random(7000 + seed)
    g = torch.Generator().manual_seed(8000 + seed)
    D = dims(rng, 32, pick(rng, 256, 256, 512, 1024), 32)
    words = pick(rng, 1, 1, 2, 4)
    H = dims(rng, 32, 192, 32)
    L = rng.randrange(2, 7)
    x = rand_bounds(g, 1, L, D, H, ordered=True, sw=0.2, sb=1.0, gap_w=0.02, gap_b=0.5)
    T_act.check(pick(rng, "relu", "tanh"), x, pick(rng, *PS), 0.05, words, pick(rng, "natural", "natural", "transposed"))


@pytest.mark.parametrize("seed", range(20))
def test_random_linear_shapes(seed):
    rng = random.Random(3000 + seed)
    g = torch.Generator().manual_seed(4000 + seed)
    L, D = rng.randrange(1, 40), rng.randrange(1, 70)
    K = pick(rng, dims(rng, 4, 200, 4), dims(rng, 16, 256, 16), rng.randrange(1, 60))
    N = rng.randrange(1, 300)
    x = rand_bounds(g, 1, L, D, K, ordered=False, sw=0.5)
    W = torch.randn(N, K, generator=g) / K ** 0.5
    bias = torch.randn(N, generator=g) if rng.random() < 0.5 else None
    T_lin.check(x, W, bias, f"random {seed}")


@pytest.mark.parametrize("seed", range(20))
def test_random_dot_shapes(seed):
    rng = random.Random(5000 + seed)
    g = torch.Generator().manual_seed(6000 + seed)
    B = rng.randrange(1, 4)
    Lx, Ly = rng.randrange(1, 150), rng.randrange(1, 150)
    if rng.random() < 0.4:
        Lx, Ly = rng.randrange(1, 65), rng.randrange(1, 65)          # short-sequence kernel territory
    D = pick(rng, 1, rng.randrange(2, 40), dims(rng, 8, 48, 8))
    d = pick(rng, dims(rng, 8, 80, 8), dims(rng, 4, 100, 4), rng.randrange(1, 50))
    words = 2 if D % 2 == 0 and rng.random() < 0.3 else 1
    p = pick(rng, *PS)
    if rng.random() < 0.5:
        x = rand_bounds(g, B, Lx, D, d, ordered=False, sw=0.3, sb=1.0)
        y = rand_bounds(g, B, Ly, D, d, ordered=False, sw=0.3, sb=1.0)
        T_dot.check(x, y, p, 0.1, words, f"random {seed}", UNIT_SCALE_ALL)
    else:
        dv = pick(rng, dims(rng, 4, 80, 4), rng.randrange(1, 40))
        probs = rand_bounds(g, B, Lx, D, Ly, ordered=False, sw=0.2, sb=0.5)
        value = rand_bounds(g, B, Ly, D, dv, ordered=False, sw=0.3, sb=1.0)
        T_dot.check_v(probs, value, p, 0.1, words, f"random {seed}", UNIT_SCALE_ALL)


@pytest.mark.parametrize("seed", range(10))
def test_random_dot_shapes_of_whole_tiles(seed):
    """Sequence lengths and head sizes that are multiples of 32 (the tiled and the per-wavefront MFMA kernels'
    territory), scores and context."""
    rng = random.Random(9000 + seed)
    g = torch.Generator().manual_seed(9500 + seed)
    B = pick(rng, 1, 2, 3)
    Lx, Ly = pick(rng, 32, 64, 96, 128, 160, 192, 256), pick(rng, 32, 64, 96, 128, 192)
    D, d = pick(rng, 4, 8, 16, 24, 32), pick(rng, 16, 32, 64, 128)
    words = pick(rng, 1, 1, 2)
    p = pick(rng, 1.0, 2.0, INF)
    if rng.random() < 0.5:
        x = rand_bounds(g, B, Lx, D, d, ordered=False, sw=0.3, sb=1.0)
        y = rand_bounds(g, B, Ly, D, d, ordered=False, sw=0.3, sb=1.0)
        T_dot.check(x, y, p, 0.1, words, f"whole tiles {seed}", UNIT_SCALE_ALL)
    else:
        dv = pick(rng, 32, 64, 128)
        probs = rand_bounds(g, B, Lx, D, Ly, ordered=False, sw=0.2, sb=0.5)
        value = rand_bounds(g, B, Ly, D, dv, ordered=False, sw=0.3, sb=1.0)
        T_dot.check_v(probs, value, p, 0.1, words, f"whole tiles {seed}", UNIT_SCALE_ALL)


@pytest.mark.parametrize("seed", range(30))
def test_random_conv_shapes(seed):
    """Kernel sizes 1 / 3 / 4 / 5, strides 1 / 2, channel counts and image sizes around the tile sizes of the
    straight-line kernels (32 / 64 / 128 channels; 8 / 16 / 32 columns)."""
    rng = random.Random(11000 + seed)
    g = torch.Generator().manual_seed(11500 + seed)
    K, s = pick(rng, 1, 3, 3, 4, 5), pick(rng, 1, 1, 2)
    pad = pick(rng, 0, K // 2, 1)
    Ci, Co = pick(rng, 1, 3, 4, 8, 16, 20, 32, 64), pick(rng, 8, 16, 24, 32, 33, 48, 64, 96, 128, 160)
    Hh, Ww = pick(rng, 7, 8, 9, 14, 16, 17, 28, 32, 33), pick(rng, 6, 8, 15, 16, 17, 28, 32, 40)
    if (Hh + 2 * pad - K) // s + 1 < 1 or (Ww + 2 * pad - K) // s + 1 < 1:
        pad = K // 2 + 1
    x = T_conv.make(g, pick(rng, 2, 3, 9), Ci, Hh, Ww, ordered=False)
    W = torch.randn(Co, Ci, K, K, generator=g) * (2.0 / (Ci * K * K)) ** 0.5
    bias = torch.randn(Co, generator=g) if rng.random() < 0.5 else None
    T_conv.check(x, W, bias, s, pad, f"random {seed}")


@pytest.mark.parametrize("seed", range(16))
def test_random_one_pass_sub_blocks(seed):
    """The one-pass operators (layer + residual + layer norm, layer + ReLU) forced on shapes of every size they take,
    against the separate operators (which the other tests hold to the oracle)."""
    from faith_amd import Bounds, _lib, ops
    from tests.helpers import worst
    rng = random.Random(13000 + seed)
    g = torch.Generator(device="cuda").manual_seed(13500 + seed)
    L, K = pick(rng, 1, 2, 3, 5, 8, 16, 30, 33), pick(rng, 16, 32, 64, 128, 192, 256, 512)
    norm = seed % 2 == 0
    D = pick(rng, 32, 64, 96, 128, 160, 256, 300) if norm else pick(rng, 128, 256)
    N = pick(rng, 128, 256) if norm else pick(rng, 64, 128, 256, 512)
    lw = torch.empty(1, L, D, K, device="cuda").normal_(0, 0.1, generator=g)
    uw = lw + 0.01 * torch.rand(1, L, D, K, device="cuda", generator=g)
    lb = torch.empty(1, L, K, device="cuda").normal_(0, 1, generator=g)
    ub = lb + 0.1 * torch.rand(1, L, K, device="cuda", generator=g)
    W = torch.empty(N, K, device="cuda").normal_(0, 1 / K ** 0.5, generator=g)
    b = torch.empty(N, device="cuda").normal_(0, 1, generator=g)
    x = Bounds(None, 2.0, 0.05, lw=lw, lb=lb, uw=uw, ub=ub)
    layer = SimpleNamespace(weight=W, bias=b)
    print(f"[case] one-pass {'norm' if norm else 'relu'} L={L} D={D} K={K} N={N}", flush=True)
    try:
        if norm:
            rlw = torch.empty(1, L, D, N, device="cuda").normal_(0, 0.1, generator=g)
            res = Bounds(None, 2.0, 0.05, lw=rlw, lb=torch.zeros(1, L, N, device="cuda"), uw=rlw + 0.01, ub=torch.ones(1, L, N, device="cuda"))
            nl = SimpleNamespace(weight=torch.empty(N, device="cuda").normal_(1, 0.3, generator=g), bias=torch.zeros(N, device="cuda"))
            got = ops.linear_layer_norm(lw, lb, uw, ub, W, b, nl.weight, nl.bias, (res.lw, res.lb, res.uw, res.ub), None)
            want = x.dense(layer).layer_norm(nl, "no_var", residual=res)
        else:
            got = ops.linear_relu(lw, lb, uw, ub, W, b, 2.0, 0.05, 1)
            want = x.dense(layer).relu()
    except _lib.FaithError as err:
        assert err.code == _lib.ERR_UNSUPPORTED
        pytest.skip("a shape the one-pass kernel does not take")
    torch.cuda.synchronize()
    for name, a_, w_ in zip(("lw", "lb", "uw", "ub"), got, (want.lw, want.lb, want.uw, want.ub)):
        scale = float(w_.abs().max())
        assert float((a_ - w_).abs().max()) <= 2e-5 * max(scale, 1.0), name
