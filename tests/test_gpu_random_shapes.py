"""Seeded random shapes through every operator, against the CPU oracle: the shapes straddle the
thresholds at which the host side switches kernels (vector width, register-resident limits,
tile sizes, short-sequence kernels), which fixed parametrised lists only sample."""
import random

import pytest
import torch

from tests.helpers import rand_bounds
from tests.parity import UNIT_SCALE_ALL
from tests import test_gpu_act as T_act
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
