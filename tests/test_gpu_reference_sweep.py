"""The reference's own correctness sweep (kernel_test/transformer_forward_test_bound.py:725-737, 796-799):
length 2 .. 128 x dim_in 64 .. 512 x dim_out 64 .. 512 for relu / tanh / matmul (batch 1), dot_product_QK
adds dim_out 16 and batches 1, 2, 4, dot_product_V takes dim_out 10, 20, 64 .. 512 -- with the inputs drawn
as that script draws them (:746-754: lb ~ U(0,1), ub = lb + U(0,1), lw and uw independent U(-.5,.5), p = 2,
eps = 0.5), every shape against the CPU oracle at the parity bar.

The dot products are capped by the oracle's cost (16 * B * L^2 * D * d flop <= COST_CAP per shape); the
shapes beyond it differ from those below only in the number of tiles walked and are covered by the
configuration-size tests."""
import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import close, worst
from tests.parity import compare_contraction, UNIT_SCALE_ALL
from tests import test_gpu_act as T_act
from tests import test_gpu_dot as T_dot
from tests import test_gpu_linear as T_lin

pytestmark = pytest.mark.gpu
LENGTHS = [2, 4, 8, 16, 32, 64, 128]
DIMS = [64, 128, 256, 512]
COST_CAP = 1.0e9


def draw(g, B, L, D, H):
    lb = torch.rand(B, L, H, generator=g)
    ub = lb + torch.rand(B, L, H, generator=g)
    lw = torch.rand(B, L, D, H, generator=g) - 0.5
    uw = torch.rand(B, L, D, H, generator=g) - 0.5
    return O.LinearBounds(lw, lb, uw, ub)


@pytest.mark.parametrize("length", LENGTHS)
@pytest.mark.parametrize("kind", ["relu", "tanh"])
def test_reference_sweep_activations(kind, length):
    g = torch.Generator().manual_seed(100 + length)
    for dim_in in DIMS:
        for dim_out in DIMS:
            T_act.check(kind, draw(g, 1, length, dim_in, dim_out), 2.0, 0.5, 1)


@pytest.mark.parametrize("length", LENGTHS)
def test_reference_sweep_matmul(length):
    g = torch.Generator().manual_seed(200 + length)
    for dim_in in DIMS:
        for dim_out in DIMS:
            x = draw(g, 1, length, dim_in, dim_out)
            W = torch.rand(dim_in, dim_out, generator=g) - 0.5          # dim_y_out = dim_in, as the script has it
            T_lin.check(x, W, None, f"reference sweep L={length}", allow=UNIT_SCALE_ALL)


def _dot_case(x, y, run, oracle, what, context=False):
    """Plain bar first; the float64 values of the same inputs (from the oracle's intervals and from the GPU's own)
    are only worked out for a case with a tensor that misses it."""
    print(f"[case] {what}", flush=True)
    *got, (x_l, _x_u, y_l, y_u) = run()
    torch.cuda.synchronize()
    exp = oracle()
    bad = [n for n, a, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()) if not close(a, e)]
    if not bad:
        return
    if context:
        y_l, y_u = y_l.transpose(1, 2), y_u.transpose(1, 2)          # intervals of the values as of value.t()
    ref, mag = T_dot.dot64(x, y, 2.0, 0.5, 1)
    own, _ = T_dot.dot64(x, y, 2.0, 0.5, 1, intervals=(x_l, y_l, y_u))
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
        compare_contraction(name, a, e, ref[name], mag[name], UNIT_SCALE_ALL, ref64_own=own[name])


@pytest.mark.parametrize("length", LENGTHS)
@pytest.mark.parametrize("batch", [1, 2, 4])
def test_reference_sweep_dot_product_qk(batch, length):
    from faith_amd import ops
    g = torch.Generator().manual_seed(300 + 10 * length + batch)
    for dim_in in DIMS:
        for dim_out in [16] + DIMS:
            if 16.0 * batch * length * length * dim_in * dim_out > COST_CAP:
                continue
            x, y = draw(g, batch, length, dim_in, dim_out), draw(g, batch, length, dim_in, dim_out)
            _dot_case(x, y, lambda: ops.dot_product_qk(T_dot.dev(x), T_dot.dev(y), 2.0, 0.5, 1, return_intervals=True),
                      lambda: O.dot_product(x, y, 2.0, 0.5, 1), f"sweep QK B={batch} L={length} D={dim_in} d={dim_out}")


@pytest.mark.parametrize("length", LENGTHS)
@pytest.mark.parametrize("batch", [1, 2, 4])
def test_reference_sweep_dot_product_v(batch, length):
    from faith_amd import ops
    g = torch.Generator().manual_seed(400 + 10 * length + batch)
    for dim_in in DIMS:
        for dim_out in [10, 20] + DIMS:
            if 16.0 * batch * length * length * dim_in * dim_out > COST_CAP:
                continue
            probs = draw(g, batch, length, dim_in, length)
            value = draw(g, batch, length, dim_in, dim_out)
            _dot_case(probs, O.transpose_bounds(value),
                      lambda: ops.dot_product_v(T_dot.dev(probs), T_dot.dev(value), 2.0, 0.5, 1, return_intervals=True),
                      lambda: O.context(probs, value, 2.0, 0.5, 1),
                      f"sweep V B={batch} L={length} D={dim_in} d={dim_out}", context=True)
