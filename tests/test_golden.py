"""Golden fixtures (tests/golden/bounds_small.npz, float64 closed forms) against the
tensorised CPU oracle (always) and against the HIP path (GPU)."""
import os

import numpy as np
import pytest
import torch

from oracle import bounds_oracle as O

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "bounds_small.npz"))
PS = {"p1": 1.0, "p2": 2.0, "pinf": float("inf")}
TOL = {"relu": dict(rtol=1e-5, atol=1e-6), "tanh": dict(rtol=1e-5, atol=1e-6)}


def t(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32))


def act_input():
    return O.LinearBounds(*(t(G[f"act_{k}"]).unsqueeze(0) for k in ("lw", "lb", "uw", "ub")))


def assert_close(got, exp, **tol):
    np.testing.assert_allclose(got.detach().cpu().double().numpy(), np.asarray(exp), **tol)


def act_impls():
    impls = [("oracle", lambda kind, x, p, w: getattr(O, kind)(x, p, 0.15, w).tensors(),
              lambda x, p, w: O.concretize(x, p, 0.15, w))]
    return impls


@pytest.mark.parametrize("kind", ["relu", "tanh"])
@pytest.mark.parametrize("pname", list(PS))
@pytest.mark.parametrize("words", [1, 2])
def test_oracle_activation_matches_golden(kind, pname, words):
    x = act_input()
    lo, hi = O.concretize(x, PS[pname], 0.15, words)
    assert_close(lo[0], G[f"interval_{pname}_w{words}"][0], rtol=1e-5, atol=1e-6)
    assert_close(hi[0], G[f"interval_{pname}_w{words}"][1], rtol=1e-5, atol=1e-6)
    y = getattr(O, kind)(x, PS[pname], 0.15, words)
    for nm, got in zip(("lw", "lb", "uw", "ub"), y.tensors()):
        assert_close(got[0], G[f"{kind}_{pname}_w{words}_{nm}"], **TOL[kind])


def test_oracle_linear_dot_conv_match_golden():
    y = O.linear(act_input(), t(G["lin_W"]), t(G["lin_bias"]))
    for nm, got in zip(("lw", "lb", "uw", "ub"), y.tensors()):
        assert_close(got[0], G[f"lin_{nm}"], rtol=1e-5, atol=1e-6)
    x = O.LinearBounds(*(t(G[f"dot_x_{k}"]).unsqueeze(0) for k in ("lw", "lb", "uw", "ub")))
    yb = O.LinearBounds(*(t(G[f"dot_y_{k}"]).unsqueeze(0) for k in ("lw", "lb", "uw", "ub")))
    for pname, p in PS.items():
        z = O.dot_product(x, yb, p, 0.2, 1)
        for nm, got in zip(("lw", "lb", "uw", "ub"), z.tensors()):
            assert_close(got[0], G[f"dot_{pname}_{nm}"], rtol=1e-5, atol=1e-6)
    xc = O.LinearBounds(t(G["conv_lw"]).unsqueeze(0), t(G["conv_lb"]), t(G["conv_uw"]).unsqueeze(0), t(G["conv_ub"]))
    for tag, s, pd in (("s1p1", 1, 1), ("s2p0", 2, 0)):
        z = O.conv2d(xc, t(G["conv_W"]), None, s, pd)
        assert_close(z.lw[0], G[f"conv_{tag}_lw"], rtol=1e-5, atol=1e-6)
        assert_close(z.uw[0], G[f"conv_{tag}_uw"], rtol=1e-5, atol=1e-6)
        assert_close(z.lb, G[f"conv_{tag}_lb"], rtol=1e-5, atol=1e-6)
        assert_close(z.ub, G[f"conv_{tag}_ub"], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["relu", "tanh"])
@pytest.mark.parametrize("pname", list(PS))
@pytest.mark.parametrize("words", [1, 2])
def test_hip_activation_matches_golden(kind, pname, words):
    from faith_amd import ops
    x = [v.cuda().contiguous() for v in act_input().tensors()]
    out = getattr(ops, kind)(*x, PS[pname], 0.15, words, return_interval=True)
    assert_close(out[4][0], G[f"interval_{pname}_w{words}"][0], rtol=1e-5, atol=1e-6)
    assert_close(out[5][0], G[f"interval_{pname}_w{words}"][1], rtol=1e-5, atol=1e-6)
    for nm, got in zip(("lw", "lb", "uw", "ub"), out[:4]):
        assert_close(got[0], G[f"{kind}_{pname}_w{words}_{nm}"], **TOL[kind])


@pytest.mark.gpu
def test_hip_linear_dot_conv_match_golden():
    from faith_amd import ops
    x = [v.cuda().contiguous() for v in act_input().tensors()]
    y = ops.linear(*x, t(G["lin_W"]).cuda(), t(G["lin_bias"]).cuda())
    for nm, got in zip(("lw", "lb", "uw", "ub"), y):
        assert_close(got[0], G[f"lin_{nm}"], rtol=1e-5, atol=1e-6)
    xd = tuple(t(G[f"dot_x_{k}"]).unsqueeze(0).cuda() for k in ("lw", "lb", "uw", "ub"))
    yd = tuple(t(G[f"dot_y_{k}"]).unsqueeze(0).cuda() for k in ("lw", "lb", "uw", "ub"))
    for pname, p in PS.items():
        z = ops.dot_product_qk(xd, yd, p, 0.2, 1)
        for nm, got in zip(("lw", "lb", "uw", "ub"), z):
            assert_close(got[0], G[f"dot_{pname}_{nm}"], rtol=1e-5, atol=1e-6)
    for tag, s, pd in (("s1p1", 1, 1), ("s2p0", 2, 0)):
        z = ops.conv2d(t(G["conv_lw"]).unsqueeze(0).cuda(), t(G["conv_lb"]).cuda(), t(G["conv_uw"]).unsqueeze(0).cuda(),
                       t(G["conv_ub"]).cuda(), t(G["conv_W"]).cuda(), None, s, pd)
        assert_close(z[0][0], G[f"conv_{tag}_lw"], rtol=1e-5, atol=1e-6)
        assert_close(z[2][0], G[f"conv_{tag}_uw"], rtol=1e-5, atol=1e-6)
        assert_close(z[1], G[f"conv_{tag}_lb"], rtol=1e-5, atol=1e-6)
        assert_close(z[3], G[f"conv_{tag}_ub"], rtol=1e-5, atol=1e-6)
