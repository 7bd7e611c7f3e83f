"""tests/golden/reference_vectors.npz holds outputs of the reference's own pure-torch code
(HandTunedKernels/python_reference_code/{relu,matmul,dot_product}_reference.py, executed once by
tests/golden/make_reference_golden.py).  The CPU oracle (always) and the HIP path (GPU) must both
reproduce them at the parity bar: rtol 1e-5, atol 1e-6."""
import os

import numpy as np
import pytest
import torch

from oracle import bounds_oracle as O

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "reference_vectors.npz"))
PS = {"p1": 1.0, "p2": 2.0, "pinf": float("inf")}
RTOL, ATOL = 1e-5, 1e-6
NAMES = ("lw", "lb", "uw", "ub")


def t(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32))


def obj(tag):
    return O.LinearBounds(*(t(G[f"{tag}_{k}"]) for k in NAMES))


def dev(b):
    return tuple(v.cuda().contiguous() for v in b.tensors())


def assert_close(got, exp, what):
    np.testing.assert_allclose(got.detach().cpu().double().numpy(), np.asarray(exp, dtype=np.float64),
                               rtol=RTOL, atol=ATOL, err_msg=what)


def test_fixture_covers_every_relu_branch_and_edge():
    l, u = G["conc_p2_w1_l"][0], G["conc_p2_w1_u"][0]
    assert (l > 0).any() and (u < 0).any() and ((l < 0) & (u > 0)).any()
    # crafted neurons 0..5: l = 0, u = 0, |u| = |l|, |u| > |l|, |u| < |l|, l = u = 0 -- exact for every norm
    for pname in PS:
        for w in (1, 2):
            l, u = G[f"conc_{pname}_w{w}_l"][0], G[f"conc_{pname}_w{w}_u"][0]
            assert (l[:, 0] == 0).all() and (u[:, 1] == 0).all() and (u[:, 2] == -l[:, 2]).all()
            assert (l[:, 5] == 0).all() and (u[:, 5] == 0).all()
    # the reference's choices, as executed: l = 0 and u = 0 are "both"; |u| = |l| gives lower slope 0
    y = {k: G[f"relu_p2_w1_{k}"][0] for k in NAMES}
    x = {k: G[f"act_in_{k}"][0] for k in NAMES}
    assert (y["ub"][:, 0] == x["ub"][:, 0]).all() and (y["lb"][:, 0] == x["lb"][:, 0]).all()   # [0, 1]: k_u = 1, k_l = 1
    assert (y["ub"][:, 1] == 0).all() and (y["lb"][:, 1] == 0).all()                          # [-1, 0]
    assert (y["lb"][:, 2] == 0).all() and np.allclose(y["ub"][:, 2], 0.5)                     # [-.5, .5]: (ub - l) / 2
    assert (y["lb"][:, 3] == x["lb"][:, 3]).all()                                             # |u| > |l|: identity below
    assert (y["lb"][:, 4] == 0).all()                                                         # |u| < |l|: zero below


@pytest.mark.parametrize("pname", list(PS))
@pytest.mark.parametrize("words", [1, 2])
def test_oracle_concretize_and_relu_match_the_reference(pname, words):
    x = obj("act_in")
    eps = float(G["act_eps"])
    lo, hi = O.concretize(x, PS[pname], eps, words)
    assert_close(lo, G[f"conc_{pname}_w{words}_l"], "l")
    assert_close(hi, G[f"conc_{pname}_w{words}_u"], "u")
    y = O.relu(x, PS[pname], eps, words)
    for nm, got in zip(NAMES, y.tensors()):
        assert_close(got, G[f"relu_{pname}_w{words}_{nm}"], f"relu {nm}")


def test_oracle_linear_matches_the_reference():
    y = O.linear(obj("act_in"), t(G["lin_W"]), None)
    for nm, got in zip(NAMES, y.tensors()):
        assert_close(got, G[f"lin_{nm}"], f"linear {nm}")


@pytest.mark.parametrize("pname", list(PS))
@pytest.mark.parametrize("words", [1, 2])
def test_oracle_dot_product_matches_the_reference(pname, words):
    z = O.dot_product(obj("dot_x"), obj("dot_y"), PS[pname], float(G["dot_eps"]), words)
    for nm, got in zip(NAMES, z.tensors()):
        assert_close(got, G[f"dot_{pname}_w{words}_{nm}"], f"dot {nm}")


def test_oracle_interval_dot_product_matches_the_reference():
    z = O.dot_product(obj("dot1_x"), obj("dot1_y"), 2.0, float(G["dot_eps"]), 1)
    for nm, got in zip(NAMES, z.tensors()):
        assert_close(got, G[f"dot1_{nm}"], f"dot D=1 {nm}")


def test_a_misread_choice_fails_the_vectors():
    """The vectors tell the reference's choice from its sound alternatives: each mutation below is a
    valid relaxation and must still miss the stored outputs."""
    x = obj("act_in")
    eps = float(G["act_eps"])
    lo, hi = O.concretize(x, 2.0, eps, 1)
    ref = G["relu_p2_w1_lb"]          # the crafted edge neurons have zero coefficients: their constant terms tell
    both = (lo <= 0) & (hi >= 0)
    # lower slope [|u| >= |l|] instead of [|u| > |l|]
    k = (hi.abs() >= lo.abs()).float()
    alt = torch.where(both, x.lb * k, torch.where(lo > 0, x.lb, torch.zeros_like(x.lb)))
    assert not np.allclose(alt.numpy(), ref, rtol=RTOL, atol=ATOL)
    # lower slope always 0 (also sound)
    alt0 = torch.where(lo > 0, x.lb, torch.zeros_like(x.lb))
    assert not np.allclose(alt0.numpy(), ref, rtol=RTOL, atol=ATOL)
    # and the reading the oracle holds does reproduce them
    k = (hi.abs() > lo.abs()).float()
    same = torch.where(both, x.lb * k, torch.where(lo > 0, x.lb, torch.zeros_like(x.lb)))
    assert np.allclose(same.numpy(), ref, rtol=RTOL, atol=ATOL)
    # McCormick with beta_u = u_x (the textbook corner) instead of the reference's l_x
    q, kk = obj("dot_x"), obj("dot_y")
    z = O.dot_product(q, kk, 2.0, float(G["dot_eps"]), 1)
    l_a, u_a = O.concretize(q, 2.0, float(G["dot_eps"]), 1)
    l_b, u_b = O.concretize(kk, 2.0, float(G["dot_eps"]), 1)
    pos, neg = (lambda v: v.clamp(min=0)), (lambda v: v.clamp(max=0))
    ub_alt = (torch.einsum("bjk,bik->bij", pos(u_b), q.ub) + torch.einsum("bjk,bik->bij", neg(u_b), q.lb)
              + torch.einsum("bik,bjk->bij", pos(u_a), kk.ub) + torch.einsum("bik,bjk->bij", neg(u_a), kk.lb)
              - torch.einsum("bjk,bik->bij", u_b, u_a))
    assert not np.allclose(ub_alt.numpy(), G["dot_p2_w1_ub"], rtol=1e-4, atol=1e-5)
    assert np.allclose(z.ub.numpy(), G["dot_p2_w1_ub"], rtol=RTOL, atol=ATOL)


# ------------------------------------------------------------------------------------------
# the HIP path against the same vectors
# ------------------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("pname", list(PS))
@pytest.mark.parametrize("words", [1, 2])
@pytest.mark.parametrize("layout", ["natural", "transposed"])
def test_hip_concretize_and_relu_match_the_reference(pname, words, layout):
    from faith_amd import ops
    x = dev(obj("act_in"))
    eps = float(G["act_eps"])
    if layout == "natural":
        out = ops.relu(*x, PS[pname], eps, words, return_interval=True)
        got = out[:4]
    else:
        lw, lb, uw, ub = x
        out = ops.relu(lw.transpose(2, 3).contiguous(), lb, uw.transpose(2, 3).contiguous(), ub, PS[pname], eps, words,
                       layout=ops.LAYOUT_TRANSPOSED, return_interval=True)
        got = (out[0].transpose(2, 3), out[1], out[2].transpose(2, 3), out[3])
    assert_close(out[4], G[f"conc_{pname}_w{words}_l"], "l")
    assert_close(out[5], G[f"conc_{pname}_w{words}_u"], "u")
    for nm, g in zip(NAMES, got):
        assert_close(g, G[f"relu_{pname}_w{words}_{nm}"], f"relu {nm}")
    lo, hi = ops.concretize(*x, PS[pname], eps, words)
    assert_close(lo, G[f"conc_{pname}_w{words}_l"], "concretize l")
    assert_close(hi, G[f"conc_{pname}_w{words}_u"], "concretize u")


@pytest.mark.gpu
def test_hip_linear_matches_the_reference():
    from faith_amd import ops
    y = ops.linear(*dev(obj("act_in")), t(G["lin_W"]).cuda(), None)
    for nm, got in zip(NAMES, y):
        assert_close(got, G[f"lin_{nm}"], f"linear {nm}")


@pytest.mark.gpu
@pytest.mark.parametrize("pname", list(PS))
@pytest.mark.parametrize("words", [1, 2])
def test_hip_dot_product_matches_the_reference(pname, words):
    from faith_amd import ops
    z = ops.dot_product_qk(dev(obj("dot_x")), dev(obj("dot_y")), PS[pname], float(G["dot_eps"]), words)
    for nm, got in zip(NAMES, z):
        assert_close(got, G[f"dot_{pname}_w{words}_{nm}"], f"dot {nm}")


@pytest.mark.gpu
def test_hip_interval_dot_product_matches_the_reference():
    from faith_amd import ops
    z = ops.dot_product_qk(dev(obj("dot1_x")), dev(obj("dot1_y")), 2.0, float(G["dot_eps"]), 1)
    for nm, got in zip(NAMES, z):
        assert_close(got, G[f"dot1_{nm}"], f"dot D=1 {nm}")
