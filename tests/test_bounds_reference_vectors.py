"""tests/golden/bounds_reference_vectors.npz holds outputs of the reference's own `Bounds` class
(Transformer_Verification_Code/Verifiers/Bounds.py, executed once by tests/golden/make_bounds_golden.py without the
six top-level statements that need tvm and nvcc).  It covers the operators that exist nowhere else in the reference
in runnable form -- tanh, exp, sqr, sqrt, reciprocal, multiply / divide of two objects, softmax, layer_norm -- next
to relu, matmul, dot_product and context.  The CPU oracle (always) and the HIP path (GPU) must both reproduce them
at the parity bar: rtol 1e-5, atol 1e-6 (the composed operators on the GPU at the bar of their composition)."""
import os
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from oracle import bounds_oracle as O

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "bounds_reference_vectors.npz"))
INF = float("inf")
CASES = {"p1_w1": (1.0, 1), "p2_w2": (2.0, 2), "pinf_w1": (INF, 1), "pinf_w2": (INF, 2), "p2_w1": (2.0, 1)}
RTOL, ATOL = 1e-5, 1e-6
NAMES = ("lw", "lb", "uw", "ub")
EPS, EPS_SOFT, EPS_NORM, EPS_DOT = (float(G[k]) for k in ("eps", "eps_soft", "eps_norm", "eps_dot"))


def t(a):
    return torch.from_numpy(np.asarray(a, dtype=np.float32))


def obj(tag):
    return O.LinearBounds(*(t(G[f"{tag}_{k}"]) for k in NAMES))


def assert_matches(got, tag, what, rtol=RTOL, atol=ATOL):
    for nm, g_ in zip(NAMES, got):
        np.testing.assert_allclose(g_.detach().cpu().double().numpy(), np.asarray(G[f"{tag}_{nm}"], dtype=np.float64),
                                   rtol=rtol, atol=atol, err_msg=f"{what} {nm}")


# operator -> (input object, eps, oracle call)
UNARY = {
    "tanh": ("any_in", EPS, O.tanh), "relu": ("any_in", EPS, O.relu), "exp": ("any_in", EPS, O.exp),
    "sqr": ("any_in", EPS, O.sqr), "sqrt": ("pos_in", EPS, O.sqrt), "reciprocal": ("pos_in", EPS, O.reciprocal),
    "softmax": ("soft_in", EPS_SOFT, O.softmax),
}


def test_fixture_covers_every_tanh_branch_and_edge():
    l, u = G["conc_p2_w1_l"][0], G["conc_p2_w1_u"][0]
    assert (l > 0).any() and (u < 0).any() and ((l < 0) & (u > 0)).any()
    # crafted neurons (zero coefficients, exact for every norm): [0, 1], [-1, 0], [-.5, .5], a point, a tiny interval
    for tag in CASES:
        l, u = G[f"conc_{tag}_l"][0], G[f"conc_{tag}_u"][0]
        assert (l[:, 0] == 0).all() and (u[:, 1] == 0).all() and (u[:, 2] == -l[:, 2]).all()
        assert (l[:, 5] == 0).all() and (u[:, 5] == 0).all() and (u[:, 8] > l[:, 8]).all()
    # the reference's choice as executed: with strict comparisons [0, 1] belongs to the straddling branch, whose upper
    # line is the tangent from (l, tanh l) found by bisection -- not the midpoint tangent of the one-signed branch,
    # which would give (1 - 0.5) / cosh(0.5)^2 + tanh(0.5) as the constant term of this zero-coefficient neuron
    one_signed = 0.5 / np.cosh(0.5) ** 2 + np.tanh(0.5)
    assert abs(G["tanh_p2_w1_ub"][0, 0, 0] - one_signed) > 1e-3


@pytest.mark.parametrize("tag", list(CASES))
@pytest.mark.parametrize("kind", list(UNARY))
def test_oracle_unary_operators_match_the_reference(kind, tag):
    p, words = CASES[tag]
    src, eps, fn = UNARY[kind]
    assert_matches(fn(obj(src), p, eps, words).tensors(), f"{kind}_{tag}", kind)


GENERAL = {"p3_w1": (3.0, 1), "p1.5_w2": (1.5, 2)}      # dual exponents 1.5 and 3


@pytest.mark.parametrize("tag", list(GENERAL))
def test_oracle_general_norms_match_the_reference(tag):
    p, words = GENERAL[tag]
    x = obj("any_in")
    assert_matches(O.tanh(x, p, EPS, words).tensors(), f"tanh_{tag}", "tanh")
    assert_matches(O.relu(x, p, EPS, words).tensors(), f"relu_{tag}", "relu")
    lo, hi = O.concretize(x, p, EPS, words)
    np.testing.assert_allclose(lo.numpy(), G[f"conc_{tag}_l"], rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(hi.numpy(), G[f"conc_{tag}_u"], rtol=RTOL, atol=ATOL)


@pytest.mark.gpu
@pytest.mark.parametrize("tag", list(GENERAL))
def test_hip_general_norms_match_the_reference(tag):
    p, words = GENERAL[tag]
    print(f"[case] tanh, relu, concretize {tag} against the executed reference", flush=True)
    x = gpu_bounds("any_in", p, EPS, words)
    assert_matches(quad(x.tanh()), f"tanh_{tag}", "tanh")
    assert_matches(quad(x.relu()), f"relu_{tag}", "relu")
    lo, hi = x.concretize()
    np.testing.assert_allclose(lo.cpu().numpy(), G[f"conc_{tag}_l"], rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(hi.cpu().numpy(), G[f"conc_{tag}_u"], rtol=RTOL, atol=ATOL)


@pytest.mark.parametrize("tag", list(CASES))
def test_oracle_products_match_the_reference(tag):
    p, words = CASES[tag]
    assert_matches(O.multiply(obj("any_in"), obj("any2_in"), p, EPS, words).tensors(), f"multiply_{tag}", "multiply")
    assert_matches(O.divide(obj("any_in"), obj("pos_in"), p, EPS, words).tensors(), f"divide_{tag}", "divide")


@pytest.mark.parametrize("tag", list(CASES))
@pytest.mark.parametrize("mode", ["no_var", "standard"])
def test_oracle_layer_norm_matches_the_reference(mode, tag):
    p, words = CASES[tag]
    y = O.layer_norm(obj("norm_in"), t(G["norm_weight"]), t(G["norm_bias"]), mode, p, EPS_NORM, words)
    assert_matches(y.tensors(), f"layernorm_{'novar' if mode == 'no_var' else 'standard'}_{tag}", f"layer_norm {mode}")


@pytest.mark.parametrize("tag", list(CASES))
def test_oracle_attention_matches_the_reference(tag):
    p, words = CASES[tag]
    assert_matches(O.dot_product(obj("dot_x"), obj("dot_y"), p, EPS_DOT, words).tensors(), f"dot_{tag}", "dot_product")
    assert_matches(O.context(obj("ctx_probs"), obj("ctx_value"), p, EPS_DOT, words).tensors(), f"context_{tag}", "context")
    lo, hi = O.concretize(obj("any_in"), p, EPS, words)
    np.testing.assert_allclose(lo.numpy(), G[f"conc_{tag}_l"], rtol=RTOL, atol=ATOL)
    np.testing.assert_allclose(hi.numpy(), G[f"conc_{tag}_u"], rtol=RTOL, atol=ATOL)


def test_oracle_affine_operators_match_the_reference():
    x = obj("any_in")
    assert_matches(O.linear(x, t(G["lin_W"]), None).tensors(), "matmul", "matmul")
    assert_matches(O.scale(x, -0.7).tensors(), "scale_neg", "multiply(-0.7)")
    assert_matches(O.scale(x, 1.3).tensors(), "scale_pos", "multiply(1.3)")
    assert_matches(O.add(x, obj("any2_in")).tensors(), "add_bounds", "add(Bounds)")
    assert_matches(O.add(x, t(G["norm_bias"])).tensors(), "add_vector", "add(vector)")


def test_a_misread_tanh_or_exp_fails_the_vectors():
    """The vectors tell the reference's choices from their sound alternatives: nine bisection steps instead of ten, or
    another tangent point for exp, are valid relaxations and must miss the stored outputs."""
    x = obj("any_in")
    nine = O.tanh(x, 2.0, EPS, 1, iters=9)
    assert not np.allclose(nine.lb.numpy(), G["tanh_p2_w1_lb"], rtol=RTOL, atol=ATOL)
    ten = O.tanh(x, 2.0, EPS, 1)
    assert np.allclose(ten.lb.numpy(), G["tanh_p2_w1_lb"], rtol=RTOL, atol=ATOL)
    # exp: lower line tangent at the midpoint without the cap l + 0.99 (sound as well): the wide neuron [-8, 9] tells
    l, u = O.concretize(x, 2.0, EPS, 1)
    mid = (l + u) / 2
    k = torch.exp(mid)
    alt_lb = (x.lb - mid) * k + torch.exp(mid)
    assert not np.allclose(alt_lb.numpy(), G["exp_p2_w1_lb"], rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------------------------------------
# the HIP path against the same vectors
# ------------------------------------------------------------------------------------------
def gpu_bounds(tag, p, eps, words):
    from faith_amd import Bounds
    lw, lb, uw, ub = (v.cuda().contiguous() for v in obj(tag).tensors())
    return Bounds(SimpleNamespace(perturbed_words=words), p, eps, lw=lw, lb=lb, uw=uw, ub=ub)


def quad(b):
    return b.lw, b.lb, b.uw, b.ub


@pytest.mark.gpu
@pytest.mark.parametrize("tag", list(CASES))
@pytest.mark.parametrize("kind", ["tanh", "relu", "exp", "sqr", "sqrt", "reciprocal"])
def test_hip_relaxations_match_the_reference(kind, tag):
    p, words = CASES[tag]
    src, eps, _ = UNARY[kind]
    print(f"[case] {kind} {tag} against the executed reference", flush=True)
    y = getattr(gpu_bounds(src, p, eps, words), kind)()
    assert_matches(quad(y), f"{kind}_{tag}", kind)


@pytest.mark.gpu
@pytest.mark.parametrize("tag", list(CASES))
def test_hip_products_softmax_and_layer_norm_match_the_reference(tag):
    p, words = CASES[tag]
    print(f"[case] products, softmax, layer_norm {tag} against the executed reference", flush=True)
    x = gpu_bounds("any_in", p, EPS, words)
    assert_matches(quad(x.multiply(gpu_bounds("any2_in", p, EPS, words))), f"multiply_{tag}", "multiply")
    # the composed operators too are held to the plain bar (measured: at most 0.05 of it on these vectors)
    assert_matches(quad(x.divide(gpu_bounds("pos_in", p, EPS, words))), f"divide_{tag}", "divide")
    assert_matches(quad(gpu_bounds("soft_in", p, EPS_SOFT, words).softmax()), f"softmax_{tag}", "softmax")
    normalizer = SimpleNamespace(weight=t(G["norm_weight"]).cuda(), bias=t(G["norm_bias"]).cuda())
    for mode, key in (("no_var", "novar"), ("standard", "standard")):
        y = gpu_bounds("norm_in", p, EPS_NORM, words).layer_norm(normalizer, mode)
        assert_matches(quad(y), f"layernorm_{key}_{tag}", f"layer_norm {mode}")


@pytest.mark.gpu
@pytest.mark.parametrize("tag", list(CASES))
def test_hip_attention_matches_the_reference(tag):
    p, words = CASES[tag]
    print(f"[case] dot_product, context {tag} against the executed reference", flush=True)
    z = gpu_bounds("dot_x", p, EPS_DOT, words).dot_product(gpu_bounds("dot_y", p, EPS_DOT, words))
    assert_matches(quad(z), f"dot_{tag}", "dot_product")
    c = gpu_bounds("ctx_probs", p, EPS_DOT, words).context(gpu_bounds("ctx_value", p, EPS_DOT, words))
    assert_matches(quad(c), f"context_{tag}", "context")


@pytest.mark.gpu
def test_hip_affine_operators_match_the_reference():
    x = gpu_bounds("any_in", 2.0, EPS, 1)
    assert_matches(quad(x.matmul(t(G["lin_W"]).cuda())), "matmul", "matmul")
    assert_matches(quad(x.multiply(-0.7)), "scale_neg", "multiply(-0.7)")
    assert_matches(quad(x.multiply(1.3)), "scale_pos", "multiply(1.3)")
    assert_matches(quad(x.add(gpu_bounds("any2_in", 2.0, EPS, 1))), "add_bounds", "add(Bounds)")
    assert_matches(quad(x.add(t(G["norm_bias"]).cuda())), "add_vector", "add(vector)")


# ------------------------------------------------------------------------------------------
# method "ibp": the reference's interval branches, executed (its relu, product and dot product call .cuda() on
# constants and could not be run where the vectors were written; tests/test_ibp.py pins those by their closed forms)
# ------------------------------------------------------------------------------------------
IBP_UNARY = {"tanh": "ibp_in", "exp": "ibp_in", "sqr": "ibp_in", "sqrt": "ibp_pos_in", "reciprocal": "ibp_pos_in"}


def interval_object(tag):
    lb, ub = t(G[f"{tag}_lb"]), t(G[f"{tag}_ub"])
    zeros = torch.zeros(1, lb.shape[1], 2, lb.shape[2])
    return O.LinearBounds(zeros, lb, zeros.clone(), ub)


def assert_interval(lo, hi, tag, what, rtol=RTOL, atol=ATOL):
    np.testing.assert_allclose(lo.detach().cpu().numpy(), G[f"ibp_{tag}_lb"], rtol=rtol, atol=atol, err_msg=f"{what} lower")
    np.testing.assert_allclose(hi.detach().cpu().numpy(), G[f"ibp_{tag}_ub"], rtol=rtol, atol=atol, err_msg=f"{what} upper")


@pytest.mark.parametrize("kind", list(IBP_UNARY))
def test_oracle_interval_operators_match_the_reference(kind):
    x = interval_object(IBP_UNARY[kind])
    assert_interval(*O.interval_unary(kind, x.lb, x.ub), kind, f"ibp {kind}")


def test_oracle_interval_affine_operators_match_the_reference():
    x = interval_object("ibp_in")
    y = O.linear(x, t(G["ibp_W"]), None)
    assert_interval(y.lb, y.ub, "matmul", "ibp matmul")
    z = O.layer_norm(x, t(G["ibp_norm_weight"]), t(G["ibp_norm_bias"]), "no_var", 2.0, 0.1, 2)
    assert_interval(z.lb, z.ub, "layernorm_novar", "ibp layer_norm")


@pytest.mark.gpu
def test_hip_interval_mode_matches_the_reference():
    from faith_amd import Bounds
    args = SimpleNamespace(perturbed_words=2, method="ibp")

    def gpu_interval(tag):
        lb, ub = t(G[f"{tag}_lb"]).cuda(), t(G[f"{tag}_ub"]).cuda()
        zeros = torch.zeros(1, lb.shape[1], 2 * lb.shape[2], lb.shape[2], device="cuda")
        return Bounds(args, 2.0, 0.1, lw=zeros, lb=lb, uw=zeros.clone(), ub=ub)
    for kind, src in IBP_UNARY.items():
        print(f"[case] ibp {kind} against the executed reference", flush=True)
        y = getattr(gpu_interval(src), kind)()
        assert float(y.lw.abs().max()) == 0.0 and float(y.uw.abs().max()) == 0.0
        assert_interval(y.lb, y.ub, kind, f"ibp {kind}")
    x = gpu_interval("ibp_in")
    y = x.matmul(t(G["ibp_W"]).cuda())
    assert_interval(y.lb, y.ub, "matmul", "ibp matmul")
    normalizer = SimpleNamespace(weight=t(G["ibp_norm_weight"]).cuda(), bias=t(G["ibp_norm_bias"]).cuda())
    z = x.layer_norm(normalizer, "no_var")
    assert_interval(z.lb, z.ub, "layernorm_novar", "ibp layer_norm")
