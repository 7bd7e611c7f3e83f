"""Writes tests/golden/bounds_reference_vectors.npz by EXECUTING the reference's own `Bounds` class.

Runs in the build container only (it reads /root/reference, which exists nowhere else); the tests load the
.npz it leaves and never this script.

    Transformer_Verification_Code/Verifiers/Bounds.py

cannot be imported as a module: its first statements import tvm (absent here) and JIT-compile the CUDA
kernels with nvcc from a path on the author's machine (Bounds.py:7-26).  Nothing else in the file needs either
as long as the `cuda_*`, `tvm_*` and `ansor_*` methods are not called.  So the file is read from where it lies,
parsed, and executed WITHOUT those six top-level statements -- `from torch.utils.cpp_extension import load`,
the three tvm imports, `base_dirc = ...` and `c_bound = load(...)` -- and with nothing put in their place: no
stand-in for tvm, for the extension or for any other name.  Every other statement is the reference's, as it is.
`args` is a four-field namespace (method, perturbed_words, current_flag = 0, kernel_type = 0: flag 0 selects the
`ori_*` PyTorch bodies in the dispatchers `relu`, `tanh`, `matmul`, `dot_product`).

What this pins that neither an invariant nor the three pure-torch files of HandTunedKernels/python_reference_code
(see make_reference_golden.py) can: the choices among sound alternatives in the operators that exist only in
Bounds.py -- tanh's tangent at the midpoint for one-signed intervals, its ten bisection steps, their start
points and update order (Bounds.py:1027-1103); exp's tangent point min(mid, l + 0.99) (:970-1003); sqr's and
sqrt's lines (:860-919), reciprocal's (:1136-1161); the McCormick planes of multiply(Bounds) and divide
(:608-664); the composition and rounding order of softmax (:1005-1014) and of layer_norm in both modes
(:1111-1131); scalar multiply with a negative factor, add, context (:843-850).

    python tests/golden/make_bounds_golden.py
"""
import ast
import os
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
SOURCE = "/root/reference/Transformer_Verification_Code/Verifiers/Bounds.py"
INF = float("inf")
# (name, p, perturbed words): every norm with one word and with two
CASES = (("p1_w1", 1.0, 1), ("p2_w2", 2.0, 2), ("pinf_w1", INF, 1), ("pinf_w2", INF, 2), ("p2_w1", 2.0, 1))
NAMES = ("lw", "lb", "uw", "ub")


def needs_what_is_absent(node):
    """The six top-level statements that need tvm or nvcc (Bounds.py:7-26)."""
    if isinstance(node, ast.Import):
        return any(a.name.split(".")[0] == "tvm" for a in node.names)
    if isinstance(node, ast.ImportFrom):
        return node.module.split(".")[0] == "tvm" or node.module == "torch.utils.cpp_extension"
    if isinstance(node, ast.Assign):
        return any(isinstance(t, ast.Name) and t.id in ("c_bound", "base_dirc") for t in node.targets)
    return False


def load_reference_bounds():
    source = open(SOURCE).read()
    tree = ast.parse(source)
    dropped = [n for n in tree.body if needs_what_is_absent(n)]
    assert len(dropped) == 6, [ast.get_source_segment(source, n).split("\n")[0] for n in dropped]
    tree.body = [n for n in tree.body if not needs_what_is_absent(n)]
    space = {"__name__": "faith_reference_bounds"}
    exec(compile(tree, SOURCE, "exec"), space)
    return space["Bounds"]


def args(words, method="baf"):
    return types.SimpleNamespace(method=method, perturbed_words=words, current_flag=0, kernel_type=0)


def draw(g, L, D, H, sw=0.3, sb=1.0, gw=0.05, gb=0.4, positive=False):
    lw = (torch.rand(1, L, D, H, generator=g) - 0.5) * 2 * sw
    uw = lw + torch.rand(1, L, D, H, generator=g) * gw
    lb = (torch.rand(1, L, H, generator=g) - 0.5) * 2 * sb
    if positive:
        lb = lb.abs() + 2.0
    ub = lb + torch.rand(1, L, H, generator=g) * gb
    return lw, lb, uw, ub


def put(out, tag, *tensors):
    for k, v in zip(NAMES, tensors):
        out[f"{tag}_{k}"] = v.detach().numpy().astype(np.float32)


def main():
    torch.manual_seed(0)
    torch.set_num_threads(1)
    Bounds = load_reference_bounds()
    g = torch.Generator().manual_seed(20250215)
    out = {}

    def ref(t, p, eps, words):
        return Bounds(args(words), p, eps, lw=t[0].clone(), lb=t[1].clone(), uw=t[2].clone(), ub=t[3].clone())

    def keep(tag, y):
        put(out, tag, y.lw, y.lb, y.uw, y.ub)

    L, D, H = 2, 32, 32
    # ---- any-sign input: tanh, relu, exp, sqr, multiply, scalar multiply, matmul, add.  Neurons 0..9 of every
    # row have zero coefficients, so their interval is [lb, ub] exactly for every norm: one-signed on both sides,
    # touching zero from either side, straddling with |u| = |l|, > and <, a point, a tiny and a wide interval
    x = list(draw(g, L, D, H))
    edge = [(0.0, 1.0), (-1.0, 0.0), (-0.5, 0.5), (-0.25, 0.5), (-0.5, 0.25), (0.0, 0.0), (0.75, 1.5), (-1.5, -0.75),
            (0.3, 0.3000001), (-8.0, 9.0)]
    for j, (a, b) in enumerate(edge):
        x[0][:, :, :, j] = 0
        x[2][:, :, :, j] = 0
        x[1][:, :, j] = a
        x[3][:, :, j] = b
    put(out, "any_in", *x)
    x2 = draw(g, L, D, H)
    put(out, "any2_in", *x2)
    # ---- strictly positive input: sqrt, reciprocal, the divisor of divide
    xp = draw(g, L, D, H, sw=0.1, positive=True)
    put(out, "pos_in", *xp)
    # ---- attention-score-like input for softmax, narrow intervals for layer_norm
    xs = draw(g, L, D, 16, sw=0.05, sb=1.0, gw=0.005, gb=0.1)
    put(out, "soft_in", *xs)
    xn = draw(g, L, D, H, sw=0.05, sb=1.0, gw=0.005, gb=0.05)
    put(out, "norm_in", *xn)
    weight = 1 + 0.1 * torch.randn(H, generator=g)
    weight[3] = -0.8                                     # a negative scale swaps the sides
    bias = 0.05 * torch.randn(H, generator=g)
    out["norm_weight"], out["norm_bias"] = weight.numpy(), bias.numpy()
    normalizer = types.SimpleNamespace(weight=weight, bias=bias)
    W = torch.randn(24, H, generator=g) / 4
    W[torch.rand(24, H, generator=g) < 0.2] = 0.0
    out["lin_W"] = W.numpy()
    # ---- attention: scores of two heads, then context with values
    q = draw(g, 4, 8, 16, sw=0.3, sb=1.0, gw=0.05, gb=0.3)
    q = tuple(torch.cat([v, v * 0.5 + 0.1], 0) for v in q)          # two (batch, head) pairs
    k = draw(g, 3, 8, 16, sw=0.3, sb=1.0, gw=0.05, gb=0.3)
    k = tuple(torch.cat([v, v * 0.7 - 0.1], 0) for v in k)
    k = (k[0], k[1], k[0] + (k[2] - k[0]).abs(), k[1] + (k[3] - k[1]).abs())
    q = (q[0], q[1], q[0] + (q[2] - q[0]).abs(), q[1] + (q[3] - q[1]).abs())
    put(out, "dot_x", *q)
    put(out, "dot_y", *k)
    probs = draw(g, 4, 8, 3, sw=0.02, sb=0.3, gw=0.004, gb=0.05)
    probs = tuple(torch.cat([v, v * 0.9], 0) for v in probs)
    probs = (probs[0], probs[1].abs(), probs[0] + (probs[2] - probs[0]).abs(), probs[1].abs() + (probs[3] - probs[1]).abs())
    value = draw(g, 3, 8, 16, sw=0.3, sb=1.0, gw=0.05, gb=0.3)
    value = tuple(torch.cat([v, v * 0.6 + 0.2], 0) for v in value)
    value = (value[0], value[1], value[0] + (value[2] - value[0]).abs(), value[1] + (value[3] - value[1]).abs())
    put(out, "ctx_probs", *probs)
    put(out, "ctx_value", *value)

    out["eps"], out["eps_soft"], out["eps_norm"], out["eps_dot"] = (np.float32(v) for v in (0.1, 0.05, 0.02, 0.2))
    for tag, p, words in CASES:
        keep(f"tanh_{tag}", ref(x, p, 0.1, words).tanh())
        keep(f"relu_{tag}", ref(x, p, 0.1, words).relu())
        keep(f"exp_{tag}", ref(x, p, 0.1, words).exp())
        keep(f"sqr_{tag}", ref(x, p, 0.1, words).sqr())
        keep(f"sqrt_{tag}", ref(xp, p, 0.1, words).sqrt())
        keep(f"reciprocal_{tag}", ref(xp, p, 0.1, words).reciprocal())
        keep(f"multiply_{tag}", ref(x, p, 0.1, words).multiply(ref(x2, p, 0.1, words)))
        keep(f"divide_{tag}", ref(x, p, 0.1, words).divide(ref(xp, p, 0.1, words)))
        keep(f"softmax_{tag}", ref(xs, p, 0.05, words).softmax())
        keep(f"layernorm_novar_{tag}", ref(xn, p, 0.02, words).layer_norm(normalizer, "no_var"))
        keep(f"layernorm_standard_{tag}", ref(xn, p, 0.02, words).layer_norm(normalizer, "standard"))
        lo, hi = ref(x, p, 0.1, words).concretize()
        out[f"conc_{tag}_l"], out[f"conc_{tag}_u"] = lo.numpy(), hi.numpy()
        keep(f"dot_{tag}", ref(q, p, 0.2, words).dot_product(ref(k, p, 0.2, words)))
        keep(f"context_{tag}", ref(probs, p, 0.2, words).context(ref(value, p, 0.2, words)))
    # any other perturbation norm (dual exponents 1.5 and 3, torch.norm(p=q)): the relaxations that the
    # configurations name, and the intervals
    for tag, p, words in (("p3_w1", 3.0, 1), ("p1.5_w2", 1.5, 2)):
        keep(f"tanh_{tag}", ref(x, p, 0.1, words).tanh())
        keep(f"relu_{tag}", ref(x, p, 0.1, words).relu())
        lo, hi = ref(x, p, 0.1, words).concretize()
        out[f"conc_{tag}_l"], out[f"conc_{tag}_u"] = lo.numpy(), hi.numpy()
    # operators without a norm in them: once
    keep("matmul", ref(x, 2.0, 0.1, 1).matmul(W))
    keep("scale_neg", ref(x, 2.0, 0.1, 1).multiply(-0.7))
    keep("scale_pos", ref(x, 2.0, 0.1, 1).multiply(1.3))
    keep("add_bounds", ref(x, 2.0, 0.1, 1).add(ref(x2, 2.0, 0.1, 1)))
    keep("add_vector", ref(x, 2.0, 0.1, 1).add(bias))

    # ---- method "ibp" (interval bound propagation: the `if self.ibp` branches, Bounds.py:285-288, 863, 896, 973,
    # 1030, 1139 and the matmul / layer_norm that serve both methods).  Its relu, get_bounds_xy (product, dot
    # product) and whatever composes them call `.cuda()` on constants (Bounds.py:230, 676, 925) and cannot run in a
    # container without a GPU: those stay pinned by their closed forms (max(., 0); the range of the four corners).
    Li, Hi = 4, 24
    ilb = torch.randn(1, Li, Hi, generator=g)
    iub = ilb + torch.rand(1, Li, Hi, generator=g) * 0.6
    plb = torch.randn(1, Li, Hi, generator=g).abs() + 0.5
    pub = plb + torch.rand(1, Li, Hi, generator=g) * 0.6
    out["ibp_in_lb"], out["ibp_in_ub"] = ilb.numpy(), iub.numpy()
    out["ibp_pos_in_lb"], out["ibp_pos_in_ub"] = plb.numpy(), pub.numpy()
    Wi = torch.randn(16, Hi, generator=g) / 4
    out["ibp_W"] = Wi.numpy()
    iw = 1 + 0.1 * torch.randn(Hi, generator=g)
    iw[2] = -0.6
    ib = 0.05 * torch.randn(Hi, generator=g)
    out["ibp_norm_weight"], out["ibp_norm_bias"] = iw.numpy(), ib.numpy()

    def interval_object(lb, ub):
        zeros = torch.zeros(1, Li, 2 * Hi, Hi)             # the constructor keeps `perturbed_words` rows of it
        return Bounds(args(2, "ibp"), 2.0, 0.1, lw=zeros, lb=lb.clone(), uw=zeros.clone(), ub=ub.clone())

    def keep_interval(tag, y):
        assert float(y.lw.abs().max()) == 0.0 and float(y.uw.abs().max()) == 0.0
        out[f"ibp_{tag}_lb"], out[f"ibp_{tag}_ub"] = y.lb.numpy(), y.ub.numpy()

    for kind in ("tanh", "exp", "sqr"):
        keep_interval(kind, getattr(interval_object(ilb, iub), kind)())
    for kind in ("sqrt", "reciprocal"):
        keep_interval(kind, getattr(interval_object(plb, pub), kind)())
    keep_interval("matmul", interval_object(ilb, iub).matmul(Wi))
    keep_interval("layernorm_novar", interval_object(ilb, iub).layer_norm(types.SimpleNamespace(weight=iw, bias=ib), "no_var"))

    path = os.path.join(HERE, "bounds_reference_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes, torch {torch.__version__}")


if __name__ == "__main__":
    main()
