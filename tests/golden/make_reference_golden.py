"""Writes tests/golden/reference_vectors.npz by EXECUTING the reference's own pure-torch code.

Runs in the build container only (it reads /root/reference, which exists nowhere else); the
tests load the .npz it leaves and never this script.  The three files

    HandTunedKernels/python_reference_code/relu_reference.py         (concretize, new, add_linear, relu)
    HandTunedKernels/python_reference_code/matmul_reference.py       (matmul, 2-D weight)
    HandTunedKernels/python_reference_code/dot_product_reference.py  (concretize, get_bounds_xy, dot_product)

import nothing but torch and carry the same method bodies as Verifiers/Bounds.py (which needs tvm and
nvcc at import and cannot be loaded).  They are loaded from where they lie with importlib, given a
two-field `args` stub (method, perturbed_words) and CPU tensors, and their outputs are stored next
to the inputs.  What this pins that no invariant can: the choices among sound alternatives -- ReLU's
lower slope [|u| > |l|], the strict comparisons at l = 0 / u = 0, k <= 0 switching the source line,
McCormick's beta_u = l_x, the index mapping of the dot product's reshapes, the order of the words
in concretize.  tanh, exp and the convolution have no importable reference and are not in the file.

    python tests/golden/make_reference_golden.py
"""
import importlib.util
import os
import types

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/HandTunedKernels/python_reference_code"
INF = float("inf")
PS = (("p1", 1.0), ("p2", 2.0), ("pinf", INF))


def load(name):
    spec = importlib.util.spec_from_file_location("faith_ref_" + name, os.path.join(REF, name + ".py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def args(words):
    return types.SimpleNamespace(method="baf", perturbed_words=words)


def draw(g, B, L, D, H, sw=0.4, sb=1.2, gw=0.05, gb=0.4):
    lw = (torch.rand(B, L, D, H, generator=g) - 0.5) * 2 * sw
    uw = lw + torch.rand(B, L, D, H, generator=g) * gw
    lb = (torch.rand(B, L, H, generator=g) - 0.5) * 2 * sb
    ub = lb + torch.rand(B, L, H, generator=g) * gb
    return lw, lb, uw, ub


def put(out, tag, lw, lb, uw, ub):
    for k, v in zip(("lw", "lb", "uw", "ub"), (lw, lb, uw, ub)):
        out[f"{tag}_{k}"] = v.detach().numpy().astype(np.float32)


def main():
    torch.manual_seed(0)
    torch.set_num_threads(1)
    g = torch.Generator().manual_seed(20250117)
    out = {}
    R = load("relu_reference")
    M = load("matmul_reference")
    Dt = load("dot_product_reference")

    # ---- relu + concretize: random neurons (all three branches occur) and crafted edge neurons ----
    L, D, H = 4, 32, 32
    lw, lb, uw, ub = draw(g, 1, L, D, H)
    # neurons 0..7 of every row: zero coefficients, so [l, u] = [lb, ub] exactly for every p
    edge = [(0.0, 1.0), (-1.0, 0.0), (-0.5, 0.5), (-0.25, 0.5), (-0.5, 0.25), (0.0, 0.0), (0.75, 1.5), (-1.5, -0.75)]
    for j, (a, b) in enumerate(edge):
        lw[:, :, :, j] = 0
        uw[:, :, :, j] = 0
        lb[:, :, j] = a
        ub[:, :, j] = b
    put(out, "act_in", lw, lb, uw, ub)
    out["act_eps"] = np.float32(0.15)
    for pname, p in PS:
        for words in (1, 2):
            x = R.Bounds(args(words), p, 0.15, lw=lw.clone(), lb=lb.clone(), uw=uw.clone(), ub=ub.clone())
            lo, hi = x.concretize()
            out[f"conc_{pname}_w{words}_l"] = lo.numpy()
            out[f"conc_{pname}_w{words}_u"] = hi.numpy()
            y = x.relu()
            put(out, f"relu_{pname}_w{words}", y.lw, y.lb, y.uw, y.ub)

    # ---- matmul: 2-D weight with exact zeros, positive and negative entries ----
    N = 24
    W = torch.randn(N, H, generator=g) / 4
    W[torch.rand(N, H, generator=g) < 0.2] = 0.0
    out["lin_W"] = W.numpy()
    x = M.Bounds(args(1), 2.0, 0.15, lw=lw.clone(), lb=lb.clone(), uw=uw.clone(), ub=ub.clone())
    y = x.matmul(W)
    put(out, "lin", y.lw, y.lb, y.uw, y.ub)

    # ---- dot product: two heads, Lx != Ly, D > 1 for every norm and word count; then D = 1 ----
    B, Lx, Ly, Dd, d = 2, 4, 3, 8, 16
    xq = draw(g, B, Lx, Dd, d, sw=0.3, sb=1.0, gw=0.05, gb=0.3)
    yk = draw(g, B, Ly, Dd, d, sw=0.3, sb=1.0, gw=0.05, gb=0.3)
    put(out, "dot_x", *xq)
    put(out, "dot_y", *yk)
    out["dot_eps"] = np.float32(0.2)
    for pname, p in PS:
        for words in (1, 2):
            a = Dt.Bounds(args(words), p, 0.2, lw=xq[0].clone(), lb=xq[1].clone(), uw=xq[2].clone(), ub=xq[3].clone())
            b = Dt.Bounds(args(words), p, 0.2, lw=yk[0].clone(), lb=yk[1].clone(), uw=yk[2].clone(), ub=yk[3].clone())
            z = a.dot_product(b)
            put(out, f"dot_{pname}_w{words}", z.lw, z.lb, z.uw, z.ub)
    x1 = draw(g, B, Lx, 1, d, sw=0.0, gw=0.0)
    y1 = draw(g, B, Ly, 1, d, sw=0.0, gw=0.0)
    put(out, "dot1_x", *x1)
    put(out, "dot1_y", *y1)
    a = Dt.Bounds(args(1), 2.0, 0.2, lw=x1[0].clone(), lb=x1[1].clone(), uw=x1[2].clone(), ub=x1[3].clone())
    b = Dt.Bounds(args(1), 2.0, 0.2, lw=y1[0].clone(), lb=y1[1].clone(), uw=y1[2].clone(), ub=y1[3].clone())
    z = a.dot_product(b)
    put(out, "dot1", z.lw, z.lb, z.uw, z.ub)

    path = os.path.join(HERE, "reference_vectors.npz")
    np.savez_compressed(path, **out)
    print(f"wrote {path}: {len(out)} arrays, {os.path.getsize(path)} bytes, torch {torch.__version__}")


if __name__ == "__main__":
    main()
