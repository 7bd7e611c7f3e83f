"""Writes tests/golden/bounds_small.npz: tiny seeded inputs and their expected outputs.

The reference holds no golden vectors for this path (its only op test draws random inputs at
run time).  The expected values here are produced by oracle/closed_form.py -- the independent
float64 per-neuron / brute-force restatement -- not by the tensorised oracle and not by the
HIP path, so both of those can be checked against this file.  These are a second reading of
the reference, not the reference: what the reference itself returns is in reference_vectors.npz
(make_reference_golden.py) and bounds_reference_vectors.npz (make_bounds_golden.py), written by
executing its own code.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import closed_form as C  # noqa: E402

INF = float("inf")


def bounds(rng, L, D, H, sw=0.4, sb=1.2):
    lw = rng.uniform(-sw, sw, (L, D, H)).astype(np.float32)
    uw = (lw + rng.uniform(0, 0.05, (L, D, H))).astype(np.float32)
    lb = rng.uniform(-sb, sb, (L, H)).astype(np.float32)
    ub = (lb + rng.uniform(0, 0.4, (L, H))).astype(np.float32)
    return lw, lb, uw, ub


def main():
    rng = np.random.default_rng(20240229)
    out = {}
    L, D, H, N = 2, 8, 6, 5
    lw, lb, uw, ub = bounds(rng, L, D, H)
    out.update(act_lw=lw, act_lb=lb, act_uw=uw, act_ub=ub)
    for pname, p in (("p1", 1.0), ("p2", 2.0), ("pinf", INF)):
        for words in (1, 2):
            iv = np.zeros((2, L, H))
            for kind, fn in (("relu", C.relu_neuron), ("tanh", C.tanh_neuron)):
                res = [np.zeros((L, D, H)), np.zeros((L, H)), np.zeros((L, D, H)), np.zeros((L, H))]
                for l in range(L):
                    for j in range(H):
                        e = fn(lw[l, :, j], lb[l, j], uw[l, :, j], ub[l, j], p, 0.15, words)
                        res[0][l, :, j], res[1][l, j], res[2][l, :, j], res[3][l, j] = e
                        iv[:, l, j] = C.interval(lw[l, :, j], lb[l, j], uw[l, :, j], ub[l, j], p, 0.15, words)
                for nm, r in zip(("lw", "lb", "uw", "ub"), res):
                    out[f"{kind}_{pname}_w{words}_{nm}"] = r
            out[f"interval_{pname}_w{words}"] = iv
    # linear
    W = rng.normal(0, 0.5, (N, H)).astype(np.float32)
    W[0, 0] = 0.0
    bias = rng.normal(0, 0.1, N).astype(np.float32)
    out.update(lin_W=W, lin_bias=bias)
    for nm, r in zip(("lw", "lb", "uw", "ub"), C.linear_brute(lw, lb, uw, ub, W, bias)):
        out[f"lin_{nm}"] = r
    # dot product: x [3, 4, 5], y [2, 4, 5]
    x = bounds(rng, 3, 4, 5)
    y = bounds(rng, 2, 4, 5)
    for nm, a in zip(("lw", "lb", "uw", "ub"), x):
        out[f"dot_x_{nm}"] = a
    for nm, a in zip(("lw", "lb", "uw", "ub"), y):
        out[f"dot_y_{nm}"] = a
    for pname, p in (("p1", 1.0), ("p2", 2.0), ("pinf", INF)):
        for nm, r in zip(("lw", "lb", "uw", "ub"), C.dot_brute(*x, *y, p, 0.2, 1)):
            out[f"dot_{pname}_{nm}"] = r
    # conv: D=3 images of [2, 6, 7], 3x3 stride 1 pad 1 and stride 2 pad 0, 4 output channels
    cl = rng.normal(0, 0.3, (3, 2, 6, 7)).astype(np.float32)
    cu = (cl + rng.uniform(0, 0.05, cl.shape)).astype(np.float32)
    bl = rng.normal(0, 1, (1, 2, 6, 7)).astype(np.float32)
    bu = (bl + rng.uniform(0, 0.3, bl.shape)).astype(np.float32)
    Wc = rng.normal(0, 0.4, (4, 2, 3, 3)).astype(np.float32)
    Wc[1, 1, 1, 1] = 0.0
    out.update(conv_lw=cl, conv_uw=cu, conv_lb=bl, conv_ub=bu, conv_W=Wc)
    for tag, s, pd in (("s1p1", 1, 1), ("s2p0", 2, 0)):
        out[f"conv_{tag}_lw"], out[f"conv_{tag}_uw"] = C.conv_brute(cl, cu, Wc, s, pd)
        out[f"conv_{tag}_lb"], out[f"conv_{tag}_ub"] = C.conv_brute(bl, bu, Wc, s, pd)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "bounds_small.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
