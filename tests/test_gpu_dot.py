"""HIP attention-score (Q.K^T) McCormick bounds against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import rand_bounds, as_bounds, close
from tests.parity import compare_contraction, CONSTANT_TERMS, UNIT_SCALE_ALL, CONFIG_RATIO

pytestmark = pytest.mark.gpu
INF = float("inf")


def dev(x):
    return tuple(t.cuda().contiguous() for t in x.tensors())


def dot64(x, y, p, eps, words, intervals=None):
    """float64 value of the planes built from fp32 concrete intervals -- the oracle's, or the (l_x, l_y, u_y)
    handed in (the ones the GPU computed and used) -- and the per-output sum of |terms|."""
    if intervals is None:
        lx, _ = O.concretize(x, p, eps, words)
        ly, uy = O.concretize(y, p, eps, words)
    else:
        lx, ly, uy = (t.detach().cpu() for t in intervals)
    lx, ly, uy = lx.double(), ly.double(), uy.double()
    X = {k: v.double() for k, v in zip(("lw", "lb", "uw", "ub"), x.tensors())}
    Y = {k: v.double() for k, v in zip(("lw", "lb", "uw", "ub"), y.tensors())}
    P, N = (lambda v: v.clamp(min=0)), (lambda v: v.clamp(max=0))
    ew = lambda a, c: torch.einsum("timk,tjk->timj", a, c)      # x-terms of the coefficients
    eyw = lambda a, c: torch.einsum("tjmk,tik->timj", a, c)     # y-terms
    eb = lambda a, c: torch.einsum("tik,tjk->tij", a, c)
    eyb = lambda a, c: torch.einsum("tjk,tik->tij", a, c)
    ref = dict(
        lw=ew(X["lw"], P(ly)) + ew(X["uw"], N(ly)) + eyw(Y["lw"], P(lx)) + eyw(Y["uw"], N(lx)),
        uw=ew(X["uw"], P(uy)) + ew(X["lw"], N(uy)) + eyw(Y["uw"], P(lx)) + eyw(Y["lw"], N(lx)),
        lb=-eb(lx, ly) + eb(X["lb"], P(ly)) + eb(X["ub"], N(ly)) + eyb(Y["lb"], P(lx)) + eyb(Y["ub"], N(lx)),
        ub=-eb(lx, uy) + eb(X["ub"], P(uy)) + eb(X["lb"], N(uy)) + eyb(Y["ub"], P(lx)) + eyb(Y["lb"], N(lx)))
    A = torch.abs
    mag = dict(
        lw=ew(A(X["lw"]), P(ly)) - ew(A(X["uw"]), N(ly)) + eyw(A(Y["lw"]), P(lx)) - eyw(A(Y["uw"]), N(lx)),
        uw=ew(A(X["uw"]), P(uy)) - ew(A(X["lw"]), N(uy)) + eyw(A(Y["uw"]), P(lx)) - eyw(A(Y["lw"]), N(lx)),
        lb=eb(A(lx), A(ly)) + eb(A(X["lb"]), P(ly)) - eb(A(X["ub"]), N(ly)) + eyb(A(Y["lb"]), P(lx)) - eyb(A(Y["ub"]), N(lx)),
        ub=eb(A(lx), A(uy)) + eb(A(X["ub"]), P(uy)) - eb(A(X["lb"]), N(uy)) + eyb(A(Y["ub"]), P(lx)) - eyb(A(Y["lb"]), N(lx)))
    return ref, mag


def check(x, y, p, eps, words, what="", allow=None, ratio_ceiling=None):
    from faith_amd import ops
    print(f"[case] dot {what} x={tuple(x.lw.shape)} y={tuple(y.lw.shape)} p={p} eps={eps} words={words}", flush=True)
    zlw, zlb, zuw, zub, (xl, xu, yl, yu) = ops.dot_product_qk(dev(x), dev(y), p, eps, words, return_intervals=True)
    torch.cuda.synchronize()
    exp = O.dot_product(x, y, p, eps, words)
    exl, exu = O.concretize(x, p, eps, words)
    eyl, eyu = O.concretize(y, p, eps, words)
    assert close(xl, exl) and close(xu, exu) and close(yl, eyl) and close(yu, eyu)
    if x.lw.shape[2] == 1:      # interval shortcut: the result does not use the intervals, which are written all the same
        for g, e in zip((zlw, zlb, zuw, zub), exp.tensors()):
            assert close(g, e)
        return
    ref, mag = dot64(x, y, p, eps, words)
    own, _ = dot64(x, y, p, eps, words, intervals=(xl, yl, yu))
    for name, g, e in zip(("lw", "lb", "uw", "ub"), (zlw, zlb, zuw, zub), exp.tensors()):
        compare_contraction(name, g, e, ref[name], mag[name], allow, ref64_own=own[name], ratio_ceiling=ratio_ceiling)
    return zlw, zlb, zuw, zub


@pytest.mark.parametrize("shape", [
    (1, 2, 2, 64, 16), (2, 8, 8, 64, 64), (4, 16, 16, 128, 64),     # reference sweep corners (d = 16 included)
    (1, 130, 70, 20, 32),       # Lx, Ly off the 128 tile; Lx != Ly
    (2, 5, 9, 7, 12),           # tiny, ragged
    (1, 6, 4, 5, 10),           # d % 4 != 0: any-shape kernel
    (2, 3, 5, 1, 8),            # dim_in == 1: interval shortcut
])
@pytest.mark.parametrize("p", [1.0, 2.0, INF, 3.0])
def test_dot_shapes(shape, p):
    B, Lx, Ly, D, d = shape
    g = torch.Generator().manual_seed(31)
    x = rand_bounds(g, B, Lx, D, d, ordered=False, sw=0.3, sb=1.0)
    y = rand_bounds(g, B, Ly, D, d, ordered=False, sw=0.3, sb=1.0)
    check(x, y, p, 0.1, 1, "sweep", UNIT_SCALE_ALL)


def test_dot_two_words():
    g = torch.Generator().manual_seed(32)
    x = rand_bounds(g, 2, 12, 64, 32, sw=0.2)
    y = rand_bounds(g, 2, 12, 64, 32, sw=0.2)
    check(x, y, 2.0, 0.05, 2, "words=2", UNIT_SCALE_ALL)


def test_dot_config3_reduced():
    """Benchmark configuration 3 with L = 32 instead of 128 (4 heads, D_in = 256, d = 64)."""
    from faith_amd.workloads import make_config
    c = make_config(3, scale=0.25)
    check(as_bounds(c["x"]), as_bounds(c["y"]), c["p"], c["eps"], c["words"], "config3/4", CONSTANT_TERMS, ratio_ceiling=CONFIG_RATIO)


@pytest.mark.parametrize("shape", [
    # B, Lx, Ly, D, d: shapes the straight-line contraction kernel takes (d % 8 == 0, Lx % 128 == 0, Ly % 64 == 0)
    (1, 128, 128, 8, 64),      # results of a tile leave during the next tile's first seven K-steps
    (1, 128, 64, 4, 128),      # sixteen K-steps: unrolled seven, then the rolled loop
    (1, 128, 64, 8, 32),       # four K-steps: too few for piecewise stores
    (2, 128, 128, 160, 16),    # 640 tiles on 512 workgroups: a workgroup walks from one tile to the next
    (1, 256, 128, 12, 64),     # two i-tiles; dim_in not a multiple of 8 (plain tile numbering)
])
def test_dot_exact_shapes_against_float64(shape):
    """The whole result against the float64 planes (the CPU oracle's broadcast would be too large here)."""
    from faith_amd import ops
    B, Lx, Ly, D, d = shape
    g = torch.Generator().manual_seed(35)
    x = rand_bounds(g, B, Lx, D, d, ordered=False, sw=0.3, sb=1.0)
    y = rand_bounds(g, B, Ly, D, d, ordered=False, sw=0.3, sb=1.0)
    print(f"[case] dot exact x={tuple(x.lw.shape)} y={tuple(y.lw.shape)}", flush=True)
    zlw, zlb, zuw, zub, (xl, xu, yl, yu) = ops.dot_product_qk(dev(x), dev(y), 2.0, 0.05, 1, return_intervals=True)
    torch.cuda.synchronize()
    exl, exu = O.concretize(x, 2.0, 0.05, 1)
    eyl, eyu = O.concretize(y, 2.0, 0.05, 1)
    assert close(xl, exl) and close(xu, exu) and close(yl, eyl) and close(yu, eyu)
    ref, mag = dot64(x, y, 2.0, 0.05, 1)
    tol = lambda r, m: 1e-6 + 1e-5 * r.abs() + 8 * 2.0 ** -24 * m
    for name, got in (("lw", zlw), ("lb", zlb), ("uw", zuw), ("ub", zub)):
        err = (got.cpu().double() - ref[name]).abs()
        assert bool((err <= tol(ref[name], mag[name])).all()), f"{name}: max err {float(err.max()):.3g}"


def test_dot_config3_full_size_properties():
    """Full configuration 3: soundness of the propagated planes on sampled perturbations
    (any x, y inside their bounds => x.y^T inside z's bounds), plus one head against float64."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(3)
    x, y = as_bounds(c["x"]), as_bounds(c["y"])
    zlw, zlb, zuw, zub = ops.dot_product_qk(dev(x), dev(y), c["p"], c["eps"], c["words"])
    torch.cuda.synchronize()
    g = torch.Generator().manual_seed(3)
    D, eps = 256, c["eps"]
    delta = (torch.sign(torch.randn(8, D, generator=g)) * eps).double().cuda()      # corners of the inf-ball
    t = 1
    X = [v[t].double().cuda() for v in x.tensors()]
    Y = [v[t].double().cuda() for v in y.tensors()]
    ev = lambda w, b: torch.einsum("nm,imk->nik", delta, w) + b
    xl, xu, yl, yu = ev(X[0], X[1]), ev(X[2], X[3]), ev(Y[0], Y[1]), ev(Y[2], Y[3])
    zl = torch.einsum("nm,imj->nij", delta, zlw[t].double()) + zlb[t].double()
    zu = torch.einsum("nm,imj->nij", delta, zuw[t].double()) + zub[t].double()
    for tx, ty in [(0, 0), (1, 1), (0, 1), (0.5, 0.25)]:
        prod = torch.einsum("nik,njk->nij", xl + tx * (xu - xl), yl + ty * (yu - yl))
        assert bool((prod >= zl - 1e-4).all()) and bool((prod <= zu + 1e-4).all())
    # head 1 against the float64 planes
    one = lambda b: O.LinearBounds(*(v[t:t + 1] for v in b.tensors()))
    ref, mag = dot64(one(x), one(y), c["p"], c["eps"], c["words"])
    tol = lambda r, m: 1e-6 + 1e-5 * r.abs() + 8 * 2.0 ** -24 * m
    assert bool(((zlw[t].cpu().double() - ref["lw"][0]).abs() <= tol(ref["lw"][0], mag["lw"][0])).all())
    assert bool(((zub[t].cpu().double() - ref["ub"][0]).abs() <= tol(ref["ub"][0], mag["ub"][0])).all())


# ------------------------------------------------------------------ context path (probs . value)
def check_v(probs, value, p, eps, words, what="", allow=None):
    from faith_amd import ops
    print(f"[case] context {what} probs={tuple(probs.lw.shape)} value={tuple(value.lw.shape)} p={p} eps={eps}", flush=True)
    zlw, zlb, zuw, zub, (xl, xu, yl, yu) = ops.dot_product_v(dev(probs), dev(value), p, eps, words,
                                                             return_intervals=True)
    torch.cuda.synchronize()
    exp = O.context(probs, value, p, eps, words)
    el, eu = O.concretize(value, p, eps, words)
    assert close(yl, el) and close(yu, eu)
    epl, epu = O.concretize(probs, p, eps, words)
    assert close(xl, epl) and close(xu, epu)
    if probs.lw.shape[2] == 1:
        for g, e in zip((zlw, zlb, zuw, zub), exp.tensors()):
            assert close(g, e)
        return
    ref, mag = dot64(probs, O.transpose_bounds(value), p, eps, words)
    own, _ = dot64(probs, O.transpose_bounds(value), p, eps, words, intervals=(xl, yl.transpose(1, 2), yu.transpose(1, 2)))
    for name, g, e in zip(("lw", "lb", "uw", "ub"), (zlw, zlb, zuw, zub), exp.tensors()):
        assert g.shape == e.shape
        compare_contraction(name, g, e, ref[name], mag[name], allow, ref64_own=own[name])


@pytest.mark.parametrize("shape", [
    # B, L (queries = keys), D, dim_out of the values
    (1, 2, 64, 16), (2, 16, 64, 64), (2, 32, 32, 20),
    (1, 130, 12, 72),      # L off the tile in both roles
    (2, 8, 5, 12),         # tiny
    (1, 6, 4, 10),         # value width % 4 != 0: any-shape kernel
    (1, 5, 3, 8),          # key length % 4 != 0: any-shape kernel
    (2, 4, 1, 8),          # dim_in == 1: interval shortcut
])
@pytest.mark.parametrize("p", [1.0, 2.0, INF, 3.0])
def test_context_shapes(shape, p):
    B, L, D, dv = shape
    g = torch.Generator().manual_seed(33)
    probs = rand_bounds(g, B, L, D, L, ordered=False, sw=0.2, sb=0.5)
    value = rand_bounds(g, B, L, D, dv, ordered=False, sw=0.3, sb=1.0)
    check_v(probs, value, p, 0.1, 1, "sweep", UNIT_SCALE_ALL)


@pytest.mark.parametrize("shape", [
    # B, queries, keys, D, value width: shapes the straight-line kernel takes on the context path
    (1, 128, 128, 8, 64), (2, 128, 64, 16, 128), (1, 128, 32, 160, 64),
])
def test_context_exact_shapes(shape):
    B, Lq, Lk, D, dv = shape
    g = torch.Generator().manual_seed(36)
    probs = rand_bounds(g, B, Lq, D, Lk, ordered=False, sw=0.2, sb=0.5)
    value = rand_bounds(g, B, Lk, D, dv, ordered=False, sw=0.3, sb=1.0)
    check_v(probs, value, 2.0, 0.05, 1, "exact", UNIT_SCALE_ALL)


@pytest.mark.parametrize("shape", [
    # B, queries, keys, D, value width: any number of key positions (the length of a sentence) on the per-wavefront
    # kernel's ragged mode -- staged operands zero beyond the last key, x read 4 bytes at a time
    (4, 30, 30, 64, 64), (2, 23, 23, 32, 64), (1, 36, 36, 16, 32), (1, 40, 77, 8, 16), (2, 33, 20, 24, 64),
    (1, 7, 1, 8, 8), (1, 31, 31, 16, 10), (1, 130, 30, 4, 64),
])
@pytest.mark.parametrize("words", [1, 2])
def test_context_any_number_of_keys(shape, words):
    B, Lq, Lk, D, dv = shape
    g = torch.Generator().manual_seed(37)
    probs = rand_bounds(g, B, Lq, D, Lk, ordered=False, sw=0.2, sb=0.5)
    value = rand_bounds(g, B, Lk, D, dv, ordered=False, sw=0.3, sb=1.0)
    check_v(probs, value, 2.0, 0.05, words, "any number of keys", UNIT_SCALE_ALL)


def test_context_rectangular_and_two_words():
    """More keys than queries, two perturbed words."""
    g = torch.Generator().manual_seed(34)
    probs = rand_bounds(g, 2, 12, 64, 40, sw=0.2, sb=0.5)      # 12 queries over 40 keys
    value = rand_bounds(g, 2, 40, 64, 32, sw=0.2)
    check_v(probs, value, 2.0, 0.05, 2, "Lx != Lk, words=2", UNIT_SCALE_ALL)


def test_bounds_class_dispatches_context_to_the_native_kernel():
    """Bounds.context(value) == dot_product(value.t()) and matches the oracle; the transposed
    object is never materialised (reference: Bounds.py:833-850)."""
    from faith_amd import Bounds
    g = torch.Generator().manual_seed(35)
    probs = rand_bounds(g, 2, 16, 32, 16, sw=0.2, sb=0.5)
    value = rand_bounds(g, 2, 16, 32, 24, sw=0.2)
    bp = Bounds(None, 2.0, 0.05, lw=probs.lw.cuda(), lb=probs.lb.cuda(), uw=probs.uw.cuda(), ub=probs.ub.cuda())
    bv = Bounds(None, 2.0, 0.05, lw=value.lw.cuda(), lb=value.lb.cuda(), uw=value.uw.cuda(), ub=value.ub.cuda())
    z = bp.context(bv)
    exp = O.context(probs, value, 2.0, 0.05)
    ref, mag = dot64(probs, O.transpose_bounds(value), 2.0, 0.05, 1)
    for name, g_, e in zip(("lw", "lb", "uw", "ub"), (z.lw, z.lb, z.uw, z.ub), exp.tensors()):
        compare_contraction(name, g_, e, ref[name], mag[name], UNIT_SCALE_ALL)
    # scores path through the class as well
    s = bp.dot_product(bp)
    es = O.dot_product(probs, probs, 2.0, 0.05)
    rs, ms = dot64(probs, probs, 2.0, 0.05, 1)
    for name, g_, e in zip(("lw", "lb", "uw", "ub"), (s.lw, s.lb, s.uw, s.ub), es.tensors()):
        compare_contraction(name, g_, e, rs[name], ms[name], UNIT_SCALE_ALL)


def test_c_bound_dot_shims():
    """Reference calling convention of the two dot-product entries (kernel.cpp:133-241): transposed
    operands, caller-allocated outputs, z_lw as [B, L, L|dim_out, dim_in]."""
    from faith_amd import c_bound
    g = torch.Generator().manual_seed(36)
    B, L, D, d = 2, 8, 16, 12
    x = rand_bounds(g, B, L, D, d, sw=0.2); y = rand_bounds(g, B, L, D, d, sw=0.2)
    T = lambda t_: t_.cuda().transpose(2, 3).contiguous()
    z = lambda *s_: torch.zeros(*s_, device="cuda")
    x_l, y_l, x_u, y_u = z(B, L, d), z(B, L, d), z(B, L, d), z(B, L, d)
    zlb, zub, zlw, zuw = z(B, L, L), z(B, L, L), z(B, L, L, D), z(B, L, L, D)
    c_bound.p, c_bound.words = 2.0, 1
    c_bound.c_dot_product_verification_QK(x_l, y_l, x_u, y_u, x.lb.cuda(), x.ub.cuda(), y.lb.cuda(), y.ub.cuda(),
                                          T(x.lw), T(x.uw), T(y.lw), T(y.uw), zlb, zub, zlw, zuw, B, L, d, D, 0.05)
    e = O.dot_product(x, y, 2.0, 0.05)
    assert close(zlw.transpose(2, 3), e.lw, rtol=1e-5, atol=2e-6) and close(zub, e.ub, rtol=1e-5, atol=2e-6)
    # context: probs [B, L, D, L], value [B, L, D, dv] handed over as the reference's adapter does
    dv = 20
    probs = rand_bounds(g, B, L, D, L, sw=0.2, sb=0.5); value = rand_bounds(g, B, L, D, dv, sw=0.2)
    vt = O.transpose_bounds(value)                         # lw [B, dv, D, L], lb [B, dv, L]
    x_l, x_u = z(B, L, L), z(B, L, L)
    y_l, y_u = z(B, dv, L), z(B, dv, L)
    zlb, zub, zlw, zuw = z(B, L, dv), z(B, L, dv), z(B, L, dv, D), z(B, L, dv, D)
    c_bound.c_dot_product_verification_V(x_l, y_l, x_u, y_u, probs.lb.cuda(), probs.ub.cuda(),
                                         vt.lb.cuda().contiguous(), vt.ub.cuda().contiguous(),
                                         T(probs.lw), T(probs.uw), T(vt.lw), T(vt.uw),
                                         zlb, zub, zlw, zuw, B, L, dv, D, 0.05)
    e = O.context(probs, value, 2.0, 0.05)
    assert close(zlw.transpose(2, 3), e.lw, rtol=1e-5, atol=2e-6) and close(zlb, e.lb, rtol=1e-5, atol=2e-6)
    assert close(zuw.transpose(2, 3), e.uw, rtol=1e-5, atol=2e-6) and close(zub, e.ub, rtol=1e-5, atol=2e-6)


@pytest.mark.parametrize("p", [2.0, INF, 1.0, 3.0])
@pytest.mark.parametrize("shape", [
    # B, Lx, Ly, D, d (scores) / B, Lx, Lk, D, dv (context); words
    (2, 8, 8, 16, 12, 1),         # D_in below a wavefront: the four wavefronts of a workgroup along the columns
    (1, 5, 9, 100, 20, 2),        # two wavefronts along m, ragged rows, columns and lanes
    (4, 32, 32, 256, 64, 1),      # configuration-3 operands at a quarter of the length: whole blocks everywhere, the MFMA kernels
    (4, 32, 32, 256, 64, -1),     # the same on the vector-ALU kernel (tuning knob): four wavefronts along m
    (1, 128, 128, 64, 64, 1),     # MFMA kernels: four row blocks per wavefront, dim_in of two wavefronts (two stay idle)
    (2, 64, 96, 160, 32, 2),      # MFMA kernels: 96 rows as three passes of one block, a partly filled second block of dim_in
    (1, 3, 70, 300, 7, 3),        # D_in beyond one workgroup's 256 lanes, more columns than a workgroup takes
    (2, 6, 4, 1, 10, 1),          # dim_in == 1: the interval shortcut
])
def test_dot_products_in_the_reference_layout_through_the_c_abi(shape, p):
    """faith_dot_product_verification_QK / _V with FAITH_LAYOUT_TRANSPOSED, called as a C binder would call them
    (raw pointers through the C ABI): operands [B, L, dim_out, dim_in], z_lw [B, Lx, Ly, dim_in], exactly the
    tensors the reference's adapters build (Bounds.py:1279-1290, 1319-1329); against the oracle."""
    import ctypes
    from faith_amd import _lib, ops
    B, Lx, L2, D, d, words = shape
    vector_alu = words < 0
    words = abs(words)
    g = torch.Generator().manual_seed(37)
    eps = 0.05
    P = lambda t_: ctypes.c_void_p(t_.data_ptr())
    T = lambda t_: t_.cuda().transpose(2, 3).contiguous()
    nan = lambda *s_: torch.full(s_, float("nan"), device="cuda")
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call(entry, x, y, Ly, K, y_shape):
        x_l, x_u = nan(B, Lx, K), nan(B, Lx, K)
        y_l, y_u = nan(*y_shape), nan(*y_shape)
        zlb, zub, zlw, zuw = nan(B, Lx, Ly), nan(B, Lx, Ly), nan(B, Lx, Ly, D), nan(B, Lx, Ly, D)
        ops_ = [x.lb.cuda().contiguous(), x.ub.cuda().contiguous(), y.lb.cuda().contiguous(), y.ub.cuda().contiguous(),
                T(x.lw), T(x.uw), T(y.lw), T(y.uw)]
        dims = (B, Lx, Ly, K, D) if entry.endswith("QK") else (B, Lx, K, Ly, D)
        if vector_alu:
            _lib.call("faith_tune_set", 2, 3)
        try:
            _lib.call(entry, P(x_l), P(y_l), P(x_u), P(y_u), *(P(t_) for t_ in ops_), P(zlb), P(zub), P(zlw), P(zuw),
                      *dims, eps, ops.q_code(p), words, _lib.LAYOUT_TRANSPOSED, stream)
            torch.cuda.synchronize()
        finally:
            if vector_alu:
                _lib.call("faith_tune_set", 2, 0)
        return (zlw.transpose(2, 3), zlb, zuw.transpose(2, 3), zub), (x_l, x_u, y_l, y_u)

    # scores: x [B, Lx, D, d], y [B, L2, D, d]
    x, y = rand_bounds(g, B, Lx, D, d, sw=0.2), rand_bounds(g, B, L2, D, d, sw=0.2)
    print(f"[case] transposed-layout QK {shape} p={p}", flush=True)
    got, (x_l, x_u, y_l, y_u) = call("faith_dot_product_verification_QK", x, y, L2, d, (B, L2, d))
    exp = O.dot_product(x, y, p, eps, words)
    exl, exu = O.concretize(x, p, eps, words)
    eyl, eyu = O.concretize(y, p, eps, words)
    assert close(x_l, exl) and close(x_u, exu) and close(y_l, eyl) and close(y_u, eyu)
    if D == 1:
        for a, e in zip(got, exp.tensors()):
            assert close(a, e)
    else:
        ref, mag = dot64(x, y, p, eps, words)
        for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
            assert a.shape == e.shape
            compare_contraction(name, a, e, ref[name], mag[name], UNIT_SCALE_ALL)

    # context: probabilities [B, Lx, D, Lk = L2], values [B, Lk, D, dv = d]; y is handed over as value.t()
    probs, value = rand_bounds(g, B, Lx, D, L2, sw=0.2, sb=0.5), rand_bounds(g, B, L2, D, d, sw=0.2)
    vt = O.transpose_bounds(value)                         # lw [B, dv, D, Lk], lb [B, dv, Lk]
    print(f"[case] transposed-layout V {shape} p={p}", flush=True)
    got, (x_l, x_u, y_l, y_u) = call("faith_dot_product_verification_V", probs, vt, d, L2, (B, d, L2))
    exp = O.context(probs, value, p, eps, words)
    epl, epu = O.concretize(probs, p, eps, words)
    evl, evu = O.concretize(vt, p, eps, words)
    assert close(x_l, epl) and close(x_u, epu) and close(y_l, evl) and close(y_u, evu)
    if D == 1:
        for a, e in zip(got, exp.tensors()):
            assert close(a, e)
    else:
        ref, mag = dot64(probs, vt, p, eps, words)
        for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
            assert a.shape == e.shape
            compare_contraction(name, a, e, ref[name], mag[name], UNIT_SCALE_ALL)


@pytest.mark.parametrize("layout", ["natural", "transposed"])
@pytest.mark.parametrize("shape", [(2, 40, 24, 96, 32, 2), (4, 128, 128, 64, 64, 1), (1, 6, 4, 1, 10, 1)])
def test_dot_product_without_the_upper_interval_of_x(shape, layout):
    """x_u = NULL through the C ABI: nothing reads the upper interval of x (the planes take x from below on both
    sides, Bounds.py:761-762; the reference's adapter drops the array, Bounds.py:1274-1296), so the entry points
    accept its absence.  Everything else -- z and the three other intervals -- is bit for bit what the call with
    x_u gives."""
    import ctypes
    from faith_amd import _lib, ops
    B, Lx, Ly, D, d, words = shape
    g = torch.Generator().manual_seed(41)
    x, y = rand_bounds(g, B, Lx, D, d, sw=0.2), rand_bounds(g, B, Ly, D, d, sw=0.2)
    P = lambda t_: None if t_ is None else ctypes.c_void_p(t_.data_ptr())
    lay = (lambda t_: t_.cuda().contiguous()) if layout == "natural" else (lambda t_: t_.cuda().transpose(2, 3).contiguous())
    code = _lib.LAYOUT_NATURAL if layout == "natural" else _lib.LAYOUT_TRANSPOSED
    nan = lambda *s_: torch.full(s_, float("nan"), device="cuda")
    operands = [x.lb.cuda().contiguous(), x.ub.cuda().contiguous(), y.lb.cuda().contiguous(), y.ub.cuda().contiguous(),
                lay(x.lw), lay(x.uw), lay(y.lw), lay(y.uw)]
    zshape = (B, Lx, D, Ly) if layout == "natural" else (B, Lx, Ly, D)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def call(with_xu):
        x_l, x_u, y_l, y_u = nan(B, Lx, d), (nan(B, Lx, d) if with_xu else None), nan(B, Ly, d), nan(B, Ly, d)
        z = [nan(B, Lx, Ly), nan(B, Lx, Ly), nan(*zshape), nan(*zshape)]
        print(f"[case] dot product {layout} {shape} x_u={'given' if with_xu else 'NULL'}", flush=True)
        _lib.call("faith_dot_product_verification_QK", P(x_l), P(y_l), P(x_u), P(y_u), *(P(t_) for t_ in operands),
                  *(P(t_) for t_ in z), B, Lx, Ly, d, D, 0.05, ops.q_code(2.0), words, code, stream)
        torch.cuda.synchronize()
        return z + [x_l, y_l, y_u], x_u

    full, x_u = call(True)
    bare, _ = call(False)
    assert not torch.isnan(x_u).any()
    for name, a, b in zip(("z_lb", "z_ub", "z_lw", "z_uw", "x_l", "y_l", "y_u"), full, bare):
        assert not torch.isnan(b).any(), name
        assert torch.equal(a, b), f"{name} differs without x_u"


def test_reference_layout_dot_product_at_configuration_3_size_equals_the_natural_layout():
    """Full-size configuration 3 through the transposed entry: every element within the parity bar of the MFMA
    path of the natural layout (same inputs re-laid out; two fp32 summation orders of 256 terms)."""
    from faith_amd import c_bound, ops
    from faith_amd.workloads import make_config
    c = make_config(3)
    x, y = dev(as_bounds(c["x"])), dev(as_bounds(c["y"]))
    B, L, D, d = x[0].shape
    nat = ops.dot_product_qk(x, y, c["p"], c["eps"], 1)
    T = lambda t_: t_.transpose(2, 3).contiguous()
    z = lambda *s_: torch.empty(*s_, device="cuda")
    scratch = [z(B, L, d) for _ in range(4)]
    zlb, zub, zlw, zuw = z(B, L, L), z(B, L, L), z(B, L, L, D), z(B, L, L, D)
    c_bound.p, c_bound.words = c["p"], 1
    try:
        c_bound.c_dot_product_verification_QK(*scratch, x[1], x[3], y[1], y[3], T(x[0]), T(x[2]), T(y[0]), T(y[2]),
                                              zlb, zub, zlw, zuw, B, L, d, D, c["eps"])
    finally:
        c_bound.p = 2.0
    # the same constant-term kernel, fed by intervals from two concretize kernels (another reduction order: last
    # bits of l, u differ) whose differences 64 O(1) terms per element carry into the sums
    torch.testing.assert_close(zlb, nat[1], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(zub, nat[3], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(zlw.transpose(2, 3), nat[0], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(zuw.transpose(2, 3), nat[2], rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------ heads addressed in place
def side_by_side(x, heads):
    """[batch*heads, L, D, w] / [batch*heads, L, w] -> [batch, L, D, heads*w] / [batch, L, heads*w], the
    object a dense layer produces (inverse of transpose_for_scores, VerifierForward.py:208-229)."""
    def w(t):
        bh, L, D, width = t.shape
        return t.reshape(bh // heads, heads, L, D, width).permute(0, 2, 3, 1, 4).reshape(bh // heads, L, D, -1).contiguous()

    def b(t):
        bh, L, width = t.shape
        return t.reshape(bh // heads, heads, L, width).permute(0, 2, 1, 3).reshape(bh // heads, L, -1).contiguous()
    return O.LinearBounds(w(x.lw), b(x.lb), w(x.uw), b(x.ub))


@pytest.mark.parametrize("shape", [
    # batch, heads, Lx, Ly, D, head size
    (1, 4, 128, 128, 16, 64),      # straight-line MFMA kernel
    (2, 2, 128, 64, 8, 32),        # the same with two batch elements
    (1, 2, 130, 70, 20, 36),       # ragged tiles, half-empty last K-step
    (1, 4, 32, 32, 64, 16),        # short sequences: one 32 x 32 block per wavefront
    (3, 2, 20, 40, 24, 24),        # short, ragged, three batch elements
    (2, 3, 6, 4, 5, 10),           # head size % 4 != 0: any-shape kernel
    (2, 2, 3, 5, 1, 8),            # dim_in == 1: interval shortcut
])
@pytest.mark.parametrize("p", [2.0, INF])
def test_attention_scores_reads_the_heads_in_place(shape, p):
    from faith_amd import ops
    batch, heads, Lx, Ly, D, d = shape
    g = torch.Generator().manual_seed(41)
    x = rand_bounds(g, batch * heads, Lx, D, d, ordered=False, sw=0.3, sb=1.0)
    y = rand_bounds(g, batch * heads, Ly, D, d, ordered=False, sw=0.3, sb=1.0)
    words = 2 if D % 2 == 0 else 1
    print(f"[case] attention_scores batch={batch} heads={heads} Lx={Lx} Ly={Ly} D={D} size={d} p={p} words={words}", flush=True)
    got = ops.attention_scores(dev(side_by_side(x, heads)), dev(side_by_side(y, heads)), heads, p, 0.1, words)
    torch.cuda.synchronize()
    exp = O.dot_product(x, y, p, 0.1, words)
    if D == 1:
        for a, e in zip(got, exp.tensors()):
            assert close(a, e)
        return
    ref, mag = dot64(x, y, p, 0.1, words)
    for name, a, e in zip(("lw", "lb", "uw", "ub"), got, exp.tensors()):
        assert a.shape == e.shape
        compare_contraction(name, a, e, ref[name], mag[name], UNIT_SCALE_ALL)


@pytest.mark.parametrize("shape", [
    # batch, heads, queries, keys, D, head size
    (1, 4, 128, 128, 16, 64), (1, 2, 128, 64, 8, 128),    # straight-line MFMA kernel
    (2, 2, 128, 64, 8, 64),        # two batch elements
    (1, 2, 130, 72, 12, 20),       # ragged
    (1, 4, 32, 32, 64, 16),        # short sequences
    (3, 2, 24, 16, 16, 24),        # short, three batch elements
    (2, 3, 6, 6, 4, 10),           # six keys: ragged reduction
    (1, 4, 30, 30, 64, 64),        # a sentence of 30 tokens
    (2, 2, 23, 23, 16, 32),
    (2, 2, 4, 4, 1, 8),            # interval shortcut
])
@pytest.mark.parametrize("p", [2.0, INF])
def test_attention_context_reads_and_writes_the_heads_in_place(shape, p):
    from faith_amd import ops
    batch, heads, Lq, Lk, D, dv = shape
    g = torch.Generator().manual_seed(42)
    probs = rand_bounds(g, batch * heads, Lq, D, Lk, ordered=False, sw=0.2, sb=0.5)
    value = rand_bounds(g, batch * heads, Lk, D, dv, ordered=False, sw=0.3, sb=1.0)
    print(f"[case] attention_context batch={batch} heads={heads} Lq={Lq} Lk={Lk} D={D} size={dv} p={p}", flush=True)
    got = ops.attention_context(dev(probs), dev(side_by_side(value, heads)), p, 0.1, 1)
    torch.cuda.synchronize()
    exp = O.context(probs, value, p, 0.1, 1)
    exp_sbs = side_by_side(exp, heads)
    if D == 1:
        for a, e in zip(got, exp_sbs.tensors()):
            assert close(a, e)
        return
    ref, mag = dot64(probs, O.transpose_bounds(value), p, 0.1, 1)
    wrap = lambda r: side_by_side(O.LinearBounds(r["lw"], r["lb"], r["uw"], r["ub"]), heads)
    ref_s, mag_s = wrap(ref), wrap(mag)
    for name, a, e, r, m in zip(("lw", "lb", "uw", "ub"), got, exp_sbs.tensors(), ref_s.tensors(), mag_s.tensors()):
        assert a.shape == e.shape
        compare_contraction(name, a, e, r, m, UNIT_SCALE_ALL)


def test_in_place_heads_equal_stacked_heads_bit_for_bit_at_configuration_3_size():
    """Same kernels, same summation order, different addressing: the in-place entry points must
    reproduce the stacked ones exactly (4 heads, L = 128, D_in = 256, d = 64; scores and context)."""
    from faith_amd import ops
    heads, L, D, d = 4, 128, 256, 64
    g = torch.Generator(device="cuda").manual_seed(43)
    mk = lambda *s: torch.randn(*s, device="cuda", generator=g)
    def obj(scale):
        lw, lb = mk(heads, L, D, d) * scale, mk(heads, L, d)
        return (lw, lb, lw + 0.01 * mk(heads, L, D, d).abs(), lb + 0.1 * mk(heads, L, d).abs())
    q, k, v = obj(0.05), obj(0.05), obj(0.05)
    sbs_w = lambda t: t.permute(1, 2, 0, 3).reshape(1, L, D, heads * d).contiguous()
    sbs_b = lambda t: t.permute(1, 0, 2).reshape(1, L, heads * d).contiguous()
    sbs = lambda o: (sbs_w(o[0]), sbs_b(o[1]), sbs_w(o[2]), sbs_b(o[3]))
    print("[case] in-place heads against stacked heads, configuration 3 size", flush=True)
    stacked = ops.dot_product_qk(q, k, INF, 0.01, 1)
    in_place = ops.attention_scores(sbs(q), sbs(k), heads, INF, 0.01, 1)
    for a, b in zip(stacked, in_place):
        assert torch.equal(a, b)
    ctx = ops.dot_product_v(stacked, v, INF, 0.01, 1)
    ctx_in_place = ops.attention_context(stacked, sbs(v), INF, 0.01, 1)
    for a, b in zip(ctx, ctx_in_place):
        want = sbs_w(a) if a.dim() == 4 else sbs_b(a)
        assert torch.equal(want, b)


@pytest.mark.parametrize("case", [
    # path, (batch, heads) layout, pairs or (batch, heads), Lx, Ly or keys, D, head size / reduction
    ("scores", "stacked", 4, 128, 128, 64, 64), ("scores", "stacked", 2, 256, 64, 24, 32), ("scores", "stacked", 1, 128, 192, 40, 128),
    ("scores", "in place", (2, 3), 128, 128, 16, 64), ("scores", "in place", (1, 4), 256, 64, 8, 32),
    ("context", "stacked", 4, 128, 128, 64, 64), ("context", "stacked", 3, 256, 32, 24, 64), ("context", "stacked", 2, 128, 64, 16, 128),
    ("context", "in place", (2, 2), 128, 128, 16, 64), ("context", "in place", (1, 3), 128, 32, 8, 64),
])
def test_straight_line_tiles_equal_the_tiles_with_run_time_extents_bit_for_bit(case):
    """Reductions of 32, 64 and 128 take a kernel whose reduction length is a template argument (operands of x
    from global memory straight to LDS, no cleared accumulators, one descriptor per array); same tiles and same
    order of summation as the kernel with run-time extents, which the tuning knob still selects: same bits."""
    from faith_amd import _lib, ops
    path, layout, pairs, Lx, Ly, D, red = case
    batch, heads = pairs if layout == "in place" else (pairs, 1)
    g = torch.Generator().manual_seed(61)
    print(f"[case] straight-line dot tiles {case}", flush=True)
    if path == "scores":
        x = rand_bounds(g, batch * heads, Lx, D, red, ordered=False, sw=0.3, sb=1.0)
        y = rand_bounds(g, batch * heads, Ly, D, red, ordered=False, sw=0.3, sb=1.0)
        if layout == "in place":
            run = lambda: ops.attention_scores(dev(side_by_side(x, heads)), dev(side_by_side(y, heads)), heads, 2.0, 0.1, 1)
        else:
            run = lambda: ops.dot_product_qk(dev(x), dev(y), 2.0, 0.1, 1)
    else:       # probabilities [.., Lx, D, keys] times values [.., keys, D, width]: the reduction runs over the keys
        width = Ly
        probs = rand_bounds(g, batch * heads, Lx, D, red, ordered=False, sw=0.2, sb=0.5)
        value = rand_bounds(g, batch * heads, red, D, width, ordered=False, sw=0.3, sb=1.0)
        if layout == "in place":
            run = lambda: ops.attention_context(dev(probs), dev(side_by_side(value, heads)), 2.0, 0.1, 1)
        else:
            run = lambda: ops.dot_product_v(dev(probs), dev(value), 2.0, 0.1, 1)
    got = run()
    torch.cuda.synchronize()
    _lib.call("faith_tune_set", 2, 1)
    try:
        want = run()
        torch.cuda.synchronize()
    finally:
        _lib.call("faith_tune_set", 2, 0)
    for name, a, b in zip(("lw", "lb", "uw", "ub"), got, want):
        assert torch.equal(a, b), f"{name}: {int((a != b).sum())} of {a.numel()} values differ"
