"""HIP concretize / ReLU / tanh against the CPU oracle, through the C ABI."""
import pytest
import torch

from oracle import bounds_oracle as O
from tests.helpers import rand_bounds, as_bounds, close, RTOL, ATOL
from tests.parity import compare_activation

pytestmark = pytest.mark.gpu
INF = float("inf")
PS = [1.0, 2.0, INF, 3.0, 1.5]     # 3.0 and 1.5: dual exponents 1.5 and 3, the general-norm kernels


def dev(*ts):
    return [t.cuda().contiguous() for t in ts]


def run_act(kind, x, p, eps, words, layout="natural"):
    from faith_amd import ops
    lw, lb, uw, ub = dev(*x.tensors())
    fn = getattr(ops, kind)
    if layout == "natural":
        out = fn(lw, lb, uw, ub, p, eps, words, return_interval=True)
        return out[:4], out[4], out[5]
    lwt, uwt = lw.transpose(2, 3).contiguous(), uw.transpose(2, 3).contiguous()
    olw, olb, ouw, oub, l, u = fn(lwt, lb, uwt, ub, p, eps, words, layout=ops.LAYOUT_TRANSPOSED,
                                  return_interval=True)
    return (olw.transpose(2, 3), olb, ouw.transpose(2, 3), oub), l, u


def check(kind, x, p, eps, words, layout="natural"):
    print(f"[case] {kind} shape={tuple(x.lw.shape)} p={p} eps={eps} words={words} layout={layout}", flush=True)
    got, l, u = run_act(kind, x, p, eps, words, layout)
    torch.cuda.synchronize()
    exp = getattr(O, kind)(x, p, eps, words)
    l_ref, u_ref = O.concretize(x, p, eps, words)
    rep = compare_activation(kind, x, got, exp.tensors(), l.cpu(), u.cpu(), l_ref, u_ref)
    print("   ", rep, flush=True)
    return rep


@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("words", [1, 2])
@pytest.mark.parametrize("layout", ["natural", "transposed"])
def test_concretize(p, words, layout):
    from faith_amd import ops
    g = torch.Generator().manual_seed(5)
    for (B, L, D, H) in [(1, 3, 64, 64), (2, 5, 96, 40), (1, 2, 600, 132), (1, 1, 6, 7), (1, 3, 256, 41), (1, 2, 512, 21)]:
        x = rand_bounds(g, B, L, D, H, ordered=False)
        lw, lb, uw, ub = dev(*x.tensors())
        if layout == "natural":
            l, u = ops.concretize(lw, lb, uw, ub, p, 0.3, words)
        else:
            l, u = ops.concretize(lw.transpose(2, 3).contiguous(), lb, uw.transpose(2, 3).contiguous(), ub,
                                  p, 0.3, words, layout=ops.LAYOUT_TRANSPOSED)
        el, eu = O.concretize(x, p, 0.3, words)
        assert close(l, el) and close(u, eu), (B, L, D, H)


@pytest.mark.parametrize("kind", ["relu", "tanh"])
@pytest.mark.parametrize("p", PS)
@pytest.mark.parametrize("layout", ["natural", "transposed"])
def test_activation_small_shapes(kind, p, layout):
    g = torch.Generator().manual_seed(6)
    # register-resident, chunked (D_in > 512), ragged H (scalar path), tiny
    for (L, D, H, words) in [(4, 64, 64, 1), (3, 128, 192, 2), (2, 256, 64, 2), (2, 512, 64, 1),
                             (1, 1100, 72, 1), (2, 48, 37, 3), (1, 2, 5, 1), (3, 256, 37, 4), (1, 512, 9, 2),
                             (2, 768, 64, 2), (1, 1024, 36, 1), (1, 516, 40, 3)]:   # 512 < D_in <= 1024: sixteen-wavefront tiles
        x = rand_bounds(g, 1, L, D, H, ordered=True, sw=0.2, sb=1.0, gap_w=0.02, gap_b=0.5)
        check(kind, x, p, 0.05, words, layout)


@pytest.mark.parametrize("kind", ["relu", "tanh", "exp"])
@pytest.mark.parametrize("knob", [0, 7, 12])
def test_register_resident_tiles_take_whole_steps_of_rows_only(kind, knob):
    """D_in between 128 and 256 that is a multiple of 32 but not of 64 (160, 224), or of 64 but not of 128 (192): a
    step of the eight-wavefront tile is 64 rows and one of the sixteen-wavefront tile (knobs 7 and 12, and objects
    beyond the memory-side cache) 128, and a tile must not reach into the rows of the next position.  Regression:
    160 rows on the eight-wavefront tile read and overwrote 32 rows of the neighbouring position."""
    from faith_amd import _lib
    g = torch.Generator().manual_seed(17)
    _lib.call("faith_tune_set", 0, knob)
    try:
        for (L, D, H, words) in [(3, 160, 64, 1), (5, 224, 96, 2), (2, 192, 64, 1), (4, 160, 32, 5), (3, 256, 64, 2)]:
            x = rand_bounds(g, 1, L, D, H, ordered=True, sw=0.2, sb=1.0, gap_w=0.02, gap_b=0.5)
            check(kind, x, 2.0, 0.05, words)
    finally:
        _lib.call("faith_tune_set", 0, 0)


@pytest.mark.parametrize("kind", ["relu", "tanh", "exp"])
@pytest.mark.parametrize("p", [2.0, INF, 1.0, 3.0])
def test_transposed_rows_of_any_length_stay_in_registers(kind, p):
    """The transposed layout (what the reference's adapters hand over) keeps rows of up to 1024 coefficients in
    registers: several neurons side by side in a wavefront for D_in = 32 / 64 / 128, one to four loads per lane
    beyond, lanes past the end of a row idle (D_in = 192, 300, 516).  Neuron counts that do not fill the last
    wavefront or workgroup; against the oracle."""
    g = torch.Generator().manual_seed(16)
    for (L, D, H, words) in [(5, 32, 50, 1), (3, 64, 70, 2), (7, 128, 33, 1), (2, 192, 40, 2), (2, 300, 24, 1),
                             (2, 384, 40, 2), (3, 768, 23, 1), (1, 1024, 20, 2), (1, 516, 19, 3), (1, 16, 9, 1)]:
        x = rand_bounds(g, 1, L, D, H, ordered=True, sw=0.2, sb=1.0, gap_w=0.02, gap_b=0.5)
        check(kind, x, p, 0.05, words, "transposed")


@pytest.mark.parametrize("kind", ["concretize", "relu", "tanh"])
@pytest.mark.parametrize("words", [8, 16])
def test_many_perturbed_words_need_more_than_64_kb_of_lds(kind, words):
    """The partial norms of every word and wavefront sit in LDS: with 8 or 16 words the sixteen-wavefront
    tiles ask for 67 ... 133 KB, beyond the 64 KB a launch gets without asking."""
    from faith_amd import ops
    g = torch.Generator().manual_seed(9)
    for (L, D, H) in [(2, 64, 64), (2, 1024, 64), (1, 256, 96), (1, 2048, 40)]:
        x = rand_bounds(g, 1, L, D, H, ordered=True, sw=0.2, sb=1.0, gap_w=0.02, gap_b=0.5)
        if kind == "concretize":
            l, u = ops.concretize(*dev(*x.tensors()), 2.0, 0.05, words)
            el, eu = O.concretize(x, 2.0, 0.05, words)
            assert close(l, el) and close(u, eu), (L, D, H, words)
        else:
            check(kind, x, 2.0, 0.05, words)


@pytest.mark.parametrize("kind", ["relu", "tanh"])
@pytest.mark.parametrize("p", PS)
def test_thread_shape_for_hbm_streams_gives_the_same_values(kind, p):
    """Objects too large for the memory-side cache take sixteen wavefronts of two rows instead of four of
    eight (tuning knob 7 forces that shape on a small object): same tile, same reduction tree per column
    group, checked against the oracle and against the default shape."""
    from faith_amd import _lib, ops
    g = torch.Generator().manual_seed(10)
    x = rand_bounds(g, 1, 3, 256, 96, ordered=True, sw=0.2, sb=1.0, gap_w=0.02, gap_b=0.5)
    ref = getattr(ops, kind)(*dev(*x.tensors()), p, 0.05, 2)
    _lib.call("faith_tune_set", 0, 7)
    try:
        check(kind, x, p, 0.05, 2)
        got = getattr(ops, kind)(*dev(*x.tensors()), p, 0.05, 2)
    finally:
        _lib.call("faith_tune_set", 0, 0)
    for a, b in zip(got, ref):
        assert close(a, b.cpu())


def test_a_knob_set_by_one_thread_selects_that_threads_kernels_only():
    """The tuning knobs are kept per calling thread.  Knob 8 (four wavefronts a tile) groups a column's partial norms
    differently from the default shape, so its results differ in the last bits of some values: a worker thread that
    sets it gets those bits, the main thread keeps getting the default's."""
    import threading
    from faith_amd import _lib, ops
    g = torch.Generator(device="cuda").manual_seed(21)
    shape = (1, 40, 256, 1024)
    lw = torch.empty(shape, device="cuda").normal_(0, 0.05, generator=g)
    uw = torch.empty(shape, device="cuda").normal_(0, 0.005, generator=g).abs_().add_(lw)
    lb = torch.empty((1, 40, 1024), device="cuda").normal_(0, 1, generator=g)
    ub = torch.empty((1, 40, 1024), device="cuda").normal_(0, 0.5, generator=g).abs_().add_(lb)
    run = lambda: [t.clone() for t in ops.relu(lw, lb, uw, ub, 2.0, 0.01, 2, return_interval=True)]
    ref = run()
    _lib.call("faith_tune_set", 0, 8)
    try:
        forced = run()
    finally:
        _lib.call("faith_tune_set", 0, 0)
    torch.cuda.synchronize()
    assert not all(torch.equal(a, b) for a, b in zip(ref, forced)), "the two shapes gave the same bits: nothing to observe"
    seen = {}

    def worker():
        _lib.call("faith_tune_set", 0, 8)          # never reset: the value ends with the thread
        seen["forced"] = run()
        torch.cuda.synchronize()

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    after = run()
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(seen["forced"], forced))
    assert all(torch.equal(a, b) for a, b in zip(after, ref))


@pytest.mark.parametrize("kind,p", [("relu", 2.0), ("relu", INF), ("exp", 1.0), ("sqr", 2.0), ("tanh", 2.0)])
@pytest.mark.parametrize("rows", [40, 43])
def test_persistent_two_tile_kernel_gives_the_one_tile_kernels_bits(kind, p, rows):
    """The persistent kernel (workgroups that hold the next tile while they finish the current one: tuning knob 15)
    against the one-tile kernel of four wavefronts (knob 8): the arithmetic per tile is the same, so the results are,
    bit for bit -- also when the tiles do not divide evenly among the workgroups (43 rows).  The default shape (eight
    wavefronts, whole rows dealt to the XCDs when the row count allows: 40 rows do, 43 do not) sums a column's partial
    norms in another grouping: it is held to the one-tile kernel at the parity bar, a neuron whose interval end moved by
    an ulp across a branch switch excepted (at most one in ten thousand), and three of its rows to the oracle."""
    from faith_amd import _lib, ops
    g = torch.Generator(device="cuda").manual_seed(12)
    shape = (1, rows, 256, 1024)
    lw = torch.empty(shape, device="cuda").normal_(0, 0.05, generator=g)
    uw = torch.empty(shape, device="cuda").normal_(0, 0.005, generator=g).abs_().add_(lw)
    lb = torch.empty((1, rows, 1024), device="cuda").normal_(0, 1, generator=g)
    ub = torch.empty((1, rows, 1024), device="cuda").normal_(0, 0.5, generator=g).abs_().add_(lb)
    if kind in ("sqr",):
        lb, ub = lb.abs() + 1.0, ub.abs() + 2.5
        lb, ub = torch.minimum(lb, ub), torch.maximum(lb, ub)
    print(f"[case] persistent kernel {kind} p={p} rows={rows}", flush=True)
    fn = getattr(ops, kind)
    by_default = fn(lw, lb, uw, ub, p, 0.01, 2, return_interval=True)
    results = {}
    for knob in (8, 15):
        _lib.call("faith_tune_set", 0, knob)
        try:
            results[knob] = fn(lw, lb, uw, ub, p, 0.01, 2, return_interval=True)
        finally:
            _lib.call("faith_tune_set", 0, 0)
    torch.cuda.synchronize()
    for name, d, one, two in zip(("lw", "lb", "uw", "ub", "l", "u"), by_default, results[8], results[15]):
        assert torch.equal(one, two), f"{kind} {name}: the persistent kernel differs from the one-tile kernel"
        off = ((d.double() - one.double()).abs() > 1e-6 + 1e-5 * one.double().abs()).double().mean().item()
        assert off <= 1e-4, f"{kind} {name}: the default shape is off the bar against the one-tile kernel on {off:.2e} of the values"
    for r in (0, rows // 2, rows - 1):
        x = O.LinearBounds(*(t[:, r:r + 1].cpu() for t in (lw, lb, uw, ub)))
        exp = getattr(O, kind)(x, p, 0.01, 2)
        l_ref, u_ref = O.concretize(x, p, 0.01, 2)
        got = tuple(t[:, r:r + 1].cpu() for t in by_default)
        rep = compare_activation(kind, x, got[:4], exp.tensors(), got[4], got[5], l_ref, u_ref)
        print("   ", rep, flush=True)


@pytest.mark.parametrize("kind", ["relu", "tanh"])
def test_activation_reference_test_distribution(kind):
    """Inputs drawn as the reference's own op test draws them
    (kernel_test/transformer_forward_test_bound.py:746-754, p=2, eps=0.5):
    lb ~ U(0,1), ub = lb + U(0,1), lw and uw independent U(-.5,.5)."""
    g = torch.Generator().manual_seed(0)
    for (L, D, H) in [(2, 64, 64), (8, 128, 64), (4, 64, 256)]:
        lb = torch.rand(1, L, H, generator=g)
        ub = lb + torch.rand(1, L, H, generator=g)
        lw = torch.rand(1, L, D, H, generator=g) - 0.5
        uw = torch.rand(1, L, D, H, generator=g) - 0.5
        check(kind, O.LinearBounds(lw, lb, uw, ub), 2.0, 0.5, 1)


def test_activation_branch_edges():
    """Neurons exactly on the switches: l == 0, u == 0, |u| == |l|, and zero-width intervals."""
    from faith_amd import ops
    H, D = 64, 8
    lw = torch.zeros(1, 1, D, H); uw = torch.zeros(1, 1, D, H)
    lw[0, 0, 0, :] = 0.25; uw[0, 0, 0, :] = 0.5
    lb = torch.linspace(-1, 1, H).view(1, 1, H).clone()
    ub = lb.clone() + 0.5
    lb[0, 0, 0] = 0.0; ub[0, 0, 0] = 1.0        # l == 0 exactly (eps = 0 below)
    lb[0, 0, 1] = -1.0; ub[0, 0, 1] = 0.0       # u == 0 exactly
    lb[0, 0, 2] = -0.5; ub[0, 0, 2] = 0.5       # |u| == |l|
    lb[0, 0, 3] = 0.0; ub[0, 0, 3] = 0.0        # degenerate at 0
    x = O.LinearBounds(lw, lb, uw, ub)
    for kind in ("relu", "tanh"):
        got, l, u = run_act(kind, x, 2.0, 0.0, 1)
        exp = getattr(O, kind)(x, 2.0, 0.0, 1)
        for a, b in zip(got, exp.tensors()):
            assert close(a, b), kind


@pytest.mark.parametrize("kind", ["relu", "tanh"])
@pytest.mark.parametrize("p", PS)
def test_activation_config1_reduced(kind, p):
    """Benchmark configuration 1 at a quarter of its length (same D_in, H, words)."""
    from faith_amd.workloads import make_config
    c = make_config(1, scale=0.25)
    rep = check(kind, as_bounds(c["x"]), p, c["eps"], c["words"])
    assert rep["neurons"] == 32 * 512


@pytest.mark.parametrize("kind", ["relu", "tanh"])
def test_activation_config1_full_properties(kind):
    """Full-size configuration 1: size-independent properties instead of the oracle.
    (i) the concrete interval of the output bounds the activation of the input interval
    end points; (ii) dead / active ReLU neurons are zero / identity; (iii) l <= u."""
    from faith_amd import ops
    from faith_amd.workloads import make_config
    c = make_config(1)
    lw, lb, uw, ub = dev(*(c["x"][k] for k in ("lw", "lb", "uw", "ub")))
    for p in PS:
        olw, olb, ouw, oub, l, u = getattr(ops, kind)(lw, lb, uw, ub, p, c["eps"], c["words"], return_interval=True)
        assert bool((l <= u).all())
        ol, ou = ops.concretize(olw, olb, ouw, oub, p, c["eps"], c["words"])
        f = torch.relu if kind == "relu" else torch.tanh
        assert bool((ol <= f(l) + 1e-4).all()) and bool((ou >= f(u) - 1e-4).all())
        if kind == "relu":
            dead, act = u < 0, l > 0
            assert torch.count_nonzero(olw.transpose(2, 3)[dead]) == 0
            assert torch.count_nonzero(ouw.transpose(2, 3)[dead]) == 0
            assert torch.equal(olw.transpose(2, 3)[act], lw.transpose(2, 3)[act])
            assert torch.equal(oub[act], ub[act])
            frac_both = 1.0 - float(dead.float().mean()) - float(act.float().mean())
            assert 0.05 < frac_both < 0.9


def test_c_bound_shim_matches_reference_calling_convention():
    """faith_amd.c_bound: reference names, transposed operands, caller-allocated outputs
    (HandTunedKernels/kernel.cpp:69-131; adapter in Bounds.py:1201-1231)."""
    from faith_amd import c_bound
    g = torch.Generator().manual_seed(7)
    L, D, H = 4, 64, 128
    x = rand_bounds(g, 1, L, D, H, sw=0.2, gap_w=0.02, gap_b=0.5)
    lw, lb, uw, ub = dev(*x.tensors())
    for name, kind in (("c_relu_verification", "relu"), ("c_tanh_verification", "tanh")):
        _lw = torch.zeros(1, L, H, D, device="cuda"); _uw = torch.zeros_like(_lw)
        _lb = torch.zeros(1, L, H, device="cuda"); _ub = torch.zeros_like(_lb)
        getattr(c_bound, name)(lb, ub, lw.transpose(2, 3).contiguous(), uw.transpose(2, 3).contiguous(),
                               _lb, _ub, _lw, _uw, L, D, H, 0.05)
        exp = getattr(O, kind)(x, 2.0, 0.05, 1)
        assert close(_lw.transpose(2, 3), exp.lw) and close(_uw.transpose(2, 3), exp.uw)
        assert close(_lb, exp.lb) and close(_ub, exp.ub)


def test_bad_arguments_are_rejected_not_launched():
    from faith_amd import ops, _lib
    lw = torch.zeros(1, 2, 8, 4, device="cuda"); lb = torch.zeros(1, 2, 4, device="cuda")
    with pytest.raises(_lib.FaithError) as e:
        ops.relu(lw, lb, lw, lb, 2.0, 0.1, words=3)          # 3 does not divide 8
    assert e.value.code == -2
    with pytest.raises(ValueError):
        ops.relu(lw, lb, lw, lb, 0.5, 0.1)                   # not a norm
    with pytest.raises(ValueError):
        ops.relu(lw.cpu(), lb, lw, lb, 2.0, 0.1)             # CPU tensor: no fallback
    with pytest.raises(TypeError):
        ops.relu(lw.double(), lb, lw, lb, 2.0, 0.1)


@pytest.mark.parametrize("p", [2.0, INF])
def test_concretize_of_very_long_rows(p):
    """Rows of 64 KB and more (image-shaped bounds flattened to [1, D_in, C*H*W]) take four-wavefront
    workgroups; D_in beyond one pass of rows, a ragged last tile, two perturbed words."""
    from faith_amd import ops
    g = torch.Generator().manual_seed(7)
    for (D, H, words) in [(12, 16384, 1), (300, 16420, 2), (64, 32768 + 8, 1)]:
        x = rand_bounds(g, 1, 1, D, H, ordered=False)
        lw, lb, uw, ub = dev(*x.tensors())
        l, u = ops.concretize(lw, lb, uw, ub, p, 0.3, words)
        el, eu = O.concretize(x, p, 0.3, words)
        assert close(l, el) and close(u, eu), (D, H, words)
