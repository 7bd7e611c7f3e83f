"""Bound objects of more than 2^31 elements (more than 8 GiB per tensor) through every hot operator.

The CPU oracle cannot run at this size, so the check is the size-independent property the domain
offers: every operator here is independent across positions (rows of L, heads, perturbation slices
of a convolution), so the rows of the full-size result must equal the result of the same operator
on those rows alone.  The rows checked straddle the offsets at which 32-bit arithmetic would wrap:
element 2^30 (byte offset 2^32), element 2^31, and the end of the tensor."""
import sys

import pytest
import torch

from faith_amd import ops

pytestmark = pytest.mark.gpu
INF = float("inf")
NEED_BYTES = 80 << 30


@pytest.fixture(autouse=True)
def _room():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    free, _ = torch.cuda.mem_get_info()
    if free < NEED_BYTES:
        pytest.skip(f"needs {NEED_BYTES >> 30} GiB of free device memory, {free >> 30} GiB available")
    yield
    torch.cuda.empty_cache()


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def big_object(shape_w, shape_b, seed, wstd=0.05, gap_w=0.005, gap_b=0.5):
    g = torch.Generator(device="cuda").manual_seed(seed)
    lw = torch.empty(shape_w, device="cuda").normal_(0, wstd, generator=g)
    uw = torch.empty(shape_w, device="cuda").normal_(0, gap_w, generator=g).abs_().add_(lw)
    lb = torch.empty(shape_b, device="cuda").normal_(0, 1, generator=g)
    ub = torch.empty(shape_b, device="cuda").normal_(0, gap_b, generator=g).abs_().add_(lb)
    return lw, lb, uw, ub


def rows_to_check(n_rows, row_elems):
    picks = {0, n_rows - 2, n_rows - 1}
    for boundary in (1 << 30, 1 << 31):
        r = boundary // row_elems
        picks.update({r - 1, r, r + 1})
    return sorted(r for r in picks if 0 <= r < n_rows)


def same(full, part, what, exact, atol=1e-6):
    if exact:
        assert torch.equal(full, part), f"{what}: differs from the run on these rows alone"
    else:
        torch.testing.assert_close(full, part, rtol=1e-5, atol=atol, msg=lambda m: f"{what}: {m}")


def check_rows(name, full, run_slice, picks, exact=True):
    """full: tuple of result tensors whose axis 1 is the position; run_slice(r) -> the same tuple for row r."""
    for r in picks:
        part = run_slice(r)
        for i, (f, q) in enumerate(zip(full, part)):
            same(f[:, r:r + 1], q, f"{name} row {r} output {i}", exact)


def sl(x, r):
    return tuple(t[:, r:r + 1] for t in x)


@pytest.mark.parametrize("op,p,layout,shape", [
    ("relu", 2.0, "natural", (2100, 1024, 1024)),       # D_in = 1024: rows in the registers of sixteen wavefronts
    ("tanh", INF, "natural", (8200, 256, 1024)),        # register-resident kernel, one tile per workgroup
    ("relu", 2.0, "natural", (8200, 256, 1024)),        # the same for another mode
    ("relu", 2.0, "persistent", (8200, 256, 1024)),     # register-resident kernel, persistent workgroups (tuning knob 15)
    ("relu", 1.0, "natural", (300, 2048, 3600)),        # chunked walk (D_in > 1024), two reads
    ("tanh", 2.0, "transposed", (2100, 4096, 256)),     # transposed, resident (D_in = 256)
    ("relu", INF, "transposed", (2100, 1000, 1040)),    # transposed, general kernel
])
def test_relaxation_rows(op, p, layout, shape):
    from faith_amd import _lib
    L, A, B = shape
    say(f"large {op} p={p} {layout} [1, {L}, {A}, {B}]")
    persistent = layout == "persistent"
    if persistent:
        layout = "natural"
    x = big_object((1, L, A, B), (1, L, A if layout == "transposed" else B), 11)
    lay = ops.LAYOUT_TRANSPOSED if layout == "transposed" else ops.LAYOUT_NATURAL
    fn = getattr(ops, op)
    if persistent:
        _lib.call("faith_tune_set", 0, 15)
    try:
        full = fn(*x, p, 0.01, 2, lay, True)
    finally:
        _lib.call("faith_tune_set", 0, 0)
    picks = rows_to_check(L, A * B)
    # an object of this size streams from HBM and takes the register-resident kernel's sixteen-wavefront thread
    # shape, where a single row would take the four-wavefront one (another reduction tree), so the slices are held
    # to the shape of the whole (tuning knob 7) and the comparison stays bit for bit; the persistent workgroups
    # have the arithmetic of the four-wavefront shape (knob 8 for the slices)
    resident = layout == "natural" and A <= 256
    if resident:
        _lib.call("faith_tune_set", 0, 8 if persistent else 7)
    try:
        check_rows(f"{op} {layout}", full, lambda r: fn(*sl(x, r), p, 0.01, 2, lay, True), picks)
    finally:
        _lib.call("faith_tune_set", 0, 0)
    conc = ops.concretize(*x, p, 0.01, 2, lay)
    # likewise the concretization: an object of 64 MB and more is walked by four-wavefront workgroups, a single
    # row by sixteen-wavefront ones; knob 11 holds the slices to the shape of the whole
    if layout == "natural":
        _lib.call("faith_tune_set", 0, 11)
    try:
        check_rows(f"concretize {layout}", conc, lambda r: ops.concretize(*sl(x, r), p, 0.01, 2, lay), picks)
    finally:
        _lib.call("faith_tune_set", 0, 0)
    same(conc[0], full[4], "interval of the relaxation against concretize (l)", False)
    same(conc[1], full[5], "interval of the relaxation against concretize (u)", False)


def test_linear_rows():
    L, D, K, N = 2100, 1024, 1024, 96
    say(f"large linear [1, {L}, {D}, {K}] x [{N}, {K}]")
    x = big_object((1, L, D, K), (1, L, K), 12)
    g = torch.Generator(device="cuda").manual_seed(13)
    W = torch.empty((N, K), device="cuda").normal_(0, K ** -0.5, generator=g)
    bias = torch.empty((N,), device="cuda").normal_(0, 0.01, generator=g)
    full = ops.linear(*x, W, bias)
    check_rows("linear", full, lambda r: ops.linear(*sl(x, r), W, bias), rows_to_check(L, D * K), exact=False)


def test_linear_wide_output_rows():
    # the outputs, not the inputs, pass 2^31 elements
    L, D, K, N = 2100, 1024, 64, 1024
    say(f"large linear [1, {L}, {D}, {K}] x [{N}, {K}]")
    x = big_object((1, L, D, K), (1, L, K), 14)
    g = torch.Generator(device="cuda").manual_seed(15)
    W = torch.empty((N, K), device="cuda").normal_(0, K ** -0.5, generator=g)
    full = ops.linear(*x, W, None)
    check_rows("linear wide", full, lambda r: ops.linear(*sl(x, r), W, None), rows_to_check(L, D * N), exact=False)


def test_whole_object_rows():
    L, D, H = 8200, 256, 1024
    say(f"large affine / layer norm / row sum / product [1, {L}, {D}, {H}]")
    x = big_object((1, L, D, H), (1, L, H), 16)
    y = big_object((1, L, D, H), (1, L, H), 17)
    g = torch.Generator(device="cuda").manual_seed(18)
    scale = torch.empty((H,), device="cuda").normal_(0, 1, generator=g)
    shift = torch.empty((H,), device="cuda").normal_(0, 1, generator=g)
    picks = rows_to_check(L, D * H)
    full = ops.affine(x, scale=scale, other=y, shift=shift)
    check_rows("affine", full, lambda r: ops.affine(sl(x, r), scale=scale, other=sl(y, r), shift=shift), picks)
    del full
    full = ops.layer_norm(*x, scale, shift)
    check_rows("layer norm", full, lambda r: ops.layer_norm(*sl(x, r), scale, shift), picks)
    del full
    full = ops.rowsum(*x)
    check_rows("row sum", full, lambda r: ops.rowsum(*sl(x, r)), picks)
    del full
    full = ops.multiply(x, y, 2.0, 0.01, 1)
    check_rows("product", full, lambda r: ops.multiply(sl(x, r), sl(y, r), 2.0, 0.01, 1), picks)


def test_softmax_rows():
    L, D, H = 66000, 128, 256
    say(f"large softmax [1, {L}, {D}, {H}]")
    x = big_object((1, L, D, H), (1, L, H), 28, gap_b=0.1)
    full = ops.softmax(*x, 2.0, 0.01, 2, return_sum_bound=True)
    for r in rows_to_check(L, D * H):
        part = ops.softmax(*sl(x, r), 2.0, 0.01, 2, return_sum_bound=True)
        for i, (f, q) in enumerate(zip(full, part)):
            same(f[:, r:r + 1], q, f"softmax row {r} output {i}", True)


def heads_to_check(n, head_elems):
    return rows_to_check(n, head_elems)


def test_dot_product_heads():
    B, L, D, d = 66, 128, 1024, 256
    say(f"large dot product [{B}, {L}, {D}, {d}]")
    x = big_object((B, L, D, d), (B, L, d), 19, gap_b=0.2)
    y = big_object((B, L, D, d), (B, L, d), 20, gap_b=0.2)
    full = ops.dot_product_qk(x, y, INF, 0.01, 1)
    for h in heads_to_check(B, L * D * d):
        part = ops.dot_product_qk(tuple(t[h:h + 1] for t in x), tuple(t[h:h + 1] for t in y), INF, 0.01, 1)
        for i, (f, q) in enumerate(zip(full, part)):
            same(f[h:h + 1], q, f"dot product head {h} output {i}", False)


def test_context_heads():
    B, L, D, d = 66, 128, 1024, 256
    say(f"large context [{B}, {L}, {D}, {L}] . [{B}, {L}, {D}, {d}]")
    probs = big_object((B, L, D, L), (B, L, L), 21, wstd=0.01, gap_w=0.001, gap_b=0.05)
    value = big_object((B, L, D, d), (B, L, d), 22, gap_b=0.2)
    full = ops.dot_product_v(probs, value, 2.0, 0.01, 1)
    for h in heads_to_check(B, L * D * d):
        part = ops.dot_product_v(tuple(t[h:h + 1] for t in probs), tuple(t[h:h + 1] for t in value), 2.0, 0.01, 1)
        for i, (f, q) in enumerate(zip(full, part)):
            same(f[h:h + 1], q, f"context head {h} output {i}", False)


def test_attention_in_place_heads():
    # heads side by side: [1, L, D, heads * size] -- a row of the object is 128 KB, a position 31 MB; 128 positions
    # of a tile still span less than 4 GB, so the MFMA kernel runs
    heads, L, D, size = 64, 270, 248, 512
    say(f"large attention scores, heads in place [1, {L}, {D}, {heads} x {size}]")
    q = big_object((1, L, D, heads * size), (1, L, heads * size), 23, gap_b=0.2)
    k = big_object((1, L, D, heads * size), (1, L, heads * size), 24, gap_b=0.2)
    full = ops.attention_scores(q, k, heads, 2.0, 0.01, 1)        # [heads, L, D, L]

    def fold(t, h):
        return t[..., h * size:(h + 1) * size].contiguous()
    for h in (0, heads // 2, heads - 1):
        part = ops.dot_product_qk(tuple(fold(t, h) for t in q), tuple(fold(t, h) for t in k), 2.0, 0.01, 1)
        for i, (f, p_) in enumerate(zip(full, part)):
            same(f[h:h + 1], p_, f"attention scores head {h} output {i}", False)


def test_context_in_place_heads():
    # value and context keep their heads side by side; three batch elements take the object past 2^31 elements
    # while one element's key positions still span less than 4 GB (the MFMA kernel's 32-bit offsets along K)
    B, heads, L, D, size = 3, 64, 128, 248, 512
    say(f"large attention context, heads in place [{B}, {L}, {D}, {heads} x {size}]")
    probs = big_object((B * heads, L, D, L), (B * heads, L, L), 26, wstd=0.01, gap_w=0.001, gap_b=0.05)
    value = big_object((B, L, D, heads * size), (B, L, heads * size), 27, gap_b=0.2)
    full = ops.attention_context(probs, value, 2.0, 0.01, 1)      # [B, L, D, heads * size]
    for b, h in ((0, 0), (1, heads - 1), (2, 0), (2, heads - 1)):
        t = b * heads + h
        v = tuple(x[b:b + 1, ..., h * size:(h + 1) * size].contiguous() for x in value)
        part = ops.dot_product_v(tuple(x[t:t + 1] for x in probs), v, 2.0, 0.01, 1)
        for i, (f, q) in enumerate(zip(full, part)):
            same(f[b:b + 1, ..., h * size:(h + 1) * size], q, f"attention context batch {b} head {h} output {i}", False)


def test_convolution_slices():
    D, C, HW, CO = 2304, 64, 128, 16
    say(f"large convolution [1, {D}, {C}, {HW}, {HW}] -> {CO} channels")
    g = torch.Generator(device="cuda").manual_seed(25)
    lw = torch.empty((1, D, C, HW, HW), device="cuda").normal_(0, 0.05, generator=g)
    uw = torch.empty((1, D, C, HW, HW), device="cuda").normal_(0, 0.005, generator=g).abs_().add_(lw)
    lb = torch.empty((1, C, HW, HW), device="cuda").normal_(0, 1, generator=g)
    ub = torch.empty((1, C, HW, HW), device="cuda").normal_(0, 0.1, generator=g).abs_().add_(lb)
    W = torch.empty((CO, C, 3, 3), device="cuda").normal_(0, (2 / (9 * C)) ** 0.5, generator=g)
    bias = torch.empty((CO,), device="cuda").normal_(0, 0.01, generator=g)
    olw, olb, ouw, oub = ops.conv2d(lw, lb, uw, ub, W, bias, 1, 1)
    for r in rows_to_check(D, C * HW * HW):
        plw, plb, puw, pub = ops.conv2d(lw[:, r:r + 1], lb, uw[:, r:r + 1], ub, W, bias, 1, 1)
        same(olw[:, r:r + 1], plw, f"convolution slice {r} lw", False)
        same(ouw[:, r:r + 1], puw, f"convolution slice {r} uw", False)
        same(olb, plb, "convolution lb", False)
        same(oub, pub, "convolution ub", False)


def test_convolution_with_images_of_a_gigabyte():
    """One image of the result takes 1.06 GB here: past what the 3 x 3 kernel's 32-bit store offsets are allowed
    (2 GB with 132 channels to spare), so the general kernel runs.  Rows at the top, in the middle and at the
    bottom must equal the convolution of the matching crop of the input."""
    D, C, HW, CO = 2, 4, 1440, 128
    say(f"large convolution images [1, {D}, {C}, {HW}, {HW}] -> {CO} channels")
    g = torch.Generator(device="cuda").manual_seed(29)
    lw = torch.empty((1, D, C, HW, HW), device="cuda").normal_(0, 0.05, generator=g)
    uw = torch.empty((1, D, C, HW, HW), device="cuda").normal_(0, 0.005, generator=g).abs_().add_(lw)
    lb = torch.empty((1, C, HW, HW), device="cuda").normal_(0, 1, generator=g)
    ub = torch.empty((1, C, HW, HW), device="cuda").normal_(0, 0.1, generator=g).abs_().add_(lb)
    W = torch.empty((CO, C, 3, 3), device="cuda").normal_(0, (2 / (9 * C)) ** 0.5, generator=g)
    bias = torch.empty((CO,), device="cuda").normal_(0, 0.01, generator=g)
    olw, olb, ouw, oub = ops.conv2d(lw, lb, uw, ub, W, bias, 1, 1)
    assert olw.shape == (1, D, CO, HW, HW)
    for r0 in (0, HW // 2, HW - 24):
        # input rows r0 - 1 .. r0 + 24 (clipped to the image) give output rows r0 .. r0 + 23 exactly, once the rows
        # next to a cut that is not the image's edge are left out
        top, bottom = max(r0 - 1, 0), min(r0 + 25, HW)
        crop = lambda t: t[..., top:bottom, :].contiguous()
        plw, plb, puw, pub = ops.conv2d(crop(lw), crop(lb), crop(uw), crop(ub), W, bias, 1, 1)
        skip = r0 - top                                 # rows of the crop's result above output row r0
        for full, part, name in ((olw, plw, "lw"), (ouw, puw, "uw"), (olb, plb, "lb"), (oub, pub, "ub")):
            same(full[..., r0:r0 + 24, :], part[..., skip:skip + 24, :], f"convolution rows {r0}.. {name}", False)


def test_linear_with_four_million_outputs():
    """A row of the result is 16.8 MB: 128 rows of it pass what the MFMA kernel's 32-bit store offsets are
    allowed, so the any-shape kernel runs.  Column ranges must equal the layer restricted to those outputs."""
    L, D, K, N = 1, 16, 4, 4_200_000
    say(f"large linear outputs [1, {L}, {D}, {K}] x [{N}, {K}]")
    x = big_object((1, L, D, K), (1, L, K), 30)
    g = torch.Generator(device="cuda").manual_seed(31)
    W = torch.empty((N, K), device="cuda").normal_(0, 0.5, generator=g)
    bias = torch.empty((N,), device="cuda").normal_(0, 0.01, generator=g)
    full = ops.linear(*x, W, bias)
    for c0 in (0, N // 2, N - 1000):
        part = ops.linear(*x, W[c0:c0 + 1000].contiguous(), bias[c0:c0 + 1000].contiguous())
        for i, (f, q) in enumerate(zip(full, part)):
            same(f[..., c0:c0 + 1000], q, f"linear columns {c0}.. output {i}", False)


def test_attention_in_place_past_the_tile_limit():
    """128 positions of an object with its heads side by side would span more than 4 GB here (dim_in 2048, rows of
    4096), past the 32-bit offsets of the MFMA kernels: the any-shape kernel runs.  Heads must equal the stacked
    entry points on folded copies."""
    heads, L, D, size = 16, 8, 2048, 256
    say(f"attention in place past the tile limit [1, {L}, {D}, {heads} x {size}]")
    q = big_object((1, L, D, heads * size), (1, L, heads * size), 32, gap_b=0.2)
    k = big_object((1, L, D, heads * size), (1, L, heads * size), 33, gap_b=0.2)
    v = big_object((1, L, D, heads * size), (1, L, heads * size), 34, gap_b=0.2)

    def fold(t, h):
        return t[..., h * size:(h + 1) * size].contiguous()
    scores = ops.attention_scores(q, k, heads, 2.0, 0.01, 1)              # [heads, L, D, L]
    context = ops.attention_context(scores, v, 2.0, 0.01, 1)              # [1, L, D, heads * size]
    # the any-shape kernel sums in double, the MFMA kernels in fp32: the bar allows for the order of 256 cancelling terms
    for h in (0, heads - 1):
        part = ops.dot_product_qk(tuple(fold(t, h) for t in q), tuple(fold(t, h) for t in k), 2.0, 0.01, 1)
        for i, (f, p_) in enumerate(zip(scores, part)):
            same(f[h:h + 1], p_, f"scores head {h} output {i}", False, atol=1e-5)
        ctx = ops.dot_product_v(tuple(t[h:h + 1] for t in scores), tuple(fold(t, h) for t in v), 2.0, 0.01, 1)
        for i, (f, p_) in enumerate(zip(context, ctx)):
            same(f[..., h * size:(h + 1) * size], p_, f"context head {h} output {i}", False, atol=1e-5)
