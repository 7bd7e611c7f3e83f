"""The layer driver's own launches -- input coefficients, recorded preconditions, verdict -- against the tensor
expressions of the reference's driver (VerifierForward.py:127-156, :311-314; Bounds.py:892, :1147) evaluated on the
CPU.  Integer / comparison work: bit-exact."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def expected_coefficients(batch, rows, words, dim, positions, scales):
    w = torch.zeros(batch, rows, dim * words, dim)
    for b in range(batch):
        for i in range(words):
            r = i if positions is None else int(positions[b, i])
            if 0 <= r < rows:
                w[b, r, dim * i:dim * (i + 1), :] = torch.eye(dim) * (1.0 if scales is None else float(scales[b]))
    return w


@pytest.mark.parametrize("batch,rows,words,dim,compact,scaled", [
    (1, 5, 1, 8, False, False),          # one query, zeros written out (vector stores)
    (1, 2, 2, 8, True, False),           # two perturbed words, rows of those words only
    (1, 6, 2, 6, False, False),          # dim not a multiple of four: scalar stores
    (3, 7, 1, 12, False, True),          # independent problems with their radii in the coefficients
    (4, 1, 1, 16, True, True),
    (2, 9, 3, 4, False, True),
    (1, 32, 1, 256, False, False),       # the encoder layer's size
])
def test_input_coefficients_are_the_identity_blocks_of_bound_input(batch, rows, words, dim, compact, scaled):
    from faith_amd import ops
    g = torch.Generator().manual_seed(batch * 100 + rows)
    positions = None if compact else torch.stack([torch.randperm(rows, generator=g)[:words] for _ in range(batch)])
    scales = torch.rand(batch, generator=g) + 0.1 if scaled else None
    w = ops.input_coefficients(batch, rows, words, dim, "cuda", None if compact else positions.cuda(),
                               None if scales is None else scales.cuda())
    # a buffer that held something else before is overwritten whole
    out = torch.full((batch, rows, dim * words, dim), 7.0, device="cuda")
    again = ops.input_coefficients(batch, rows, words, dim, "cuda", None if compact else positions.cuda(),
                                   None if scales is None else scales.cuda(), out=out)
    torch.cuda.synchronize()
    want = expected_coefficients(batch, rows, words, dim, positions, scales)
    assert again is out
    assert torch.equal(w.cpu(), want) and torch.equal(out.cpu(), want)


def test_input_coefficients_scalar_scale_and_a_position_outside_the_sentence():
    from faith_amd import ops
    positions = torch.tensor([[2], [9], [-1]])
    w = ops.input_coefficients(3, 4, 1, 8, "cuda", positions.cuda(), scale=0.25)
    torch.cuda.synchronize()
    want = torch.zeros(3, 4, 8, 8)
    want[0, 2] = 0.25 * torch.eye(8)
    assert torch.equal(w.cpu(), want)
    with pytest.raises(ValueError):
        ops.input_coefficients(1, 3, 1, 8, "cuda")                      # no positions: one row per word
    with pytest.raises(ValueError):
        ops.input_coefficients(1, 3, 1, 8, "cuda", torch.zeros(1, 1).cuda())   # positions are int64
    with pytest.raises(ValueError, match="no CPU path"):
        ops.input_coefficients(1, 1, 1, 8, "cpu")


def test_flag_below_records_the_preconditions_per_batch_element():
    from faith_amd import ops
    g = torch.Generator().manual_seed(5)
    l = torch.rand(6, 3, 50, generator=g) + 0.5
    l[1, 2, 7] = 0.0                      # reaches zero: fails `> 0`, passes `>= 0`
    l[2, 0, 0] = -1e-3                    # below: fails both
    l[4, 1, 49] = float("nan")            # fails both, as it fails the reference's assert
    l[5, 2, 49] = 1e-12                   # exactly the reciprocal's bound: passes `>=`
    for bound, strict, want in ((0.0, True, [0, 1, 1, 0, 1, 0]), (0.0, False, [0, 0, 1, 0, 1, 0]),
                                (1e-12, False, [0, 1, 1, 0, 1, 0]), (1e-12, True, [0, 1, 1, 0, 1, 1])):
        flags = torch.zeros(6, dtype=torch.bool, device="cuda")
        ops.flag_below(l.cuda(), flags, bound, strict)
        torch.cuda.synchronize()
        assert flags.cpu().tolist() == [bool(v) for v in want], (bound, strict)
    # flags are only ever set
    flags = torch.tensor([True, False, False, False, False, False], device="cuda")
    ops.flag_below(l.cuda(), flags, 0.0, True)
    assert flags.cpu().tolist() == [True, True, True, False, True, False]
    # more values per batch element than one round of the grid takes
    big = torch.ones(2, 3_000_000)
    big[1, 2_999_999] = -1.0
    flags = torch.zeros(2, dtype=torch.bool, device="cuda")
    ops.flag_below(big.cuda(), flags, 0.0, True)
    assert flags.cpu().tolist() == [False, True]
    with pytest.raises(ValueError):
        ops.flag_below(l.cuda(), torch.zeros(6, device="cuda"), 0.0, True)      # flags are bytes


@pytest.mark.parametrize("host", [False, True])
def test_verdict_is_the_comparison_of_bound_classifier(host):
    from faith_amd import ops
    l = torch.tensor([0.5, -0.1, 0.0, 2.0, float("nan"), 1.0]).reshape(6, 1, 1)
    u = torch.tensor([0.7, 0.3, 0.1, -0.5, -1.0, -0.0]).reshape(6, 1, 1)
    flags = torch.tensor([False, False, False, True, False, False])
    for label in (0, 1):
        ok = (l[:, 0, 0] > 0) if label == 0 else (u[:, 0, 0] < 0)
        for f in (None, flags):
            got = ops.verdict(l.cuda(), u.cuda(), None if f is None else f.cuda(), label, host=host)
            if not host:
                assert got.dtype == torch.bool
                got = got.cpu().tolist()
            assert got == (ok if f is None else ok & ~f).tolist(), (label, f is None)
    # wider rows: the first value of each batch element decides
    l3 = torch.randn(4, 1, 3)
    got = ops.verdict(l3.cuda(), l3.cuda(), None, 0, host=host)
    assert (got if host else got.cpu().tolist()) == (l3[:, 0, 0] > 0).tolist()
