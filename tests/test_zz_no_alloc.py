"""The allocation-free dot product (faith_dot_product_verification_QK_static, scratch in a device array
inside the library) against faith_dot_product_verification_QK with caller-owned scratch, both through
the C ABI: same kernels, same inputs, so the results must be identical bit for bit.  Two calls in a
row, the second smaller, so that what the first left in the shared array cannot leak into the second.
Collected last: a failure here must not hide the other tests under `pytest -x`."""
import ctypes

import pytest
import torch

from tests.helpers import rand_bounds

pytestmark = pytest.mark.gpu
INF = float("inf")


def _call_both(B, Lx, Ly, D, d, p, words, seed, transposed=False):
    """transposed: the reference adapters' layout (coefficients [B, L, d, D], result [B, Lx, Ly, D]) with x_u = NULL on
    the caller-scratch entry, which is what the static entry does inside."""
    from faith_amd import _lib, ops
    g = torch.Generator().manual_seed(seed)
    x = [t.cuda().contiguous() for t in rand_bounds(g, B, Lx, D, d, sw=0.2, sb=1.0).tensors()]
    y = [t.cuda().contiguous() for t in rand_bounds(g, B, Ly, D, d, sw=0.2, sb=1.0).tensors()]
    xlw, xlb, xuw, xub = x
    ylw, ylb, yuw, yub = y
    zshape = (B, Lx, Ly, D) if transposed else (B, Lx, D, Ly)
    if transposed:
        xlw, xuw, ylw, yuw = (t.transpose(2, 3).contiguous() for t in (xlw, xuw, ylw, yuw))
    new = lambda *s: torch.full(s, float("nan"), device="cuda")
    outs = []
    for static in (False, True):
        zlb, zub, zlw, zuw = new(B, Lx, Ly), new(B, Lx, Ly), new(*zshape), new(*zshape)
        P = lambda t: ctypes.c_void_p(t.data_ptr())
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        tail = (B, Lx, Ly, d, D, 0.05, ops.q_code(p), words, _lib.LAYOUT_TRANSPOSED if transposed else _lib.LAYOUT_NATURAL,
                stream)
        if static:
            # a first call so that whatever the runtime sets up once (module load, the symbol's address) is done, then
            # the call that is watched: neither torch's allocator nor the device's free memory may move -- the latter
            # is what a hipMalloc inside the library would change (torch's own counter cannot see one)
            args = (P(xlb), P(xub), P(ylb), P(yub), P(xlw), P(xuw), P(ylw), P(yuw), P(zlb), P(zub), P(zlw), P(zuw), *tail)
            _lib.call("faith_dot_product_verification_QK_static", *args)
            torch.cuda.synchronize()
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            _lib.call("faith_dot_product_verification_QK_static", *args)
            torch.cuda.synchronize()
            assert torch.cuda.memory_allocated() == before
            assert torch.cuda.mem_get_info()[0] == free_before, "device memory was allocated or freed inside the call"
        else:
            xl, xu, yl, yu = new(B, Lx, d), new(B, Lx, d), new(B, Ly, d), new(B, Ly, d)
            _lib.call("faith_dot_product_verification_QK", P(xl), P(yl), None if transposed else P(xu), P(yu), P(xlb), P(xub),
                      P(ylb), P(yub), P(xlw), P(xuw), P(ylw), P(yuw), P(zlb), P(zub), P(zlw), P(zuw), *tail)
        torch.cuda.synchronize()
        outs.append((zlw, zlb, zuw, zub))
    return outs


def test_static_scratch_dot_product_equals_the_caller_scratch_entry_twice_in_a_row():
    # first call: configuration-3-like (tiled kernel); second: smaller and ragged (short-sequence kernel), other norm
    for case in ((4, 128, 128, 32, 64, INF, 1, 11), (2, 24, 17, 8, 32, 2.0, 2, 12), (1, 5, 3, 1, 16, 2.0, 1, 13)):
        print(f"[case] static-scratch dot product B,Lx,Ly,D,d,p,words,seed={case}", flush=True)
        ref, got = _call_both(*case)
        for name, a, b in zip(("lw", "lb", "uw", "ub"), got, ref):
            assert not torch.isnan(a).any(), f"{name}: not fully written"
            assert torch.equal(a, b), f"{name} differs from the caller-scratch entry point at {case}"


def test_static_scratch_dot_product_in_the_reference_layout_equals_the_caller_scratch_entry():
    # FAITH_LAYOUT_TRANSPOSED: intervals through the transposed concretization (x_u == NULL), then the kernel with lanes
    # along dim_in; two calls, the second smaller
    for case in ((2, 32, 48, 64, 32, 2.0, 1, 21), (1, 7, 5, 24, 16, INF, 2, 22)):
        print(f"[case] static-scratch dot product, transposed layout, B,Lx,Ly,D,d,p,words,seed={case}", flush=True)
        ref, got = _call_both(*case, transposed=True)
        for name, a, b in zip(("lw", "lb", "uw", "ub"), got, ref):
            assert not torch.isnan(a).any(), f"{name}: not fully written"
            assert torch.equal(a, b), f"{name} differs from the caller-scratch entry point at {case}"


def test_static_scratch_dot_product_rejects_what_does_not_fit():
    from faith_amd import _lib
    z = torch.zeros(8, device="cuda")
    P = ctypes.c_void_p(z.data_ptr())
    with pytest.raises(_lib.FaithError, match="scratch"):
        _lib.call("faith_dot_product_verification_QK_static", *([P] * 12), 16, 512, 512, 64, 8, 0.1, 1, 1, 0, None)
