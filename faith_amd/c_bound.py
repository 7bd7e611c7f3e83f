"""Drop-in for the reference's pybind module (HandTunedKernels/kernel.cpp:297-304).

Same function names, argument order and in-place output convention as the
module the reference loads as ``c_bound`` (Bounds.py:14-26), so its
``Bounds.cuda_*`` adapters (Bounds.py:1201-1343) can call this module
unchanged.  As there, lw / uw arrive transposed ([.., dim_out, dim_in]) and
every output tensor is pre-allocated by the caller.

Two differences from the reference kernels, both towards the PyTorch
semantics they were meant to reproduce: the dual norm follows ``p`` (module
attribute, default 2; the CUDA kernels hard-wire q = 2) and ``words`` blocks
are honoured.
"""
from __future__ import annotations

import torch

from . import _lib, ops
from ._lib import LAYOUT_TRANSPOSED

p = 2.0        # perturbation norm used by the calls below
words = 1      # perturbed_words


def _s(t):
    return ops._stream(t)


def _act(entry, src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw, length, dim_in, dim_out, epsilon):
    for n, t in (("src_lb", src_lb), ("src_ub", src_ub), ("src_lw", src_lw), ("src_uw", src_uw),
                 ("out_lb", out_lb), ("out_ub", out_ub), ("out_lw", out_lw), ("out_uw", out_uw)):
        ops._check(n, t)
    if src_lw.numel() != length * dim_in * dim_out or src_lb.numel() != length * dim_out:
        raise ValueError("tensor sizes do not match length * dim_in * dim_out (batch must be 1)")
    with torch.cuda.device(src_lw.device):
        _lib.call(entry, src_lb.data_ptr(), src_ub.data_ptr(), src_lw.data_ptr(), src_uw.data_ptr(),
                  out_lb.data_ptr(), out_ub.data_ptr(), out_lw.data_ptr(), out_uw.data_ptr(), None, None,
                  length, dim_in, dim_out, float(epsilon), ops.q_code(p), words, LAYOUT_TRANSPOSED, _s(src_lw))


def c_relu_verification(src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw,
                        length, dim_in, dim_out, epsilon):
    """kernel.cpp:69-99."""
    _act("faith_relu_verification", src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw,
         length, dim_in, dim_out, epsilon)


def c_tanh_verification(src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw,
                        length, dim_in, dim_out, epsilon):
    """kernel.cpp:101-131."""
    _act("faith_tanh_verification", src_lb, src_ub, src_lw, src_uw, out_lb, out_ub, out_lw, out_uw,
         length, dim_in, dim_out, epsilon)


def _sizes(expected):
    """Every tensor must hold exactly the number of elements its role implies: the library only sees pointers, so a
    short tensor would be written (or read) past its end on the device."""
    for name, t, n in expected:
        if t.numel() != n:
            raise ValueError(f"{name} holds {t.numel()} elements, the call's sizes imply {n} "
                             f"(shape {tuple(t.shape)})")


def _dot(entry, x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw, z_lb, z_ub, z_lw, z_uw,
         batch_size, x_rows, x_width, y_rows, y_width, z_width, length_x, length_y, dim_out, dim_in, epsilon):
    """x_rows x x_width / y_rows x y_width: the neurons of the two operands per batch element (their constant terms
    and concrete intervals have that many elements, their coefficients dim_in times as many); the result has
    x_rows x z_width neurons."""
    B, D = int(batch_size), int(dim_in)
    if x_lw.dim() != 4 or y_lw.dim() != 4:
        raise ValueError("x_lw and y_lw must have four axes ([batch, rows, width, dim_in])")
    if x_lw.shape[0] != B or y_lw.shape[0] != B:
        raise ValueError(f"batch_size = {B}, but x_lw / y_lw have {x_lw.shape[0]} / {y_lw.shape[0]} batch elements")
    if min(B, x_rows, x_width, y_rows, y_width, z_width, D) < 1:
        raise ValueError("every extent must be at least 1")
    nx, ny, nz = B * x_rows * x_width, B * y_rows * y_width, B * x_rows * z_width
    _sizes([("x_lw", x_lw, nx * D), ("x_uw", x_uw, nx * D), ("y_lw", y_lw, ny * D), ("y_uw", y_uw, ny * D),
            ("x_lb", x_lb, nx), ("x_ub", x_ub, nx), ("x_l", x_l, nx), ("x_u", x_u, nx),
            ("y_lb", y_lb, ny), ("y_ub", y_ub, ny), ("y_l", y_l, ny), ("y_u", y_u, ny),
            ("z_lw", z_lw, nz * D), ("z_uw", z_uw, nz * D), ("z_lb", z_lb, nz), ("z_ub", z_ub, nz)])
    for n, t in (("x_l", x_l), ("y_l", y_l), ("x_u", x_u), ("y_u", y_u), ("x_lb", x_lb), ("x_ub", x_ub), ("y_lb", y_lb),
                 ("y_ub", y_ub), ("x_lw", x_lw), ("x_uw", x_uw), ("y_lw", y_lw), ("y_uw", y_uw), ("z_lb", z_lb),
                 ("z_ub", z_ub), ("z_lw", z_lw), ("z_uw", z_uw)):
        ops._check(n, t)
    with torch.cuda.device(x_lw.device):
        _lib.call(entry, x_l.data_ptr(), y_l.data_ptr(), x_u.data_ptr(), y_u.data_ptr(), x_lb.data_ptr(), x_ub.data_ptr(),
                  y_lb.data_ptr(), y_ub.data_ptr(), x_lw.data_ptr(), x_uw.data_ptr(), y_lw.data_ptr(), y_uw.data_ptr(),
                  z_lb.data_ptr(), z_ub.data_ptr(), z_lw.data_ptr(), z_uw.data_ptr(), B, length_x, length_y,
                  dim_out, D, float(epsilon), ops.q_code(p), int(words), _lib.LAYOUT_TRANSPOSED, _s(x_lw))


def c_dot_product_verification_QK(x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw,
                                  z_lb, z_ub, z_lw, z_uw, batch_size, length, dim_out, dim_in, epsilon):
    """kernel.cpp:133-186.  x_lw .. y_uw are [B, L, dim_out, dim_in]; z_lw, z_uw are [B, L, L, dim_in]: the
    library takes these tensors as they are (FAITH_LAYOUT_TRANSPOSED), nothing is copied.  x and y may differ
    in length (the lengths are read off the tensors; `length` is the reference's single argument)."""
    if x_lw.dim() != 4 or y_lw.dim() != 4:
        raise ValueError("x_lw and y_lw must be [batch, length, dim_out, dim_in]")
    Lx, Ly = x_lw.shape[1], y_lw.shape[1]
    _dot("faith_dot_product_verification_QK", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw,
         z_lb, z_ub, z_lw, z_uw, batch_size, Lx, dim_out, Ly, dim_out, Ly, Lx, Ly, dim_out, dim_in, epsilon)


def c_dot_product_verification_V(x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw,
                                 z_lb, z_ub, z_lw, z_uw, batch_size, length, dim_out, dim_in, epsilon):
    """kernel.cpp:188-241; adapter Bounds.py:1306-1343.  x_* is the probability object with lw transposed
    to [B, L, L, dim_in]; y_* is the TRANSPOSED value object (lb [B, dim_out, L], lw [B, dim_out, L, dim_in]);
    z_lw, z_uw are [B, L, dim_out, dim_in].  Taken as they are (FAITH_LAYOUT_TRANSPOSED), nothing is copied."""
    if x_lw.dim() != 4 or y_lw.dim() != 4:
        raise ValueError("x_lw must be [batch, length, keys, dim_in] and y_lw [batch, dim_out, keys, dim_in]")
    Lx, Lk = x_lw.shape[1], x_lw.shape[2]
    _dot("faith_dot_product_verification_V", x_l, y_l, x_u, y_u, x_lb, x_ub, y_lb, y_ub, x_lw, x_uw, y_lw, y_uw,
         z_lb, z_ub, z_lw, z_uw, batch_size, Lx, Lk, dim_out, Lk, dim_out, Lx, Lk, dim_out, dim_in, epsilon)


def c_matmul_verification(x_lb, x_ub, x_lw, x_uw, W, y_lb, y_ub, y_lw, y_uw,
                          batch_size, length, dim_in, dim_out, dim_y_out):
    """kernel.cpp:243-266 (commented out there; natural layout, no bias)."""
    rows = int(batch_size) * int(length)
    _sizes([("x_lw", x_lw, rows * dim_in * dim_out), ("x_uw", x_uw, rows * dim_in * dim_out),
            ("x_lb", x_lb, rows * dim_out), ("x_ub", x_ub, rows * dim_out), ("W", W, dim_y_out * dim_out),
            ("y_lw", y_lw, rows * dim_in * dim_y_out), ("y_uw", y_uw, rows * dim_in * dim_y_out),
            ("y_lb", y_lb, rows * dim_y_out), ("y_ub", y_ub, rows * dim_y_out)])
    for n, t in (("x_lb", x_lb), ("x_ub", x_ub), ("x_lw", x_lw), ("x_uw", x_uw), ("W", W),
                 ("y_lb", y_lb), ("y_ub", y_ub), ("y_lw", y_lw), ("y_uw", y_uw)):
        ops._check(n, t)
    with torch.cuda.device(x_lw.device):
        _lib.call("faith_matmul_verification", x_lb.data_ptr(), x_ub.data_ptr(), x_lw.data_ptr(), x_uw.data_ptr(),
                  W.data_ptr(), None, y_lb.data_ptr(), y_ub.data_ptr(), y_lw.data_ptr(), y_uw.data_ptr(),
                  batch_size, length, dim_in, dim_out, dim_y_out, _s(x_lw))


def c_convolution_verification(x_lb, x_ub, x_lw, x_uw, W, y_lb, y_ub, y_lw, y_uw,
                               batch_size, Height, Width, CIN, COUT, K, Stride, padding_size, dim_in):
    """kernel.cpp:268-295 (commented out there)."""
    ho, wo = (Height + 2 * padding_size - K) // Stride + 1, (Width + 2 * padding_size - K) // Stride + 1
    if min(ho, wo) < 1:
        raise ValueError("the kernel does not fit the padded image")
    xin, yout = int(batch_size) * CIN * Height * Width, int(batch_size) * COUT * ho * wo
    _sizes([("x_lw", x_lw, xin * dim_in), ("x_uw", x_uw, xin * dim_in), ("x_lb", x_lb, xin), ("x_ub", x_ub, xin),
            ("W", W, COUT * CIN * K * K), ("y_lw", y_lw, yout * dim_in), ("y_uw", y_uw, yout * dim_in),
            ("y_lb", y_lb, yout), ("y_ub", y_ub, yout)])
    for n, t in (("x_lb", x_lb), ("x_ub", x_ub), ("x_lw", x_lw), ("x_uw", x_uw), ("W", W),
                 ("y_lb", y_lb), ("y_ub", y_ub), ("y_lw", y_lw), ("y_uw", y_uw)):
        ops._check(n, t)
    with torch.cuda.device(x_lw.device):
        _lib.call("faith_convolution_verification", x_lb.data_ptr(), x_ub.data_ptr(), x_lw.data_ptr(),
                  x_uw.data_ptr(), W.data_ptr(), None, y_lb.data_ptr(), y_ub.data_ptr(), y_lw.data_ptr(),
                  y_uw.data_ptr(), batch_size, Height, Width, CIN, COUT, K, Stride, padding_size, dim_in, _s(x_lw))
