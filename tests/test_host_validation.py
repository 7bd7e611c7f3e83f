"""Argument checks that happen on the host, before anything reaches the device: a tensor of the wrong size or a
position outside the sentence must be a Python error, because the library only sees pointers and a kernel
that follows them past the end of an allocation faults the GPU.  No GPU is needed: the checks fire first."""
import pytest
import torch

from faith_amd import c_bound, forward


def _dot_tensors(B=2, Lx=3, Ly=5, K=4, D=6):
    f = lambda *s: torch.zeros(*s)
    return dict(x_l=f(B, Lx, K), y_l=f(B, Ly, K), x_u=f(B, Lx, K), y_u=f(B, Ly, K),
                x_lb=f(B, Lx, K), x_ub=f(B, Lx, K), y_lb=f(B, Ly, K), y_ub=f(B, Ly, K),
                x_lw=f(B, Lx, K, D), x_uw=f(B, Lx, K, D), y_lw=f(B, Ly, K, D), y_uw=f(B, Ly, K, D),
                z_lb=f(B, Lx, Ly), z_ub=f(B, Lx, Ly), z_lw=f(B, Lx, Ly, D), z_uw=f(B, Lx, Ly, D)), (B, Lx, K, D)


ORDER = ("x_l", "y_l", "x_u", "y_u", "x_lb", "x_ub", "y_lb", "y_ub", "x_lw", "x_uw", "y_lw", "y_uw",
         "z_lb", "z_ub", "z_lw", "z_uw")


@pytest.mark.parametrize("short", ["z_lw", "z_uw", "z_lb", "x_l", "y_u", "y_lw", "x_ub"])
def test_scores_shim_rejects_a_tensor_of_the_wrong_size(short):
    t, (B, Lx, K, D) = _dot_tensors()
    t[short] = t[short].reshape(-1)[:-1].clone()
    with pytest.raises(ValueError, match=short):
        c_bound.c_dot_product_verification_QK(*(t[n] for n in ORDER), B, Lx, K, D, 0.01)


def test_scores_shim_rejects_a_wrong_batch_size_and_a_wrong_rank():
    t, (B, Lx, K, D) = _dot_tensors()
    with pytest.raises(ValueError, match="batch_size"):
        c_bound.c_dot_product_verification_QK(*(t[n] for n in ORDER), B + 1, Lx, K, D, 0.01)
    t["x_lw"] = t["x_lw"].reshape(B * Lx, K, D)
    with pytest.raises(ValueError, match="x_lw"):
        c_bound.c_dot_product_verification_QK(*(t[n] for n in ORDER), B, Lx, K, D, 0.01)


def test_scores_shim_accepts_consistent_sizes_up_to_the_device_check():
    # consistent sizes pass the size checks; what stops the call is then the CPU tensor (there is no CPU path)
    t, (B, Lx, K, D) = _dot_tensors()
    with pytest.raises(ValueError, match="GPU"):
        c_bound.c_dot_product_verification_QK(*(t[n] for n in ORDER), B, Lx, K, D, 0.01)


def test_context_shim_rejects_a_short_result():
    B, Lx, Lk, K, D = 2, 3, 5, 4, 6
    f = lambda *s: torch.zeros(*s)
    t = dict(x_l=f(B, Lx, Lk), y_l=f(B, K, Lk), x_u=f(B, Lx, Lk), y_u=f(B, K, Lk),
             x_lb=f(B, Lx, Lk), x_ub=f(B, Lx, Lk), y_lb=f(B, K, Lk), y_ub=f(B, K, Lk),
             x_lw=f(B, Lx, Lk, D), x_uw=f(B, Lx, Lk, D), y_lw=f(B, K, Lk, D), y_uw=f(B, K, Lk, D),
             z_lb=f(B, Lx, K), z_ub=f(B, Lx, K), z_lw=f(B, Lx, K, D), z_uw=f(B, Lx, K, D))
    with pytest.raises(ValueError, match="GPU"):
        c_bound.c_dot_product_verification_V(*(t[n] for n in ORDER), B, Lx, K, D, 0.01)
    t["z_lw"] = f(B, Lx, K, D - 1)
    with pytest.raises(ValueError, match="z_lw"):
        c_bound.c_dot_product_verification_V(*(t[n] for n in ORDER), B, Lx, K, D, 0.01)


def test_matmul_and_convolution_shims_reject_wrong_sizes():
    f = lambda *s: torch.zeros(*s)
    B, L, D, H, N = 1, 2, 3, 4, 5
    a = [f(B, L, H), f(B, L, H), f(B, L, D, H), f(B, L, D, H), f(N, H), f(B, L, N), f(B, L, N), f(B, L, D, N), f(B, L, D, N)]
    with pytest.raises(ValueError, match="GPU"):
        c_bound.c_matmul_verification(*a, B, L, D, H, N)
    a[7] = f(B, L, D, N - 1)
    with pytest.raises(ValueError, match="y_lw"):
        c_bound.c_matmul_verification(*a, B, L, D, H, N)
    Hh, Ci, Co, K = 6, 2, 3, 3
    c = [f(1, Ci, Hh, Hh), f(1, Ci, Hh, Hh), f(1, D, Ci, Hh, Hh), f(1, D, Ci, Hh, Hh), f(Co, Ci, K, K),
         f(1, Co, Hh, Hh), f(1, Co, Hh, Hh), f(1, D, Co, Hh, Hh), f(1, D, Co, Hh, Hh)]
    with pytest.raises(ValueError, match="GPU"):
        c_bound.c_convolution_verification(*c, 1, Hh, Hh, Ci, Co, K, 1, 1, D)
    c[8] = f(1, D, Co, Hh, Hh - 1)
    with pytest.raises(ValueError, match="y_uw"):
        c_bound.c_convolution_verification(*c, 1, Hh, Hh, Ci, Co, K, 1, 1, D)


def _never(*a, **k):
    raise AssertionError("the bound object must not be built from bad positions")


@pytest.mark.parametrize("index, words, what", [(7, 1, "outside"), (-1, 1, "outside"), ([1, 1], 2, "distinct"),
                                                ([0, 9], 2, "outside"), ([1], 2, "2 perturbed words")])
def test_input_builder_checks_positions_on_the_host(index, words, what):
    emb = torch.zeros(1, 7, 4)
    with pytest.raises(ValueError, match=what):
        forward.bound_input(_never, emb, index, 0.01, words)


def test_batched_input_builder_checks_positions_and_radii_on_the_host():
    emb = torch.zeros(1, 7, 4)
    with pytest.raises(ValueError, match="outside"):
        forward.bound_inputs(_never, emb, [1, 7], [0.1, 0.1])
    with pytest.raises(ValueError, match="radii"):
        forward.bound_inputs(_never, emb, [1, 2], [0.1])
    with pytest.raises(ValueError, match="integer"):
        forward.bound_inputs(_never, emb, [1.5], [0.1])
