"""`Bounds`: the reference's operator surface for forward bound propagation, on HIP.

Mirrors the constructor and the method names / return conventions of the
reference class (Transformer_Verification_Code/Verifiers/Bounds.py:270-297) for
the methods on the accelerated path:

    concretize   Bounds.py:319-326        relu        :1163-1169 (ori_relu :921-963)
    matmul       :1177-1199 (ori_matmul :397-413)     tanh        :1171-1175 (ori_tanh :1027-1103)
    dense        :1016-1025               dot_product :833-841 (ori_dot_product :710-823)
    t / context  :335-346, :843-850       exp / sqr / sqrt / reciprocal  :970-1003, :860-919, :1136-1161
    multiply / divide / softmax / layer_norm  :594-664, :825-830, :1005-1014, :1111-1131
    add          :383-395                 conv2d      HandTunedKernels/convolution_verification.cu:219-239

Every method launches hand-written HIP kernels through the C ABI; none has a
PyTorch fallback.  Known defects of the reference are not reproduced: `dense`
is `matmul(weight).add(bias)` (the reference line raises NameError), and the
dot product uses the true upper constant term (the reference's CUDA adapter
overwrites ub with lb, Bounds.py:1286).
"""
from __future__ import annotations

from types import SimpleNamespace

import torch

from . import _lib, ops


def _written_out(x):
    """An operand that may be a `CompactBounds`: its dense form."""
    return x.dense_form() if isinstance(x, CompactBounds) else x


class Bounds:
    def __init__(self, args, p, eps, w=None, b=None, lw=None, lb=None, uw=None, ub=None, clone=True):
        self.args = args if args is not None else SimpleNamespace(perturbed_words=1)
        self.p = p
        self.eps = eps
        self.perturbed_words = getattr(self.args, "perturbed_words", 1)
        # interval bound propagation (args.method == "ibp", Bounds.py:274): zero coefficients, every
        # relaxation maps the concrete interval to the interval of its image
        self.ibp = getattr(self.args, "method", None) == "ibp"
        self.lw = lw if lw is not None else (w.clone() if clone else w)
        self.uw = uw if uw is not None else (w.clone() if clone else w)
        self.lb = lb if lb is not None else (b.clone() if clone else b)
        self.ub = ub if ub is not None else (b.clone() if clone else b)
        if self.ibp:                                        # Bounds.py:285-288
            self.lw, self.uw = self.lw[:, :, :self.perturbed_words, :], self.uw[:, :, :self.perturbed_words, :]
        self.device = self.lw.device
        self.update_shape()

    def update_shape(self):
        self.batch_size, self.length, self.dim_in, self.dim_out = self.lw.shape[:4]

    def _like(self, lw, lb, uw, ub):
        return Bounds(self.args, self.p, self.eps, lw=lw, lb=lb, uw=uw, ub=ub)

    def _c(self):
        return (self.lw.contiguous(), self.lb.contiguous(), self.uw.contiguous(), self.ub.contiguous())

    def first_position(self):
        """The bounds of position 0 alone, [B, 1, ...] (what VerifierForward._bound_pooling, :269-287, slices out).
        One batch element: views.  Several: the rows are strided, so they are gathered -- a launch per pair of
        tensors instead of a strided copy per tensor."""
        if self.batch_size == 1:
            return self._like(self.lw[:, :1], self.lb[:, :1], self.uw[:, :1], self.ub[:, :1])
        lw, lb, uw, ub = self._c()
        B, L, D, H = lw.shape
        at = ops.positions_tensor([[0]] * B, lw.device)
        flw, fuw = ops.gather_positions(lw.view(B, L, D * H), uw.view(B, L, D * H), at)
        flb, fub = ops.gather_positions(lb, ub, at)
        return self._like(flw.view(B, 1, D, H), flb, fuw.view(B, 1, D, H), fub)

    def _interval(self, kind):
        """method "ibp": the operator applied to the concrete interval; coefficients are zero
        (the `if self.ibp` branches of Bounds.py:863-866, :896-898, :924-926, :973-975, :1030-1032, :1139-1143)."""
        l, u = self.concretize()
        if kind == "sqrt":
            self._require(l, 0.0, True, "sqrt of a bound that reaches zero")
        if kind == "reciprocal":
            self._require(l, 1e-12, False, "reciprocal of a bound that reaches zero")
        lb, ub = ops.interval_unary(kind, l, u)
        return self._like(torch.zeros_like(self.lw), lb, torch.zeros_like(self.uw), ub)

    # ---- Bounds.py:319-326
    def concretize(self):
        lw, lb, uw, ub = self._c()
        return ops.concretize(lw, lb, uw, ub, self.p, self.eps, self.perturbed_words)

    # ---- Bounds.py:311-317: -/+ eps * ||w||_q over the whole of dim_in (no perturbed-word blocks)
    def concretize_l(self, lw=None):
        lw = (self.lw if lw is None else lw).contiguous()
        zero = torch.zeros(lw.shape[:2] + lw.shape[3:], device=lw.device)
        return ops.concretize(lw, zero, lw, zero, self.p, self.eps, 1)[0]

    def concretize_u(self, uw=None):
        uw = (self.uw if uw is None else uw).contiguous()
        zero = torch.zeros(uw.shape[:2] + uw.shape[3:], device=uw.device)
        return ops.concretize(uw, zero, uw, zero, self.p, self.eps, 1)[1]

    # ---- Bounds.py:328-333
    def clone(self):
        return self._like(self.lw.clone(), self.lb.clone(), self.uw.clone(), self.ub.clone())

    # ---- Bounds.py:299-309
    def print(self, message):
        print(message)
        l, u = self.concretize()
        print("mean abs %.5f %.5f" % (l.abs().mean(), u.abs().mean()))
        print("diff %.5f %.5f %.5f" % ((u - l).min(), (u - l).max(), (u - l).mean()))
        print("min", l.min())
        print("max", u.max())
        print()

    # ---- Bounds.py:383-395
    def add(self, delta):
        delta = _written_out(delta)
        if isinstance(delta, Bounds):
            return self._like(*ops.add(self._c(), delta._c()))
        return self._like(*ops.shift(*self._c(), delta))

    # ---- Bounds.py:594-664: by a float, by a per-neuron tensor, or by another bound object
    def multiply(self, W):
        W = _written_out(W)
        if isinstance(W, Bounds):
            if self.ibp:                                    # Bounds.py:667-676: the interval of the product
                (xl, xu), (yl, yu) = self.concretize(), W.concretize()
                lb, ub = ops.interval_product(xl, xu, yl, yu)
                return self._like(torch.zeros_like(self.lw), lb, torch.zeros_like(self.uw), ub)
            return self._like(*ops.multiply(self._c(), W._c(), self.p, self.eps, self.perturbed_words))
        return self._like(*ops.scale(*self._c(), W))

    # ---- Bounds.py:825-830
    def divide(self, W):
        W = _written_out(W)
        if not isinstance(W, Bounds):
            raise NotImplementedError
        return self.multiply(W.reciprocal())

    # ---- Bounds.py:1005-1014
    def softmax(self, scale=None):
        """scale (beyond the reference's signature): `self.multiply(scale).softmax()` for a positive float --
        the 1 / sqrt(head size) of the attention scores (VerifierForward.py:232-240) -- in the same launch."""
        if scale is not None and not (isinstance(scale, (int, float)) and scale > 0):
            return self.multiply(scale).softmax()
        if not self.ibp and ops.softmax_fits(self.dim_in, self.dim_out):
            # the four operators below on a slab that stays in registers: one launch, one read, one write
            try:
                out = ops.softmax(*self._c(), self.p, self.eps, self.perturbed_words, return_sum_bound=True,
                                  scale=1.0 if scale is None else scale)
            except _lib.FaithError as err:
                if err.code != _lib.ERR_UNSUPPORTED:         # e.g. tensors that are not 16-byte aligned
                    raise
            else:
                self._require(out[4], 1e-12, False, "reciprocal of a bound that reaches zero")
                return self._like(*out[:4])
        e = (self if scale is None else self.multiply(scale)).exp()
        return e.divide(self._like(*ops.rowsum(*e._c())))

    # ---- Bounds.py:1111-1131
    def layer_norm(self, normalizer, layer_norm, residual=None):
        """residual (beyond the reference's signature): a bound object added first, i.e.
        `self.add(residual).layer_norm(...)` (VerifierForward.py:166, 181-189) without the pass of the sum
        through memory; same values."""
        if layer_norm == "no":
            return self if residual is None else self.add(residual)
        weight, bias = normalizer.weight.detach().contiguous(), normalizer.bias.detach().contiguous()
        other = None if residual is None else residual._c()
        if layer_norm == "no_var":
            # (residual sum,) mean subtraction, weight and bias in one launch
            return self._like(*ops.layer_norm(*self._c(), weight, bias, other))
        assert layer_norm == "standard"
        minus_mu = self._like(*ops.layer_norm(*self._c(), other=other))
        # the variance: matmul with the H x H matrix of 1 / H (Bounds.py:1116, :1123) is a row mean
        variance = minus_mu._like(*ops.rowmean(*minus_mu.sqr()._c()))
        normalized = minus_mu.divide(variance.add(1e-12).sqrt())
        return normalized._like(*ops.affine(normalized._c(), scale=weight, shift=bias))

    # ---- Bounds.py:397-413, :1177-1199
    def matmul(self, W, bias=None):
        if isinstance(W, (Bounds, CompactBounds)):
            raise NotImplementedError("matmul with a Bounds operand is dot_product")
        lw, lb, uw, ub = self._c()
        if W.dim() == 3:
            # one weight per position (Bounds.py:414-428: W [length, H_out, H], a single batch element): the layer
            # kernel on each position's rows, which are contiguous in both objects
            if bias is not None or lw.shape[0] != 1 or W.shape[0] != lw.shape[1] or W.shape[2] != lw.shape[3]:
                raise ValueError(f"a per-position weight must be [length={lw.shape[1]}, H_out, {lw.shape[3]}] for one batch "
                                 f"element and come without a bias, got {tuple(W.shape)} for lw {tuple(lw.shape)}")
            W = W.contiguous()
            L, N = W.shape[0], W.shape[1]
            out = (lw.new_empty(1, L, lw.shape[2], N), lb.new_empty(1, L, N), lw.new_empty(1, L, lw.shape[2], N),
                   lb.new_empty(1, L, N))
            for i in range(L):
                ops.linear(lw[:, i:i + 1], lb[:, i:i + 1], uw[:, i:i + 1], ub[:, i:i + 1], W[i], None,
                           out=tuple(t[:, i:i + 1] for t in out))
            return self._like(*out)
        if W.dim() != 2:
            raise NotImplementedError("a weight is [H_out, H] or, per position, [length, H_out, H]")
        return self._like(*ops.linear(lw, lb, uw, ub, W.contiguous(), bias))

    # ---- Bounds.py:1016-1025 (bias fused into the same launch)
    def dense(self, dense):
        bias = getattr(dense, "bias", None)
        return self.matmul(dense.weight.detach(), None if bias is None else bias.detach().contiguous())

    def dense_act(self, dense, act_name):
        """`self.dense(dense).act(act_name)` (VerifierForward.py:171-179).  ReLU with a dim_in the kernel takes and
        enough positions to fill the device: one pass over the coefficients, in which the layer's result does not
        reach memory; otherwise the separate operators."""
        W = dense.weight.detach().contiguous()
        if (act_name == "relu" and not self.ibp and W.dim() == 2
                and ops.linear_relu_fits(self.lb.shape[0] * self.lb.shape[1], self.dim_in, W.shape[1], W.shape[0],
                                         self.perturbed_words) == 2):
            bias = getattr(dense, "bias", None)
            bias = None if bias is None else bias.detach().contiguous()
            try:
                return self._like(*ops.linear_relu(*self._c(), W, bias, self.p, self.eps, self.perturbed_words))
            except _lib.FaithError as err:
                if err.code != _lib.ERR_UNSUPPORTED:         # e.g. tensors that are not 16-byte aligned
                    raise
        return self.dense(dense).act(act_name)

    def dense_layer_norm(self, dense, normalizer, layer_norm, residual=None):
        """`self.dense(dense).add(residual).layer_norm(normalizer, layer_norm)` (VerifierForward.py:166, 181-189).
        Mode "no_var" with a hidden size the kernel takes: one pass over the coefficients, in which neither the
        layer's result nor the sum reaches memory (a residual that is a CompactBounds is read from the rows it
        holds); otherwise the separate operators."""
        W = dense.weight.detach().contiguous()
        words = residual._lw.shape[1] if isinstance(residual, CompactBounds) else 0
        if (layer_norm == "no_var" and not self.ibp and W.dim() == 2
                and ops.linear_layer_norm_fits(self.lb.shape[0] * self.lb.shape[1], self.dim_in, W.shape[1], W.shape[0],
                                               words) == 2):
            bias = getattr(dense, "bias", None)
            bias = None if bias is None else bias.detach().contiguous()
            weight, shift = normalizer.weight.detach().contiguous(), normalizer.bias.detach().contiguous()
            other = positions = None
            if isinstance(residual, CompactBounds):
                other = (residual._lw.contiguous(), residual._lb.contiguous(), residual._uw.contiguous(),
                         residual._ub.contiguous())
                positions = residual.positions
            elif residual is not None:
                other = residual._c()
            try:
                return self._like(*ops.linear_layer_norm(*self._c(), W, bias, weight, shift, other, positions))
            except _lib.FaithError as err:
                if err.code != _lib.ERR_UNSUPPORTED:         # e.g. tensors that are not 16-byte aligned
                    raise
        return self.dense(dense).layer_norm(normalizer, layer_norm, residual=residual)

    def dense_concretize(self, dense):
        """(self.dense(dense), its concrete interval) through one entry point -- one launch for small problems such
        as the classifier, whose result is concretized at once (VerifierForward.py:300-314).  Returns (bounds, l, u)."""
        bias = getattr(dense, "bias", None)
        out = ops.linear_concretize(*self._c(), dense.weight.detach().contiguous(),
                                    None if bias is None else bias.detach().contiguous(),
                                    self.p, self.eps, self.perturbed_words)
        return self._like(*out[:4]), out[4], out[5]

    def dense_group(self, layers):
        """[self.dense(layer) for layer in layers] for up to three layers of one shape, in one launch where that
        pays (beyond the reference's surface: its `_bound_attention` calls dense three times,
        VerifierForward.py:202-204)."""
        layers = list(layers)
        shapes = {tuple(layer.weight.shape) for layer in layers}
        if len(layers) > 3 or len(shapes) != 1:
            return [self.dense(layer) for layer in layers]
        weights = [layer.weight.detach().contiguous() for layer in layers]
        biases = [None if getattr(layer, "bias", None) is None else layer.bias.detach().contiguous() for layer in layers]
        return [self._like(*out) for out in ops.linear_group(*self._c(), weights, biases)]

    # ---- Bounds.py:1163-1175
    def relu(self):
        if self.ibp:
            return self._interval("relu")
        return self._like(*ops.relu(*self._c(), self.p, self.eps, self.perturbed_words))

    def tanh(self):
        if self.ibp:
            return self._interval("tanh")
        return self._like(*ops.tanh(*self._c(), self.p, self.eps, self.perturbed_words))

    # ---- Bounds.py:970-1003, :860-890
    def exp(self):
        if self.ibp:
            return self._interval("exp")
        return self._like(*ops.exp(*self._c(), self.p, self.eps, self.perturbed_words))

    def sqr(self):
        if self.ibp:
            return self._interval("sqr")
        return self._like(*ops.sqr(*self._c(), self.p, self.eps, self.perturbed_words))

    # ---- Bounds.py:892-919, :1136-1161.  Both assert a positive interval in the reference; the
    # check reads the concrete lower bound back from the kernel (one synchronisation).
    def sqrt(self):
        if self.ibp:
            return self._interval("sqrt")
        out = ops.sqrt(*self._c(), self.p, self.eps, self.perturbed_words, return_interval=True)
        self._require(out[4], 0.0, True, "sqrt of a bound that reaches zero")
        return self._like(*out[:4])

    def reciprocal(self):
        if self.ibp:
            return self._interval("reciprocal")
        out = ops.reciprocal(*self._c(), self.p, self.eps, self.perturbed_words, return_interval=True)
        self._require(out[4], 1e-12, False, "reciprocal of a bound that reaches zero")
        return self._like(*out[:4])

    # The reference asserts these preconditions (Bounds.py:894, :1147), which costs a device
    # synchronisation per call and fails a whole batch for one element.  Inside collect_failures the
    # violation is recorded per batch element on the device instead and nothing waits.
    _collector = None

    @classmethod
    def _require(cls, l, bound, strict, message):
        c = cls._collector
        if c is None:
            low = float(l.min())
            assert (low > bound) if strict else (low >= bound), message
            return
        ops.flag_below(l.contiguous(), c.mask, bound, strict)           # leading axis is batch-major; one launch

    @staticmethod
    def verdict(l, u, flags, label, host=False):
        """Safe or not per batch element (VerifierForward.py:311-314) in one launch: see ops.verdict."""
        return ops.verdict(l.contiguous(), u.contiguous(), flags, label, host)

    class collect_failures:
        """with Bounds.collect_failures(batch, device) as f: ... ; f.mask[b] is True where a
        precondition failed for batch element b (its results are then meaningless)."""

        def __init__(self, batch, device):
            self.mask = torch.zeros(batch, dtype=torch.bool, device=device)

        def __enter__(self):
            assert Bounds._collector is None, "collect_failures does not nest"
            Bounds._collector = self
            return self

        def __exit__(self, *exc):
            Bounds._collector = None
            return False

    def act(self, act_name):
        if act_name == "relu":
            return self.relu()
        if act_name == "tanh":
            return self.tanh()
        raise NotImplementedError(act_name)

    # ---- Bounds.py:335-346.  The transposed object is a pair of views that remembers where it came
    # from, so that dot_product can read the original layout instead of materialising it.
    def t(self):
        r = self._like(self.lw.transpose(1, 3), self.lb.transpose(1, 2),
                       self.uw.transpose(1, 3), self.ub.transpose(1, 2))
        r._transpose_of = self
        return r

    # ---- Bounds.py:833-841.  Scores path: self = query, other = key.  Context path: other is the
    # transposed value object (the reference tells the two apart by the shape of self.lb; here the
    # transposed object says so itself).
    def dot_product(self, other, debug=False, verbose=False, lower=True, upper=True):
        # (the reference's extra arguments are accepted; both halves are always computed)
        src = getattr(other, "_transpose_of", None)
        if self.ibp and self.dim_in > 1:
            # interval arithmetic on the constant terms (get_bounds_xy's ibp branch makes every
            # coefficient zero, Bounds.py:667-676): the dim_in == 1 kernel on one row of the zero
            # coefficients, its zero result repeated dim_in times
            if src is not None:
                return self._ibp_rows(lambda x, v: x.dot_product(v.t()), src)
            return self._ibp_rows(lambda x, y: x.dot_product(y), other)
        if src is not None:
            return self._like(*ops.dot_product_v(self._c(), src._c(), self.p, self.eps, self.perturbed_words))
        return self._like(*ops.dot_product_qk(self._c(), other._c(), self.p, self.eps, self.perturbed_words))

    # ---- Bounds.py:843-850
    def context(self, value):
        return self.dot_product(value.t())

    # ---- VerifierForward.py:208-229 + Bounds.py:833-841: scores of all heads, self = query and key
    # both [1, L, D, heads * size]; the kernels address each head in place
    def attention_scores(self, key, heads):
        if self.ibp and self.dim_in > 1:
            return self._ibp_rows(lambda q, k: q.attention_scores(k, heads), key)
        return self._like(*ops.attention_scores(self._c(), key._c(), heads, self.p, self.eps, self.perturbed_words))

    def _ibp_rows(self, op, other):
        """method "ibp" with dim_in > 1: the interval kernels run on one row of the (zero) coefficients
        and the zero result is repeated dim_in times."""
        one = lambda b: b._like(b.lw[:, :, :1], b.lb, b.uw[:, :, :1], b.ub)
        z = op(one(self), one(other))
        zero = z.lw.expand(-1, -1, self.dim_in, -1).contiguous()
        return self._like(zero, z.lb, zero.clone(), z.ub)

    # ---- VerifierForward.py:208-229 + Bounds.py:843-850 + VerifierForward.py:253-263: self = probabilities
    # [heads, Lx, D, Lk], value [1, Lk, D, heads * size] -> [1, Lx, D, heads * size]
    def attention_context(self, value):
        if self.ibp and self.dim_in > 1:
            return self._ibp_rows(lambda pr, v: pr.attention_context(v), value)
        if isinstance(value, CompactBounds):
            out = value._context_of(self)
            if out is not None:
                return out
        return self._like(*ops.attention_context(self._c(), value._c(), self.p, self.eps, self.perturbed_words))


# The reference keeps three spellings of its hot methods -- the dispatcher (relu), the PyTorch body
# (ori_relu) and the CUDA adapter (cuda_relu), chosen by a module-level FLAG (Bounds.py:1163-1175,
# :833-841, :397-401).  Here there is one implementation, so the other spellings are the same method.
for _name, _target in (("ori_relu", "relu"), ("cuda_relu", "relu"), ("ori_tanh", "tanh"), ("cuda_tanh", "tanh"),
                       ("ori_matmul", "matmul"), ("ori_dot_product", "dot_product"),
                       ("cuda_dot_product_QK", "dot_product"), ("cuda_dot_product_V", "dot_product")):
    setattr(Bounds, _name, getattr(Bounds, _target))


class CompactBounds:
    """A bound object whose coefficients vanish outside a few positions, stored without the zeros.

    The input object of a verification query has identity coefficients at the perturbed position(s) and
    zero coefficients at every other one (VerifierForward.py:127-156), and stays that way through the
    embedding layer norm and the first dense layers, which treat positions independently; the attention
    scores are the first operator that mixes positions.  Held here:

        positions  int64 [B, P]     the positions of batch element b that have coefficients (distinct)
        lw, uw     [B, P, D, H]     the coefficients at those positions      (as _lw, _uw)
        lb, ub     [B, L, H]        the constant terms at every position     (as _lb, _ub)

    `layer_norm` and `matmul` / `dense` / `dense_group` keep the form: they run their kernels on the P rows
    that are not zero (the affine ones also on the constants, as an object with one zero coefficient row per
    position); `attention_scores` of two compact objects -- the first operator that mixes positions -- takes
    the kernel that writes the dense scores from the compact rows, and `probs.attention_context(value)` with a
    compact value the context kernel that reads its rows; every other attribute or method is that of
    `dense_form()`, the equal `Bounds` object with the zeros written out (built on first use).  Beyond the
    reference's surface, which carries the zeros through every operator.

    `positions` lives on the device and is not inspected here (that would wait for the GPU): whoever builds it
    must keep every entry inside 0 ... length-1 and the entries of a batch element distinct, as the input builders
    of faith_amd.forward do on the host before they create it.  The compact kernels skip a row whose position lies
    outside that range; `dense_form`, `concrete_intervals` and everything that goes through them index with it."""

    collect_failures = Bounds.collect_failures
    verdict = Bounds.verdict

    def __init__(self, args, p, eps, positions, lw, lb, uw, ub):
        self.args, self.p, self.eps = args, p, eps
        self.positions = positions
        self._lw, self._lb, self._uw, self._ub = lw, lb, uw, ub
        B, P = positions.shape
        if lw.shape[:2] != (B, P) or uw.shape != lw.shape or lb.shape != (B, lb.shape[1], lw.shape[3]) \
                or ub.shape != lb.shape:
            raise ValueError(f"positions {tuple(positions.shape)}, lw {tuple(lw.shape)}, uw {tuple(uw.shape)}, "
                             f"lb {tuple(lb.shape)}, ub {tuple(ub.shape)} do not describe one compact object")
        self.length = lb.shape[1]
        self.device = lw.device
        self.perturbed_words = getattr(args, "perturbed_words", 1)
        self._dense = None
        self._intervals = None

    def _compact_like(self, lw, lb, uw, ub):
        return CompactBounds(self.args, self.p, self.eps, self.positions, lw, lb, uw, ub)

    def dense_form(self):
        """The same object as `Bounds`, zeros written out (built once)."""
        if self._dense is None:
            lw = ops.spread_positions(self._lw, self.positions, self.length)
            uw = lw if self._uw is self._lw else ops.spread_positions(self._uw, self.positions, self.length)
            self._dense = Bounds(self.args, self.p, self.eps, lw=lw, lb=self._lb, uw=uw, ub=self._ub)
        return self._dense

    def __getattr__(self, name):            # whatever is not defined here
        if name.startswith("__") or name in ("_lw", "_lb", "_uw", "_ub", "_dense", "_intervals"):
            raise AttributeError(name)
        return getattr(self.dense_form(), name)

    # ---- Bounds.py:1111-1131: rows are independent, so the rows that are zero stay out of the launch
    def layer_norm(self, normalizer, layer_norm, residual=None):
        if layer_norm == "no" and residual is None:
            return self
        if layer_norm != "no_var" or residual is not None:
            return self.dense_form().layer_norm(normalizer, layer_norm, residual=residual)
        weight, bias = normalizer.weight.detach().contiguous(), normalizer.bias.detach().contiguous()
        c = (self._lw.contiguous(), self._lb.contiguous(), self._uw.contiguous(), self._ub.contiguous())
        return self._compact_like(*ops.layer_norm(*c, weight, bias))

    # ---- Bounds.py:397-413, :1016-1025
    def _affine(self, weights, biases):
        """The affine kernels on the P coefficient rows per batch element and the L constant rows: the entry points
        that count the two separately."""
        c = (self._lw.contiguous(), self._lb.contiguous(), self._uw.contiguous(), self._ub.contiguous())
        return [self._compact_like(*out) for out in ops.linear_rows(*c, weights, biases)]

    def matmul(self, W, bias=None):
        if isinstance(W, (Bounds, CompactBounds)) or W.dim() != 2:
            return self.dense_form().matmul(W, bias)
        return self._affine([W.contiguous()], [bias])[0]

    def dense(self, dense):
        bias = getattr(dense, "bias", None)
        return self.matmul(dense.weight.detach(), None if bias is None else bias.detach().contiguous())

    def dense_group(self, layers):
        layers = list(layers)
        if len(layers) > 3 or len({tuple(layer.weight.shape) for layer in layers}) != 1:
            return [self.dense(layer) for layer in layers]
        weights = [layer.weight.detach().contiguous() for layer in layers]
        biases = [None if getattr(layer, "bias", None) is None else layer.bias.detach().contiguous() for layer in layers]
        return self._affine(weights, biases)

    def dense_layer_norm(self, dense, normalizer, layer_norm, residual=None):
        return self.dense(dense).layer_norm(normalizer, layer_norm, residual=residual)

    def dense_act(self, dense, act_name):
        return self.dense(dense).act(act_name)

    # ---- Bounds.py:319-326 on the rows that have coefficients; the constants are the bounds of the others
    def concrete_intervals(self):
        """(l, u) [B, L, H], as concretize() of the dense form gives them (computed once)."""
        if self._intervals is None:
            self._intervals = ops.concretize_positions(self._lw.contiguous(), self._lb.contiguous(), self._uw.contiguous(),
                                                       self._ub.contiguous(), self.positions, self.p, self.eps,
                                                       self.perturbed_words)
        return self._intervals

    # ---- VerifierForward.py:208-229 + Bounds.py:833-841 for two objects with coefficients at the same positions
    def attention_scores(self, key, heads):
        B, P, D, H = self._lw.shape
        if (isinstance(key, CompactBounds) and key.positions is self.positions and key._lw.shape == self._lw.shape
                and key._lb.shape == self._lb.shape and H % heads == 0
                and ops.attention_scores_compact_fits(self.length, P, H // heads, D)):
            x = (self._lw.contiguous(), self._lb.contiguous(), self._uw.contiguous(), self._ub.contiguous())
            y = (key._lw.contiguous(), key._lb.contiguous(), key._uw.contiguous(), key._ub.contiguous())
            x_l, _ = self.concrete_intervals()
            y_l, y_u = key.concrete_intervals()
            try:
                out = ops.attention_scores_compact(x, y, x_l, y_l, y_u, self.positions, heads)
            except _lib.FaithError as err:
                if err.code != _lib.ERR_UNSUPPORTED:         # e.g. tensors that are not 16-byte aligned
                    raise
            else:
                return Bounds(self.args, self.p, self.eps, lw=out[0], lb=out[1], uw=out[2], ub=out[3])
        return self.dense_form().attention_scores(_written_out(key), heads)

    # ---- VerifierForward.py:208-229 + Bounds.py:843-850 + VerifierForward.py:253-263 with this object as the value
    def _context_of(self, probs):
        """probs.attention_context(self) from the rows that exist, or None where the kernel does not take the shapes
        (the caller then writes the zeros out)."""
        B, P, D, H = self._lw.shape
        heads = probs.lw.shape[0] // B if probs.lw.shape[0] % B == 0 else 0
        if (self._dense is not None or heads == 0 or H % heads or probs.dim_in != D or probs.dim_out != self.length
                or not ops.attention_context_compact_fits(self.length, H // heads, D)):
            return None
        y = (self._lw.contiguous(), self._lb.contiguous(), self._uw.contiguous(), self._ub.contiguous())
        y_l, y_u = self.concrete_intervals()
        try:
            out = ops.attention_context_compact(probs._c(), y, y_l, y_u, self.positions, probs.p, probs.eps,
                                                probs.perturbed_words)
        except _lib.FaithError as err:
            if err.code != _lib.ERR_UNSUPPORTED:
                raise
            return None
        return probs._like(*out)


class BoundsMaker:
    """`make_bounds` for faith_amd.forward: maker(p, eps, lw, lb, uw, ub) builds a `Bounds`, and
    maker.compact(p, eps, positions, lw, lb, uw, ub) a `CompactBounds`, which the input builders of
    faith_amd.forward use when the maker has it and its compact_pays() says so.

    compact_from: size in bytes of one coefficient tensor with the zeros written out from which the compact
    form is kept; a smaller object is written out at once.  A propagation that small is bound by its ~30
    launches, of which the compact form needs a few more: with hidden size 256 and 32 positions the two break
    even near 3 queries per propagation (32 MiB is 4), and at 30 the compact form saves 31 % of the time.
    Replayed from a captured graph the launches cost the device's time only and the compact form is never
    slower (one query 345 against 368 us, two 481 against 577, four 703 against 699): there it is always kept."""

    def __init__(self, args=None, compact_from=32 << 20):
        self.args = args
        self.compact_from = compact_from

    def __call__(self, p, eps, lw, lb, uw, ub):
        return Bounds(self.args, p, eps, lw=lw, lb=lb, uw=uw, ub=ub)

    def compact_pays(self, batch, length, dim_in, dim_out, captured=False):
        """Asked by the input builders before they build either form; captured: for replays from a graph."""
        ibp = getattr(self.args, "method", None) == "ibp"       # keeps no coefficients: nothing to leave out
        return not ibp and (captured or 4 * batch * length * dim_in * dim_out >= self.compact_from)

    def compact(self, p, eps, positions, lw, lb, uw, ub):
        return CompactBounds(self.args, p, eps, positions, lw, lb, uw, ub)

    # the input builders' device work, one launch each
    @staticmethod
    def positions_tensor(groups, device):
        return ops.positions_tensor(groups, device)

    @staticmethod
    def input_coefficients(batch, rows, words, dim, device, positions=None, scales=None, out=None):
        return ops.input_coefficients(batch, rows, words, dim, device, positions, scales, out=out)


class ConvBounds:
    """Bounds of an image-shaped activation: lw, uw [1, D_in, C, H, W]; lb, ub [1, C, H, W]."""

    def __init__(self, p, eps, lw, lb, uw, ub):
        self.p, self.eps = p, eps
        self.lw, self.lb, self.uw, self.ub = lw, lb, uw, ub

    def conv2d(self, weight, bias=None, stride=1, padding=0):
        out = ops.conv2d(self.lw.contiguous(), self.lb.contiguous(), self.uw.contiguous(), self.ub.contiguous(),
                         weight.contiguous(), bias, stride, padding)
        return ConvBounds(self.p, self.eps, *out)

    def concretize(self):
        return ops.concretize_conv(self.lw.contiguous(), self.lb.contiguous(), self.uw.contiguous(),
                                   self.ub.contiguous(), self.p, self.eps)
