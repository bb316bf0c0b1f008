"""RMS norm: ``y = x / sqrt(mean(x^2) + eps) * w`` with 32-bit statistics
(``crates/mach-model/src/kernels.rs:63-80``), and the forms in which it is folded into the product that
reads it: the norm's factor is one number a row, so a product's kernel can apply it to its finished sums."""
from __future__ import annotations

from .base import Norm, PendingNorm, TensorDecl, require_kernel_sizes
from .registry import register_norm


@register_norm("rmsnorm")
class RMSNorm(Norm):
    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        require_kernel_sizes(rt, "rmsnorm", norm_width=spec.width)

    def tensor_decls(self):
        decls = [TensorDecl("weight", (self.spec.width,), "vector")]
        if getattr(self.spec, "scaled", False):
            decls.append(TensorDecl("scale", (self.spec.width,), "vector"))
        return decls

    def load(self, tensors):
        # A weight stored around zero is applied as ``offset + w``; a layer's scale per coordinate multiplies the normed
        # row as well.  Both are folded into the one vector that every form of the norm's kernel takes.
        w = tensors["weight"]
        if getattr(self.spec, "offset", 0.0):
            w = w + float(self.spec.offset)
        if getattr(self.spec, "scaled", False):
            w = w * tensors["scale"]
        self.weight = w.contiguous()

    def forward(self, stream, rows=None):
        """``rmsnorm(x) * weight`` of the stream with everything added (of its ``rows`` if given), in the
        element type; partial sums that are pending are added by the norm's own kernel."""
        stream.launch_deferred()
        h = stream.ops.rmsnorm(stream.x, self.weight, self.spec.eps, rows, False, stream.pending)
        if rows is None:
            stream.pending = None  # the kernel wrote the sum back
        return h

    def pending(self, stream):
        return PendingRMSNorm(self, stream)

    def add_normed(self, stream, a, w, bias=None) -> None:
        """``x += rmsnorm(a @ w.T (+ bias)) * weight``: the norm after a branch whose last step is a product.  The product
        leaves its sums in 32-bit, and one kernel adds them up, normalises the row and adds it to the stream."""
        stream.flush()
        if bias is None:
            stream.ops.norm_add(stream.x, stream.ops.linear_split(a, w), self.weight, self.spec.eps)
        else:
            stream.ops.norm_add_bias(stream.x, stream.ops.linear_split(a, w), bias, self.weight, self.spec.eps)

    def add_normed_mean(self, stream, branches, eps) -> None:
        """``x += rmsnorm((rmsnorm(a) * wa + rmsnorm(b) * wb) / 2) * weight`` for two branches side by side, given as
        ``branches = [((a, w_a), wa), ((b, w_b), wb)]`` with each branch the operands of its last product."""
        if len(branches) != 2:
            raise ValueError(f"{len(branches)} branches side by side under a norm: the kernel takes two")
        ((a, w_a), wa), ((b, w_b), wb) = branches
        if eps != self.spec.eps:
            raise ValueError(f"branches normed with eps {eps} under a norm with eps {self.spec.eps}")
        stream.flush()
        ops = stream.ops
        ops.pair_norm_add(stream.x, ops.linear_split(a, w_a), wa, ops.linear_split(b, w_b), wb, self.weight, self.spec.eps)

    def add_normed_tensor(self, stream, y) -> None:
        """``x += rmsnorm(y) * weight`` for a branch that computes its output by other means."""
        stream.flush()
        stream.ops.norm_add(stream.x, y.float().contiguous().unsqueeze(0), self.weight, self.spec.eps)


@register_norm("rmsnorm_scalar")
class ScalarRMSNorm(RMSNorm):
    """RMS norm whose weight is one number for all coordinates: ``y = x / sqrt(mean(x^2) + eps) * g``.  The number is
    spread over the width when it is loaded, so every kernel and every folded form of the norm with a weight per
    coordinate serves it."""

    def tensor_decls(self):
        return [TensorDecl("weight", (), "vector")]

    def load(self, tensors):
        self.weight = tensors["weight"].reshape(1).expand(self.spec.width).contiguous()


@register_norm("layernorm")
class LayerNorm(Norm):
    """``y = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * weight + bias`` with 32-bit statistics; the bias is
    optional in the checkpoint.  Pending sums of the stream are added by the norm's own kernel."""

    def __init__(self, spec, rt):
        super().__init__(spec, rt)
        require_kernel_sizes(rt, "layernorm", norm_width=spec.width)

    def tensor_decls(self):
        return [TensorDecl("weight", (self.spec.width,), "vector"), TensorDecl("bias", (self.spec.width,), "vector", optional=True)]

    def load(self, tensors):
        self.weight, self.bias = tensors["weight"], tensors.get("bias")

    def forward(self, stream, rows=None):
        stream.launch_deferred()
        h = stream.ops.layernorm(stream.x, self.weight, self.bias, self.spec.eps, rows, False, stream.pending)
        if rows is None:
            stream.pending = None  # the kernel wrote the sum back
        return h


class PendingRMSNorm(PendingNorm):
    """The RMS norm left to its reader's first product, folded into it where the kernels take the shape."""

    def linear_split(self, w):
        stream, ops, weight, eps = self.stream, self.stream.ops, self.norm.weight, self.norm.spec.eps
        stream.launch_deferred()
        T, K = stream.x.shape
        P = 0 if stream.pending is None else stream.pending.shape[0]
        if ops.norm_folds_into(T, w.shape[0], K, P):
            out, x_new = ops.linear_split_normed(stream.x, stream.pending, weight, eps, w)
            if x_new is not None:
                stream.x, stream.pending = x_new, None
            return out
        return ops.linear_split(self.tensor(), w)

    def linear_swiglu(self, w_gate_up, intermediate, activation="silu"):
        stream, ops, weight, eps = self.stream, self.stream.ops, self.norm.weight, self.norm.spec.eps
        if stream.deferred is not None and stream.pending is None:
            # a product that is still to be added: where the kernels can, it leaves what the norm needs beside its
            # sum, and the gated product applies the norm's factor to its own finished sums
            a, w = stream.deferred
            takes = getattr(ops, "prenorm_swiglu_takes", None)
            if takes is not None and takes(a.shape[0], w.shape[0], w.shape[1], w_gate_up.shape[0]):
                stream.deferred = None
                hn, row_ss = ops.linear_residual_prenorm(a, w, stream.x, weight)
                return ops.linear_swiglu_scaled(hn, row_ss, eps, w_gate_up, intermediate, activation)
        stream.launch_deferred()
        T, K = stream.x.shape
        P = 0 if stream.pending is None else stream.pending.shape[0]
        if ops.norm_folds_into(T, w_gate_up.shape[0], K, P):
            out, x_new = ops.linear_swiglu_normed(stream.x, stream.pending, weight, eps, w_gate_up, intermediate, activation)
            if x_new is not None:
                stream.x, stream.pending = x_new, None
            return out
        return ops.linear_swiglu(self.tensor(), w_gate_up, intermediate, activation)
